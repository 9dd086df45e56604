"""Rotary position encoding with half-split pairs (reference layers/rotary_embedding.py:5-25)."""
from __future__ import annotations

import math

import torch

from .base import PositionEncoding, register_part


@register_part("position_encoding", "rotary")
class RotaryEmbedding(PositionEncoding):
    """angle[p, i] = p * theta^(-2i/D); the pair (x_i, x_{i+D/2}) is rotated by angle[p, i].

    One instance is shared by all layers that use it (reference models/qwen3.py:81). The
    angles, their cos/sin and the rotation are float32 (the reference rounds cos/sin to the
    activations' dtype, layers/rotary_embedding.py:21-22). The table is [P, D/2, 2] with
    (cos, sin) adjacent, the form the fused query/key kernel reads.
    """

    def __init__(self, head_dim: int, theta: float, rotary_dims: int | None = None, interleaved: bool = False,
                 stored_dim: int | None = None, exact_angles: bool = False, scaling: dict | None = None):
        """`rotary_dims`: only the first so many of a head's `stored_dim` dimensions turn, with angles
        p * theta^(-2i/rotary_dims); the others pass unchanged (None: all `head_dim` turn). `interleaved`: the
        stored pairs are (x_2i, x_2i+1) instead of (x_i, x_i+rotary_dims/2). Either way the kernels see the
        half-split form over `head_dim` slots (which may exceed `stored_dim`: slots that hold nothing): a mixer
        lays its query and key heads out by `head_order()`, which puts the two members of pair i into slots i and
        head_dim/2 + i, the dimensions that do not turn into the slots left, whose table entries are (cos, sin)
        = (1, 0). A dot product does not care about the order of the dimensions as long as q and k share it.

        `scaling` stretches the positions a model was made for. {"kind": "linear", "factor": s}: every rate is divided
        by s. {"kind": "yarn", "factor": s, "original": L, "fast": b, "slow": a}: with where(t) = dims * ln(L / (2 pi t)) /
        (2 ln theta), lo = max(floor(where(b)), 0), hi = min(ceil(where(a)), dims - 1) and ramp_i = clamp((i - lo) /
        max(hi - lo, 0.001), 0, 1), pair i turns at rate_i / s * ramp_i + rate_i * (1 - ramp_i) (pairs that turn fast keep
        their rate, slow ones are stretched), and cos and sin are both multiplied by 0.1 ln(s) + 1."""
        super().__init__()
        if head_dim % 2:
            raise ValueError("rotary encoding needs an even head size")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.stored_dim = head_dim if stored_dim is None else int(stored_dim)
        self.rotary_dims = self.stored_dim if rotary_dims is None else int(rotary_dims)
        self.interleaved = bool(interleaved)
        self.exact_angles = bool(exact_angles)     # angles, cos and sin formed in float64 and rounded once to float32
        self.scaling = dict(scaling) if scaling else None
        if self.scaling is not None:
            kind = self.scaling.get("kind")
            need = {"linear": ("factor",), "yarn": ("factor", "original", "fast", "slow")}.get(kind)
            if need is None or any(k not in self.scaling for k in need) or not float(self.scaling["factor"]) > 0:
                raise ValueError(f"rotary scaling {self.scaling!r}: kind 'linear' (factor) or 'yarn' (factor, original, fast, slow)")
            self.exact_angles = True               # scaled rates are formed in float64
        if self.rotary_dims % 2 or not 0 <= self.rotary_dims <= self.stored_dim <= head_dim:
            raise ValueError(f"{self.rotary_dims} rotating dimensions of {self.stored_dim} stored in {head_dim} slots")
        self.table = None

    def head_order(self) -> list | None:
        """Which stored dimension of a head each of the `head_dim` slots holds (-1: none, the slot is zero); None
        when the stored order is the kernels' order already."""
        D, n, r = self.head_dim, self.stored_dim, self.rotary_dims
        if n == D and r == D and not self.interleaved:
            return None
        if self.interleaved:
            low, high = [2 * i for i in range(r // 2)], [2 * i + 1 for i in range(r // 2)]
        else:
            low, high = list(range(r // 2)), list(range(r // 2, r))
        rest = list(range(r, n))
        room = D // 2 - r // 2
        low, high = low + rest[:room], high + rest[room:]
        return low + [-1] * (D // 2 - len(low)) + high + [-1] * (D // 2 - len(high))

    def rates(self) -> tuple:
        """(float64 rates of the turning pairs, the factor on cos and sin)."""
        turning = self.rotary_dims
        i = torch.arange(0, turning, 2, dtype=torch.float64)
        rate = self.theta ** (-i / max(turning, 1))
        sc = self.scaling
        if sc is None:
            return rate, 1.0
        s = float(sc["factor"])
        if sc["kind"] == "linear":
            return rate / s, 1.0
        where = lambda turns: turning * math.log(float(sc["original"]) / (2.0 * math.pi * float(turns))) / (2.0 * math.log(self.theta))
        lo = max(math.floor(where(sc["fast"])), 0)
        hi = min(math.ceil(where(sc["slow"])), turning - 1)
        ramp = ((i / 2 - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        return rate / s * ramp + rate * (1.0 - ramp), 0.1 * math.log(s) + 1.0

    def finalize(self, device, dtype, max_positions):
        if self.table is not None and self.table.shape[0] >= max_positions and self.table.device == torch.device(device):
            return
        half = self.head_dim // 2
        # same expression as the reference: 1 / theta^(2i/D), float32 throughout
        turning = self.rotary_dims
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, turning, 2, dtype=torch.float32) / max(turning, 1)))
        t = torch.arange(max_positions, dtype=torch.float32)
        ang = torch.zeros((max_positions, half), dtype=torch.float32)
        ang[:, :turning // 2] = torch.outer(t, inv_freq)    # [P, D/2]; angle 0 where nothing turns
        if self.exact_angles:
            ang = ang.double()
            rate, mult = self.rates()
            ang[:, :turning // 2] = torch.outer(torch.arange(max_positions, dtype=torch.float64), rate)
            if mult != 1.0:
                if self.rotary_dims != 2 * half:
                    raise ValueError("a factor on cos and sin needs a rotation of all slots (the others' entries are (1, 0))")
                self.table = (torch.stack((ang.cos(), ang.sin()), dim=-1) * mult).float().contiguous().to(device)
                return
        self.table = torch.stack((ang.cos(), ang.sin()), dim=-1).float().contiguous().to(device)
        assert self.table.shape == (max_positions, half, 2)

    def rotary_table(self):
        return self.table

    def apply(self, q, k, positions):
        """Unfused form for mixers that do not use the fused kernel. q: [T, Hq, D], k: [T, Hkv, D]."""
        cs = self.table[positions.long()]                   # [T, D/2, 2]
        c, s = cs[..., 0].unsqueeze(1), cs[..., 1].unsqueeze(1)
        half = self.head_dim // 2
        for x in (q, k):
            x1, x2 = x[..., :half].float(), x[..., half:].float()
            lo, hi = x1 * c - x2 * s, x2 * c + x1 * s      # both halves before either is overwritten
            x[..., :half] = lo.to(x.dtype)
            x[..., half:] = hi.to(x.dtype)
