"""Two token mixers side by side, and two recurrences whose state rows decay each at a rate of their own.

`SideBySide` hands one input to a left and a right mixer and returns left_scale * left + right_scale * right; what
the two need from the engine (pages of keys and values, a state row) is the sum of their needs, so any mixer with
pages may stand beside any mixer with state. `ShiftedDecay` and `GatedDelta` both run on one recurrence kernel
(`ops.decay_rows_recurrence`): per head a float32 matrix S [key channels, value channels] in the request's state
slot, every key channel with a decay that the token chooses. They differ in the update rule and in what surrounds it.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, StateNeed, few_tokens, register_part, side_branch
from .linear import Linear


class ScaledTerms:
    """What `SideBySide.forward` returns where its consumer can form the sum itself: terms of (rows or float32 partial
    sums, scale, bias or None) whose weighted sum is the mixer's output (`ops.weighted_sum`)."""

    def __init__(self, terms: list):
        self.terms = list(terms)

    def value(self) -> torch.Tensor:
        return ops.weighted_sum(self.terms)


@register_part("mixer", "side_by_side")
class SideBySide(Mixer):
    """left_scale * left(x) + right_scale * right(x). At most one of the two keeps pages and at most one keeps state.
    With `side_stream`, in steps of few tokens the right mixer runs on a second stream beside the left one
    (`base.side_branch`)."""

    side_stream = True
    returns_terms = True       # forward(..., terms=True) hands the two outputs on unadded

    def __init__(self, left: Mixer, right: Mixer, left_scale: float = 1.0, right_scale: float = 1.0):
        super().__init__()
        self.add_child("left", left)
        self.add_child("right", right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        needs = [m.cache_need() for m in (left, right)]
        states = [m.state_need() for m in (left, right)]
        if all(n is not None for n in needs) or all(s is not None for s in states):
            raise ValueError("of two mixers side by side one may keep pages and one may keep state")
        self._cache_of = 0 if needs[0] is not None else (1 if needs[1] is not None else None)
        self._state_of = 0 if states[0] is not None else (1 if states[1] is not None else None)
        self.capturable = getattr(left, "capturable", True) and getattr(right, "capturable", True)
        left.defer_bias = right.defer_bias = True         # an output bias joins the weighted sum's kernel (`Biased`)

    def cache_need(self):
        return None if self._cache_of is None else (self.left, self.right)[self._cache_of].cache_need()

    def state_need(self):
        return None if self._state_of is None else (self.left, self.right)[self._state_of].state_need()

    def forward(self, x, step, cache, state, terms: bool = False):
        """`terms`: return the two outputs unadded (`ScaledTerms`) for a consumer that forms the weighted sum itself."""
        give = lambda i: (cache if self._cache_of == i else None, state if self._state_of == i else None)
        if self.side_stream and few_tokens(x):
            with side_branch(x.device, 1) as branch:
                b = self.right.forward(x, step, *give(1))
            a = self.left.forward(x, step, *give(0))
            branch.join()
        else:
            a = self.left.forward(x, step, *give(0))
            b = self.right.forward(x, step, *give(1))
        out = ScaledTerms([_term(a, self.left_scale), _term(b, self.right_scale)])
        return out if terms else out.value()


class Biased:
    """A mixer's output whose bias is still to be added: (rows or float32 partial sums, float32 bias [n]). A mixer returns
    one only to a caller that asked for it (`defer_bias`); `SideBySide` does, and adds the bias inside its weighted sum."""

    def __init__(self, rows: torch.Tensor, bias: torch.Tensor):
        self.rows, self.bias = rows, bias


def _term(y, scale: float) -> tuple:
    return (y.rows, scale, y.bias) if isinstance(y, Biased) else (y, scale, None)


def _decay_base(shape, generator, device):
    """Biases of the decay's exponent spread over -6..-1: per-step decays between 0.998 and 0.69."""
    return -6.0 + 5.0 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device)


def _half(shape, generator, device):
    return torch.rand(shape, generator=generator, dtype=torch.float32, device=device)


def _decay_bias(shape, generator, device):
    """Biases of a sigmoid decay spread over 1..5: per-step decays between 0.73 and 0.993 before the temperature."""
    return 1.0 + 4.0 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device)


def _bonus(shape, generator, device):
    return torch.rand(shape, generator=generator, dtype=torch.float32, device=device) - 0.5


@register_part("mixer", "shifted_decay")
class ShiftedDecay(Mixer):
    """With x' the previous token's input (zeros before the first token), each of r, k, v, g, w reads its own mix
    x + (x' - x) * mu_s. r, k, v = W_r, W_k, W_v of their mixes ([heads, key_dim] each), gate = silu(W_g mix_g), and the
    decay of every key channel d = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0)). Per head, with a bonus u for the current token,
        y_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,      S_t = diag(d_t) S_(t-1) + k_t v_t^T.
    Every head's y is divided by its root mean square; the heads side by side are multiplied by a weight and the gate and
    projected. A request's state row holds the heads' matrices and, behind them, the previous token's input."""

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, decay_rank: int, norm_eps: float):
        super().__init__()
        self.hidden_size, self.num_heads, self.key_dim, self.decay_rank = hidden_size, num_heads, key_dim, decay_rank
        self.norm_eps = float(norm_eps)
        self.inner = num_heads * key_dim
        self.add_param("mu", ParamSpec((len(self.MIXES) * hidden_size,), init=_half, dtype="float32"))      # one row per mix, flat
        for name in ("r", "k", "v", "g"):
            self.add_child(name, Linear(hidden_size, self.inner))
        self.add_child("w1", Linear(hidden_size, decay_rank))
        self.add_child("w2", Linear(decay_rank, self.inner))
        self.add_param("w0", ParamSpec((self.inner,), init=_decay_base, dtype="float32"))
        self.add_param("u", ParamSpec((num_heads, key_dim), init=_bonus, dtype="float32"))
        self.add_param("norm_weight", ParamSpec((self.inner,), init="norm", dtype="float32"))
        self.add_child("o", Linear(self.inner, hidden_size))
        self.value_dim = key_dim
        self.matrix_floats = num_heads * key_dim * key_dim

    def state_need(self):
        return StateNeed((self.matrix_floats + self.hidden_size,), "float32")

    def forward(self, x, step, cache, state):
        H, N = self.num_heads, self.key_dim
        mixes = ops.token_shift(x, self.mu.view(len(self.MIXES), self.hidden_size), state[:, self.matrix_floats:], step.state_slots, step.cu_seqlens, step.seq_of_token)
        r, k, v, g = (getattr(self, name).forward(mixes[i]) for i, name in enumerate(("r", "k", "v", "g")))
        raw = self.w2.forward(ops.activation(self.w1.forward(mixes[4]), "tanh"))
        y = ops.decay_rows_recurrence(r, k, v, raw, state[:, : self.matrix_floats], step.state_slots, step.cu_seqlens, step.q_lens,
                                      H, H, N, N, "bonus", base=self.w0, bonus=self.u.reshape(-1))
        o = ops.gated_rms_norm(y, g, self.norm_weight, self.norm_eps, H, "silu_behind", g.dtype)
        return self.o.forward(o, allow_partials=True)


def _log_rates(shape, generator, device):
    return torch.log(1.0 + 15.0 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device))


def _step_bias(shape, generator, device):
    """Biases whose softplus lies between 0.001 and 0.1."""
    dt = torch.exp(torch.rand(shape, generator=generator, dtype=torch.float32, device=device)
                   * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
    return dt + torch.log(-torch.expm1(-dt))


def _taps(shape, generator, device):
    return (torch.rand(shape, generator=generator, dtype=torch.float32, device=device) - 0.5) * (2.0 / math.sqrt(shape[1]))


@register_part("mixer", "gated_delta")
class GatedDelta(Mixer):
    """q, k ([key_heads, key_dim]) and v ([heads, value_dim]) from one packed product, each through a short causal
    convolution per channel (no bias; the last tap is the current token's) and silu; q and k are made unit vectors per
    head, x / sqrt(sum(x^2) + unit_eps), and q is multiplied by key_dim^(-1/2). A write strength per head, beta =
    sigmoid(W_b x), and a decay per head and key channel, d = exp(-exp(A_log_h) softplus(W_a2 (W_a1 x) + dt_bias)). Per
    head (heads share q and k by groups):
        S <- diag(d) S;   u = beta (v - S^T k);   S <- S + k u^T;   y = S^T q.
    Every head's y is divided by its root mean square, multiplied by a weight shared by the heads and by
    sigmoid(W_g2 (W_g1 x)), and projected. A request's state row holds the heads' matrices and, behind them, the
    convolutions' last taps - 1 inputs per channel."""

    def __init__(self, hidden_size: int, num_heads: int, key_heads: int, key_dim: int, value_dim: int, taps: int,
                 decay_rank: int, gate_rank: int, norm_eps: float, unit_eps: float = 1e-6):
        super().__init__()
        if num_heads % key_heads or taps < 1:
            raise ValueError("heads must be a multiple of the key heads, taps positive")
        self.hidden_size, self.num_heads, self.key_heads = hidden_size, num_heads, key_heads
        self.key_dim, self.value_dim, self.taps = key_dim, value_dim, taps
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        self.qk, self.inner, self.decays = key_heads * key_dim, num_heads * value_dim, num_heads * key_dim
        self.channels = 2 * self.qk + self.inner
        # one product for everything that reads x directly: q | k | v | beta | a1 | g1
        self.add_child("in_proj", Linear(hidden_size, self.channels + num_heads + decay_rank + gate_rank,
                                         parts={"q": self.qk, "k": self.qk, "v": self.inner, "b": num_heads, "a1": decay_rank, "g1": gate_rank}))
        self.decay_rank, self.gate_rank = decay_rank, gate_rank
        self.add_param("conv_weight", ParamSpec((self.channels, taps), init=_taps, dtype="float32"))
        self.add_child("a2", Linear(decay_rank, self.decays))
        self.add_child("g2", Linear(gate_rank, self.inner))
        self.add_param("dt_bias", ParamSpec((self.decays,), init=_step_bias, dtype="float32"))
        self.add_param("A_log", ParamSpec((num_heads,), init=_log_rates, dtype="float32"))
        self.add_param("norm_weight", ParamSpec((value_dim,), init="norm", dtype="float32"))
        self.add_child("o", Linear(self.inner, hidden_size))
        self.matrix_floats = num_heads * key_dim * value_dim
        self.rate = self.wide_norm = None

    def state_need(self):
        return StateNeed((self.matrix_floats + self.channels * (self.taps - 1),), "float32")

    def finalize(self, device, dtype, max_positions):
        self.rate = torch.exp(self.A_log.float()).contiguous()
        self.wide_norm = self.norm_weight.float().repeat(self.num_heads).contiguous()
        w = self.in_proj.weight
        if w.shape[0] % 8:                  # the packed rows in whole steps of 8: views of them keep 16-byte row strides
            self.in_proj.weight = torch.cat((w, w.new_zeros(8 - w.shape[0] % 8, w.shape[1])), 0).contiguous()

    def forward(self, x, step, cache, state):
        H, G, N, P = self.num_heads, self.key_heads, self.key_dim, self.value_dim
        rows = self.in_proj.forward(x)                                # [T, q | k | v | b | a1 | g1 (| padding)]
        C = self.channels
        qkv = ops.causal_conv(rows[:, :C], self.conv_weight, None, state[:, self.matrix_floats:], step.state_slots,
                              step.cu_seqlens, step.q_lens)
        at = C + H
        raw = self.a2.forward(_rows(rows, at, self.decay_rank))
        gate = self.g2.forward(_rows(rows, at + self.decay_rank, self.gate_rank))
        y = ops.decay_rows_recurrence(qkv[:, : self.qk], qkv[:, self.qk: 2 * self.qk], qkv[:, 2 * self.qk:], raw,
                                      state[:, : self.matrix_floats], step.state_slots, step.cu_seqlens, step.q_lens, H, G, N, P,
                                      "delta", base=self.dt_bias, rate=self.rate, beta=rows[:, C: C + H],
                                      unit_eps=self.unit_eps, q_scale=N ** -0.5)
        o = ops.gated_rms_norm(y, gate, self.wide_norm, self.norm_eps, H, "sigmoid_behind", gate.dtype)
        return self.o.forward(o, allow_partials=True)


def _rows(rows: torch.Tensor, start: int, width: int) -> torch.Tensor:
    """Columns [start, start + width) of packed rows as an operand of a product: a view where the products take one
    (their rows start at whole steps of 16 bytes), else a copy."""
    view = rows[:, start:start + width]
    if (start * rows.element_size()) % 16 == 0 and (rows.stride(0) * rows.element_size()) % 16 == 0:
        return view
    return view.contiguous()


@register_part("mixer", "gla")
class GatedLinearAttention(Mixer):
    """Linear attention whose state rows decay each at a rate the token chooses, without a bonus and without a shift:
    q = W_q x * key_dim^(-1/2), k = W_k x ([heads, key_dim]), v = W_v x ([heads, value_dim]); the decay of every key
    channel alpha = sigmoid(W_a2 (W_a1 x) + bias) ^ (1 / tau) (a thin matrix pair). Per head
        S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t.
    Every head's o is divided by its root mean square and multiplied by a weight of the value size that the heads share;
    the heads side by side are multiplied by silu(W_g x) and projected. q, k, v, the gate and the pair's first matrix are
    one packed product. The decay and everything behind it is float32; a request's state row holds the heads' matrices."""

    takes_pending_norm = True      # x goes to the packed product and nowhere else

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay_rank: int, tau: float, norm_eps: float):
        super().__init__()
        if not tau > 0:
            raise ValueError("the decay's temperature must be positive")
        self.hidden_size, self.num_heads, self.key_dim, self.value_dim = hidden_size, num_heads, key_dim, value_dim
        self.decay_rank, self.tau, self.norm_eps = decay_rank, float(tau), float(norm_eps)
        qk, inner = num_heads * key_dim, num_heads * value_dim
        self.qk, self.inner = qk, inner
        self.add_child("in_proj", Linear(hidden_size, 2 * qk + 2 * inner + decay_rank,
                                         parts={"q": qk, "k": qk, "v": inner, "g": inner, "a1": decay_rank}))
        self.add_child("a2", Linear(decay_rank, qk))
        self.add_param("a2_bias", ParamSpec((qk,), init=_decay_bias, dtype="float32"))
        self.add_param("norm_weight", ParamSpec((value_dim,), init="norm", dtype="float32"))
        self.add_child("o", Linear(inner, hidden_size))
        self._rate = self._norm = None

    def state_need(self):
        return StateNeed((self.num_heads * self.key_dim * self.value_dim,), "float32")

    def set_param(self, local, tensor):
        super().set_param(local, tensor)
        self._rate = None

    def finalize(self, device, dtype, max_positions):
        self._rate = torch.full((self.num_heads,), 1.0 / self.tau, dtype=torch.float32, device=device)
        self._norm = self.norm_weight.repeat(self.num_heads).contiguous()         # one weight for every head's values

    def forward(self, x, step, cache, state):
        H, N, P, qk, inner = self.num_heads, self.key_dim, self.value_dim, self.qk, self.inner
        rows = self.in_proj.forward(x)                                            # [T, q | k | v | g | a1]
        raw = self.a2.forward(rows[:, 2 * qk + 2 * inner:])
        y = ops.decay_rows_recurrence(rows[:, :qk], rows[:, qk:2 * qk], rows[:, 2 * qk:2 * qk + inner], raw, state, step.state_slots,
                                      step.cu_seqlens, step.q_lens, H, H, N, P, "gated", base=self.a2_bias, rate=self._rate,
                                      q_scale=N ** -0.5)
        g = rows[:, 2 * qk + inner:2 * qk + 2 * inner]
        o = ops.gated_rms_norm(y, g, self._norm, self.norm_eps, H, "silu_behind", g.dtype)
        return self.o.forward(o, allow_partials=True)
