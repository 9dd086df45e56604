"""Grouped-query attention over the paged cache (reference models/qwen3.py:12-38,
layers/attention.py:43-76)."""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import CacheNeed, Mixer, ParamSpec, PositionEncoding, register_part
from .linear import Linear


def _half(shape, generator, device):
    return 0.25 + 0.5 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device)


@register_part("mixer", "attention")
class Attention(Mixer):
    """q, k, v from one packed product; optional per-head RMSNorm of q and k over the head
    size (applied before the position encoding, not to v); position encoding; causal
    attention of the new tokens over all cached keys of the request (or the last `window`);
    output product.

    Consecutive query heads share a key/value head: kv head = q head // (Hq/Hkv).
    `own_kv=False` builds a mixer with queries only, for a layer call that reads the cache
    another call has written.

    Further options, all off by default: `value_dim` (values of another size than queries and keys),
    `chunk` (a block mask: the query at position i sees the keys j <= i with floor(j / chunk) = floor(i / chunk),
    blocks counted from position 0 of the request), `head_gate` (each head's output is multiplied by the
    sigmoid of one more output feature of the packed product, one per head), and a position encoding that
    wants the heads laid out differently from how they are stored (`PositionEncoding.head_order`: partial or
    interleaved rotations). The parameters are declared as they are stored (q, k, v and gate rows, heads of
    `head_dim` and `value_dim`); where the kernels need another layout (one head size for keys and values, a
    multiple of 16; the rotation's pairs half a head apart; rows in steps of 8), `finalize` builds it once: rows
    reordered within each head, zero rows and columns where a head is padded, the norm weights scaled so that a
    mean over the padded head equals the mean over the stored one.

    A second family of options runs through a prologue kernel of its own (`ops.qkv_prepare_store`) on the unrounded
    sums of the packed product: `qkv_bias` (q, k and v carry biases), `qk_norm_over="projection"` (q and k are each
    normed as a whole, all heads at once, with weights of the projection's size; this needs no position encoding),
    `q_temperature=(coef, every)` (the query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)),
    and `value_mix`: "first" keeps this layer's values of the step's tokens under `value_mix_key` in the step's shared
    values; "blend" replaces its own by (1 - lambda) v + lambda v_first with a learned scalar lambda (`vmix`) before
    they are cached. Layers that share a key have the same number of value dimensions.

    Options of the mask and the softmax (they go to the attention kernels as they are): `keep_first` (behind the window
    the keys at positions below it stay visible, at their true positions), `score_cap` c (a score s becomes c * tanh(s /
    c)), `sinks` (a learned number per query head whose exponential joins the softmax's denominator without a key or a
    value). Options around the products: `output_gate` (the concatenated heads are multiplied element by element by the
    sigmoid of further output features of the packed product, as many as the heads' values), `out_bias` (a bias on the
    output product), and `qkv_bias` together with per-head norms or a position encoding (the biases are then added to
    the packed product's unrounded sums by a kernel of their own in front of the per-head norm and rotation).
    `qk_norm_weights=False`: the per-head norm of q and k has no learned weights (every head is brought to unit root mean
    square and that is all). Such a norm may stand in front of the rotation or behind it: a rotation changes no pair's
    length, so the head's mean square, and with it the result, is the same either way.
    """

    takes_pending_norm = True      # x goes to the packed product and nowhere else

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, qk_norm_eps: float | None = None, position: PositionEncoding | None = None,
                 window: int | None = None, own_kv: bool = True, value_dim: int | None = None,
                 chunk: int | None = None, head_gate: bool = False, qkv_bias: bool = False, qk_norm_over: str = "head",
                 q_temperature: tuple | None = None, value_mix: str | None = None, value_mix_key: str = "v_first",
                 keep_first: int = 0, score_cap: float | None = None, sinks: bool = False, output_gate: bool = False,
                 out_bias: bool = False, qk_norm_weights: bool = True):
        super().__init__()
        if qk_norm_over not in ("head", "projection") or value_mix not in (None, "first", "blend"):
            raise ValueError("qk_norm_over is 'head' or 'projection', value_mix None, 'first' or 'blend'")
        self.qkv_bias_on = bool(qkv_bias)
        self.norm_over = qk_norm_over
        self.q_temperature = None if q_temperature is None else (float(q_temperature[0]), int(q_temperature[1]))
        if self.q_temperature is not None and self.q_temperature[1] < 1:
            raise ValueError("the query temperature's period must be positive")
        self.value_mix, self.value_mix_key = value_mix, value_mix_key
        self.keep_first, self.score_cap = int(keep_first or 0), (float(score_cap) if score_cap else None)
        self.output_gate, self.out_bias_on = bool(output_gate), bool(out_bias)
        if self.keep_first and not window:
            raise ValueError("keys are kept behind a window only")
        if head_gate and output_gate:
            raise ValueError("a gate per head and a gate per element exclude each other")
        per_head_path = (position is not None or not own_kv or head_gate or output_gate
                         or (qk_norm_eps is not None and qk_norm_over == "head"))
        self.prologue = bool(qk_norm_over == "projection" or q_temperature is not None or value_mix or (qkv_bias and not per_head_path))
        if self.prologue and per_head_path:
            raise ValueError("biases, whole-projection norms, query temperatures and value mixing come without a position "
                             "encoding, head gates or per-head norms, on keys and values of the layer's own")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = float(scale)
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.own_kv = own_kv
        if window is not None and chunk is not None:
            raise ValueError("a trailing window and a block mask exclude each other")
        self.chunk = chunk
        self.head_gate = bool(head_gate)
        self.stored_dim = head_dim
        self.value_dim = head_dim if value_dim is None else int(value_dim)
        order = position.head_order() if position is not None and hasattr(position, "head_order") else None
        slots = getattr(position, "head_dim", head_dim) if position is not None else head_dim
        if self.value_dim != head_dim or slots != head_dim:
            # one head size for the kernels: the larger of the two, in whole steps of 16
            head_dim = self.head_dim = max(slots, -(-max(head_dim, self.value_dim) // 16) * 16)
            if position is not None and slots != head_dim:
                raise ValueError(f"the position encoding must be built for the kernels' head size {head_dim}")
        self._relayout = order is not None or head_dim != self.stored_dim or head_dim != self.value_dim
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim
        stored_q, stored_k, stored_v = num_heads * self.stored_dim, num_kv_heads * self.stored_dim, num_kv_heads * self.value_dim
        blocks = {"q": stored_q}
        if own_kv:
            blocks.update(k=stored_k, v=stored_v)
        if head_gate:
            blocks["g"] = num_heads
        if output_gate:
            blocks["g"] = num_heads * self.value_dim
        self.add_child("qkv", Linear(hidden_size, sum(blocks.values()), parts=blocks))
        self.add_child("o", Linear(num_heads * self.value_dim, hidden_size))
        rows = self.q_size + (2 * self.kv_size if own_kv else 0) + (num_heads if head_gate else 0) + (self.q_size if output_gate else 0)
        self._relayout = self._relayout or rows % 8 != 0
        self.gate_at = self.q_size + (2 * self.kv_size if own_kv else 0)      # first gate column of the kernels' rows
        self._laid_out = False
        self.qk_norm_weights = bool(qk_norm_weights)
        if qk_norm_eps is not None and not self.qk_norm_weights:
            if qk_norm_over != "head":
                raise ValueError("a norm without weights is a norm per head")
            self.q_norm_weight = self.k_norm_weight = None
        elif qk_norm_eps is not None:
            whole = qk_norm_over == "projection"
            self.add_param("q_norm_weight", ParamSpec((stored_q if whole else self.stored_dim,), init="norm", dtype="float32"))
            if own_kv:
                self.add_param("k_norm_weight", ParamSpec((stored_k if whole else self.stored_dim,), init="norm", dtype="float32"))
        if qkv_bias:
            self.add_param("qkv_bias", ParamSpec((stored_q + stored_k + stored_v,), init="matrix", dtype="float32"))
        if sinks:
            self.add_param("sinks", ParamSpec((num_heads,), init="matrix", dtype="float32"))
        else:
            self.sinks = None
        if out_bias:
            self.add_param("o_bias", ParamSpec((hidden_size,), init="matrix", dtype="float32"))
        else:
            self.o_bias = None
        if value_mix == "blend":
            self.add_param("vmix", ParamSpec((), init=_half, dtype="float32"))
        self.norm_eps = qk_norm_eps
        if position is not None:
            self.add_child("position", position)
        else:
            self.position = None

    def cache_need(self):
        return CacheNeed.keys_and_values(self.num_kv_heads, self.head_dim, self.window, self.chunk, self.keep_first)

    def set_param(self, local, tensor):
        super().set_param(local, tensor)
        self._laid_out = False

    def finalize(self, device, dtype, max_positions):
        """The kernels' layout of the stored parameters, where it differs (see the class text)."""
        if self.norm_eps is not None and not self.qk_norm_weights and not self._laid_out:
            self.q_norm_weight = torch.ones(self.stored_dim, dtype=torch.float32, device=device)
            self.k_norm_weight = torch.ones(self.stored_dim, dtype=torch.float32, device=device) if self.own_kv else None
        if not self._relayout or self._laid_out:
            return
        H, G, D, n, nv = self.num_heads, self.num_kv_heads, self.head_dim, self.stored_dim, self.value_dim
        order = self.position.head_order() if self.position is not None and hasattr(self.position, "head_order") else None
        take = torch.tensor(order if order is not None else list(range(n)) + [-1] * (D - n), dtype=torch.long)
        w = self.qkv.weight
        hidden = w.shape[1]

        def heads(block, count, size, pick):
            """[count * size, hidden] -> [count * D, hidden]: slot s of every head holds stored row pick[s] (zeros for -1)."""
            wide = torch.cat((block.view(count, size, hidden), block.new_zeros(count, 1, hidden)), 1)
            return wide[:, pick.to(block.device)].reshape(count * D, hidden)       # index -1 is the zero row

        stored_q, stored_k = H * n, G * n
        parts = [heads(w[:stored_q], H, n, take)]
        at = stored_q
        if self.own_kv:
            keep = torch.tensor(list(range(nv)) + [-1] * (D - nv), dtype=torch.long)
            parts += [heads(w[at:at + stored_k], G, n, take), heads(w[at + stored_k:at + stored_k + G * nv], G, nv, keep)]
            at += stored_k + G * nv
        if self.head_gate:
            parts.append(w[at:at + H])
        if self.output_gate:                 # the gates take the slots of the values they multiply
            keep_o = torch.tensor(list(range(nv)) + [-1] * (D - nv), dtype=torch.long)
            parts.append(heads(w[at:at + H * nv], H, nv, keep_o))
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:
            parts.append(w.new_zeros(8 - rows % 8, hidden))
        self.qkv.weight = torch.cat(parts, 0).contiguous()
        o = self.o.weight.view(-1, H, nv)
        self.o.weight = torch.cat((o, o.new_zeros(o.shape[0], H, D - nv)), 2).reshape(-1, H * D).contiguous()
        if self.qkv_bias_on:
            b = self.qkv_bias
            wide = lambda block, count, size, pick: torch.cat((block.view(count, size), block.new_zeros(count, 1)), 1)[:, pick.to(block.device)].reshape(-1)
            self.qkv_bias = torch.cat((wide(b[:stored_q], H, n, take), wide(b[stored_q:stored_q + stored_k], G, n, take),
                                       wide(b[stored_q + stored_k:], G, nv, keep))).contiguous()
        if self.norm_eps is not None and self.norm_over == "projection":
            # the kernel divides the sum of squares by the stored count itself: the weights only move to their slots
            for name, count in (("q_norm_weight", H), ("k_norm_weight", G)):
                wn = getattr(self, name)
                setattr(self, name, torch.cat((wn.view(count, n), wn.new_zeros(count, 1)), 1)[:, take.to(wn.device)].reshape(-1).contiguous())
        elif self.norm_eps is not None:
            # mean over D slots instead of n stored dimensions: eps and the weights take the ratio
            self.qk_norm_eps = self.norm_eps * n / D
            fix = math.sqrt(n / D)
            for name in ("q_norm_weight", "k_norm_weight") if self.own_kv else ("q_norm_weight",):
                wn = getattr(self, name)
                wide = torch.cat((wn * fix, wn.new_zeros(1)))
                setattr(self, name, wide[take.to(wn.device)].contiguous())
        self._laid_out = True

    def _forward_with_prologue(self, x, step, cache):
        """Bias, whole-projection norm, temperature and value mixing on the product's float32 sums, then attention."""
        Hq, Hkv, D, nv = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        grp = step.groups[cache.group]
        rows = self.qkv.forward(x, out_dtype=torch.float32)
        mix, v_first = 0, None
        if self.value_mix is not None:
            if self.value_mix == "first":
                mix, v_first = 1, torch.empty((rows.shape[0], Hkv * nv), dtype=torch.float32, device=rows.device)
                step.shared[self.value_mix_key] = v_first
            else:
                mix, v_first = 2, step.shared.get(self.value_mix_key)
                if v_first is None or v_first.shape != (rows.shape[0], Hkv * nv):
                    raise RuntimeError(f"value mixing: no layer before this one has left {Hkv * nv} value dimensions "
                                       f"per token under {self.value_mix_key!r}")
        normed = self.norm_eps is not None
        q = ops.qkv_prepare_store(rows, self.qkv_bias if self.qkv_bias_on else None, self.q_norm_weight if normed else None,
                                  self.k_norm_weight if normed else None, self.norm_eps or 0.0, Hq * self.stored_dim,
                                  Hkv * self.stored_dim, self.q_temperature, step.positions, grp.slot_mapping, cache.k, cache.v,
                                  Hq, Hkv, D, cache.page_size, nv, mix, self.vmix if mix == 2 else None, v_first)
        o = ops.paged_attention(q, cache.k, cache.v, cache.page_size, grp.block_tables, step.context_lens,
                                step.seq_of_token, step.positions, step.prefill_cu, step.num_decodes,
                                step.max_decode_context, self.scale, self.window, Hq, Hkv, D,
                                max_prefill_context=step.max_prefill_context,
                                even_contexts=step.decode_contexts_even, chunk=self.chunk)
        return self.o.forward(o, allow_partials=True)

    def forward(self, x, step, cache, state):
        if self.prologue:
            return self._forward_with_prologue(x, step, cache)
        Hq, Hkv, D = self.num_heads, self.num_kv_heads, self.head_dim
        grp = step.groups[cache.group]
        if self.qkv_bias_on:                # the bias joins the unrounded sums; one rounding behind it
            dtype = self.qkv.weight.dtype
            packed = ops.add_bias(self.qkv.forward(x, out_dtype=torch.float32), self.qkv_bias, dtype)
        else:
            packed = self.qkv.forward(x)
        gated = self.head_gate
        extras = dict(keep_first=self.keep_first, softcap=self.score_cap, sinks=self.sinks)
        plain_scores = not self.keep_first and self.score_cap is None and self.sinks is None
        # the kernels' rows end where the gate columns (and the padding to whole steps of 8) begin
        qkv = packed if packed.shape[1] == self.gate_at else packed[:, : self.gate_at]
        store = self.own_kv and cache.write
        qw = self.q_norm_weight if self.qk_norm_eps is not None else None
        kw = self.k_norm_weight if (self.qk_norm_eps is not None and self.own_kv) else qw
        table = self.position.rotary_table() if self.position is not None else None
        eps = self.qk_norm_eps or 0.0
        if (store and step.num_decodes == step.num_tokens and (self.position is None or table is not None)
                and plain_scores and ops.decode_step_fuses(qkv.dtype, D, cache.page_size)):
            # only single tokens: norm, rotary, cache write and attention in one launch
            o = ops.decode_step_attention(qkv, qw, kw, eps, table, cache.k, cache.v, cache.page_size, grp.block_tables,
                                          step.context_lens, step.max_decode_context, self.scale, self.window,
                                          Hq, Hkv, D, even_contexts=step.decode_contexts_even, chunk=self.chunk)
            if gated:
                ops.head_gate(o, packed[:, self.gate_at:self.gate_at + Hq], Hq, D)
            return self._project(o, packed)
        if self.position is None or table is not None:
            # norm + rotary + cache write in one pass
            bound = max(step.max_decode_context, step.max_prefill_context)
            if store:
                ops.qk_norm_rope_store(qkv, qw, kw, eps, table, step.positions, grp.slot_mapping,
                                       cache.k, cache.v, Hq, Hkv, D, cache.page_size, store=True, position_bound=bound)
            else:
                rows = qkv[:, : self.q_size]
                ops.qk_norm_rope_store(rows, qw, kw, eps, table, step.positions, None, None, None,
                                       Hq, 0, D, cache.page_size, store=False, position_bound=bound)
        else:
            # another position encoding: norm in place, the encoding's own apply, then the cache write
            nk = Hkv if self.own_kv else 0
            ops.qk_norm_rope_store(qkv[:, : self.q_size + nk * D], qw, kw, eps, None, step.positions, None, None,
                                   None, Hq, nk, D, cache.page_size, store=False)
            T = qkv.shape[0]
            q3 = qkv[:, : self.q_size].view(T, Hq, D)
            k3 = qkv[:, self.q_size: self.q_size + nk * D].view(T, nk, D)
            self.position.apply(q3, k3, step.positions)
            if store:
                v3 = qkv[:, self.q_size + self.kv_size: self.q_size + 2 * self.kv_size].view(T, Hkv, D)
                ops.store_kv(k3, v3, grp.slot_mapping, cache.k, cache.v, cache.page_size)
        q = qkv[:, : self.q_size]
        o = ops.paged_attention(q, cache.k, cache.v, cache.page_size, grp.block_tables, step.context_lens,
                                step.seq_of_token, step.positions, step.prefill_cu, step.num_decodes,
                                step.max_decode_context, self.scale, self.window, Hq, Hkv, D,
                                max_prefill_context=step.max_prefill_context,
                                even_contexts=step.decode_contexts_even, chunk=self.chunk, **extras)
        if gated:
            ops.head_gate(o, packed[:, self.gate_at:self.gate_at + Hq], Hq, D)
        return self._project(o, packed)

    def _project(self, o, packed):
        """The element gate, the output product and its bias."""
        if self.output_gate:
            ops.sigmoid_gate_(o, packed[:, self.gate_at:self.gate_at + self.q_size])
        y = self.o.forward(o, allow_partials=True)
        if self.out_bias_on:
            if getattr(self, "defer_bias", False):       # the caller adds it where it adds the output itself
                from .hybrid import Biased
                return Biased(y, self.o_bias)
            y = ops.add_bias(y, self.o_bias, self.o.weight.dtype)
        return y
