"""Attention whose keys and values are made, head by head, from one small latent vector per token."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import CacheNeed, Mixer, ParamSpec, PositionEncoding, register_part
from .linear import Linear


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """Per token the layer makes a latent c = norm(W_dkv x)[: rank] (RMS norm with a weight) and one rotated key part
    r = rot(W_dkv x)[rank :] that all heads share. Head h has the key [W_uk[h] c | r] and the value W_uv[h] c; its query
    W_q x is laid out [nope_dim unrotated | rot_dim rotated]. score = (q_nope . W_uk[h] c + q_rot . r) * scale, causal,
    optionally inside a trailing window; softmax; the heads side by side are, with `output_gate`, multiplied element by
    element by sigmoid(W_g x), then projected.

    Only c and r are cached, and the keys and values of a head are never formed: q_nope . (W_uk[h] c) = (W_uk[h]^T q_nope) . c,
    so the queries are carried into the latent's space (`ops.heads_linear`), every head then attends to the same keys
    [c | r] and values c (one key/value head of `rank + rot_dim` dimensions for the paged attention kernels, prompts and
    single tokens alike), and W_uv[h] carries each head's result out of the latent's space again. `own_kv=False`: a layer
    call that reads the pages of an earlier latent layer with its own queries and W_uk, W_uv; it has no W_dkv.

    `position`: a rotary encoding over `rot_dim` dimensions in adjacent pairs (its table is read as it stands; any scaling
    of the positions lives there). q, the latent's rows and the gate are one packed product."""

    takes_pending_norm = True      # x goes to the packed product and nowhere else

    def __init__(self, hidden_size: int, num_heads: int, nope_dim: int, rot_dim: int, value_dim: int, rank: int, scale: float,
                 norm_eps: float, position: PositionEncoding | None, window: int | None = None, own_kv: bool = True,
                 output_gate: bool = False):
        super().__init__()
        if rot_dim % 2 or (rot_dim and position is None):
            raise ValueError("the rotating part has an even size and needs a position encoding")
        if position is not None and (position.head_dim != rot_dim or position.rotary_dims != rot_dim or not position.interleaved):
            raise ValueError("the position encoding must turn all of the rotating part, in adjacent pairs")
        self.hidden_size, self.num_heads, self.nope_dim, self.rot_dim = hidden_size, num_heads, nope_dim, rot_dim
        self.value_dim, self.rank, self.scale, self.norm_eps = value_dim, rank, float(scale), float(norm_eps)
        self.window, self.own_kv, self.output_gate = window, bool(own_kv), bool(output_gate)
        self.head_dim = -(-(rank + rot_dim) // 16) * 16          # the attention kernels' head size: whole steps of 16
        H = num_heads
        blocks = {"q": H * (nope_dim + rot_dim)}
        if own_kv:
            blocks["dkv"] = rank + rot_dim
        if output_gate:
            blocks["g"] = H * value_dim
        self.kv_at = blocks["q"] if own_kv else None
        self.gate_at = blocks["q"] + (blocks["dkv"] if own_kv else 0)
        self.add_child("in_proj", Linear(hidden_size, sum(blocks.values()), parts=blocks))
        if own_kv:
            self.add_param("latent_norm_weight", ParamSpec((rank,), init="norm", dtype="float32"))
        else:
            self.latent_norm_weight = None
        self.add_param("uk", ParamSpec((H * nope_dim, rank), init="matrix", dtype="compute"))
        self.add_param("uv", ParamSpec((H * value_dim, rank), init="matrix", dtype="compute"))
        self.add_child("o", Linear(H * value_dim, hidden_size))
        if position is not None:
            self.add_child("position", position)
        else:
            self.position = None
        self._uk_t = None

    def cache_need(self):
        return CacheNeed.keys_and_values(1, self.head_dim, self.window)

    def set_param(self, local, tensor):
        super().set_param(local, tensor)
        self._uk_t = None

    def finalize(self, device, dtype, max_positions):
        # W_uk[h]^T, [heads, rank, nope_dim]: the matrix that carries a head's unrotated query part into the latent's space
        self._uk_t = self.uk.view(self.num_heads, self.nope_dim, self.rank).transpose(1, 2).contiguous()

    def forward(self, x, step, cache, state):
        H, dn, dr, R, D, nv = self.num_heads, self.nope_dim, self.rot_dim, self.rank, self.head_dim, self.value_dim
        grp = step.groups[cache.group]
        rows = self.in_proj.forward(x)
        T = rows.shape[0]
        write = self.own_kv and cache.write
        table = self.position.rotary_table() if self.position is not None else None
        qa = ops.latent_prepare(rows, 0, self.kv_at if write else None, H, dn, dr, R, D, self.latent_norm_weight, self.norm_eps,
                                table, step.positions, grp.slot_mapping, cache.k, cache.v, cache.page_size)
        q3 = qa.view(T, H, D)
        ops.heads_linear(rows[:, : H * (dn + dr)].view(T, H, dn + dr)[:, :, :dn], self._uk_t, q3[:, :, :R])
        o = ops.paged_attention(qa, cache.k, cache.v, cache.page_size, grp.block_tables, step.context_lens, step.seq_of_token,
                                step.positions, step.prefill_cu, step.num_decodes, step.max_decode_context, self.scale,
                                self.window, H, 1, D, max_prefill_context=step.max_prefill_context,
                                even_contexts=step.decode_contexts_even)
        heads = torch.empty((T, H * nv), dtype=rows.dtype, device=rows.device)
        ops.heads_linear(o.view(T, H, D)[:, :, :R], self.uv.view(H, nv, R), heads.view(T, H, nv))
        if self.output_gate:
            ops.sigmoid_gate_(heads, rows[:, self.gate_at:self.gate_at + H * nv])
        return self.o.forward(heads, allow_partials=True)
