"""Tavevik: a decoder whose every layer runs softmax attention and a recurrence side by side, assembled from parts.

Per layer the norm sits on the sublayer's output only (`OutputNormBlock`, plain weights). The mixer is a `SideBySide`
of an `Attention` (grouped key/value heads of their own value size, per-head q/k norm, a rotation of the first
dimensions of each head with pairs half the rotating width apart, a trailing window) and a recurrence:
kind `parallel`   the attention keeps its first positions behind the window, caps its scores and gates its heads
                  element by element; beside it a `ShiftedDecay`;
kind `parallel_2` the attention has biases on q, k, v and o and a sink per head; beside it a `GatedDelta`.
A layer may have a feed-forward with a clamped gated activation (`ClampedGLU`). A final norm, then the embedding
matrix as the head.

Checkpoint names: `embed`, `l<i>.norm1|norm2`, `l<i>.mix.left.q|k|v|o` (`.b` behind them for biases, `.norm` behind q
and k), `l<i>.mix.left.g|sink`, `l<i>.mix.right.*`, `l<i>.mlp.gate|up|down`, `final.norm`. The inner widths of the thin
matrix pairs of the right side (`w1`/`w2`, `a1`/`a2`, `g1`/`g2`) are read from the tensors' shapes.
"""
from __future__ import annotations

from ..config.model_config import ConfigError, TavevikConfig
from ..parts.base import LayerCall, make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import register_architecture
from .model import DecoderModel, WeightSource
from .sigosun import _kernel_head_size


def default_rank(width: int) -> int:
    """The inner width of a thin matrix pair when neither the file nor a checkpoint names one (random weights)."""
    return max(8, width // 16 // 8 * 8)


def _rank(named, shapes, tensor: str, width: int, where: str) -> int:
    if named is not None:
        return int(named)
    if shapes is not None:
        if tensor not in shapes:
            raise ConfigError(f"{where}: the checkpoint lacks {tensor!r}, whose shape gives the pair's inner width")
        return int(shapes[tensor][0])
    return default_rank(width)


@register_architecture("Tavevik")
def build_tavevik(cfg: TavevikConfig, checkpoint_shapes=None) -> DecoderModel:
    h, eps = cfg.hidden_size, cfg.norm_eps
    norm = lambda: make_part("norm", "rms", size=h, eps=eps)
    layers, sources = [], {}
    rotations: dict = {}                      # layers with equal rotations share one table
    for i, layer in enumerate(cfg.layers):
        l, r = layer.left, layer.right
        second = layer.kind == "parallel_2"
        # ---- the left side
        ck, me = f"l{i}.mix.left.", f"layers.{i}.mixer.left."
        D = _kernel_head_size(l["dim"], l["vdim"])
        position = None
        if l["rot_dims"]:
            key = (D, l["dim"], l["rot_dims"], l["rot_base"])
            if key not in rotations:
                rotations[key] = make_part("position_encoding", "rotary", head_dim=D, theta=l["rot_base"], stored_dim=l["dim"],
                                           rotary_dims=l["rot_dims"], interleaved=False, exact_angles=True)
            position = rotations[key]
        left = make_part("mixer", "attention", hidden_size=h, num_heads=l["heads"], num_kv_heads=l["kv_heads"], head_dim=l["dim"],
                         value_dim=l["vdim"], scale=l["scale"], qk_norm_eps=eps, position=position, window=l["window"],
                         keep_first=l["keep_first"], score_cap=l["softcap"], sinks=second, qkv_bias=second, out_bias=second,
                         output_gate=not second)
        q, k, v = l["heads"] * l["dim"], l["kv_heads"] * l["dim"], l["kv_heads"] * l["vdim"]
        blocks = [WeightSource(ck + "q", 0, q), WeightSource(ck + "k", q, k), WeightSource(ck + "v", q + k, v)]
        if second:
            sources[me + "qkv_bias"] = [WeightSource(ck + "q.b", 0, q), WeightSource(ck + "k.b", q, k), WeightSource(ck + "v.b", q + k, v)]
            sources[me + "sinks"] = [WeightSource(ck + "sink")]
            sources[me + "o_bias"] = [WeightSource(ck + "o.b")]
        else:
            blocks.append(WeightSource(ck + "g", q + k + v, l["heads"] * l["vdim"]))
        sources[me + "qkv.weight"] = blocks
        sources[me + "q_norm_weight"] = [WeightSource(ck + "q.norm")]
        sources[me + "k_norm_weight"] = [WeightSource(ck + "k.norm")]
        sources[me + "o.weight"] = [WeightSource(ck + "o")]
        # ---- the right side
        ck, me = f"l{i}.mix.right.", f"layers.{i}.mixer.right."
        where = f"layers[{i}].mixer.right"
        if second:
            rank_a = _rank(r["decay_rank"], checkpoint_shapes, ck + "a1", h, where)
            rank_g = _rank(r["gate_rank"], checkpoint_shapes, ck + "g1", h, where)
            right = make_part("mixer", "gated_delta", hidden_size=h, num_heads=r["heads"], key_heads=r["kv_heads"], key_dim=r["dim"],
                              value_dim=r["vdim"], taps=r["conv"], decay_rank=rank_a, gate_rank=rank_g, norm_eps=eps)
            qk, inner, H = r["kv_heads"] * r["dim"], r["heads"] * r["vdim"], r["heads"]
            at = 2 * qk + inner
            sources[me + "in_proj.weight"] = [WeightSource(ck + "q", 0, qk), WeightSource(ck + "k", qk, qk), WeightSource(ck + "v", 2 * qk, inner),
                                              WeightSource(ck + "b", at, H), WeightSource(ck + "a1", at + H, rank_a),
                                              WeightSource(ck + "g1", at + H + rank_a, rank_g)]
            sources[me + "conv_weight"] = [WeightSource(ck + "q.conv", 0, qk), WeightSource(ck + "k.conv", qk, qk),
                                           WeightSource(ck + "v.conv", 2 * qk, inner)]
            for mine, stored in (("a2.weight", "a2"), ("g2.weight", "g2"), ("dt_bias", "dt_bias"), ("A_log", "A_log"),
                                 ("norm_weight", "norm"), ("o.weight", "o")):
                sources[me + mine] = [WeightSource(ck + stored)]
        else:
            rank_w = _rank(r["decay_rank"], checkpoint_shapes, ck + "w1", h, where)
            right = make_part("mixer", "shifted_decay", hidden_size=h, num_heads=r["heads"], key_dim=r["dim"], decay_rank=rank_w,
                              norm_eps=eps)
            sources[me + "mu"] = [WeightSource(f"{ck}mu.{s}", j * h, h) for j, s in enumerate(right.MIXES)]
            for name in ("r", "k", "v", "g", "w1", "w2", "o"):
                sources[me + name + ".weight"] = [WeightSource(ck + name)]
            for mine, stored in (("w0", "w0"), ("u", "u"), ("norm_weight", "norm")):
                sources[me + mine] = [WeightSource(ck + stored)]
        mixer = make_part("mixer", "side_by_side", left=left, right=right, left_scale=layer.left_scale, right_scale=layer.right_scale)
        ffn = norm2 = None
        if layer.mlp is not None:
            F = layer.mlp["ff"]
            ffn, norm2 = make_part("feed_forward", "clamped_glu", hidden_size=h, intermediate_size=F, limit=layer.mlp["limit"]), norm()
            sources[f"layers.{i}.norm2.weight"] = [WeightSource(f"l{i}.norm2")]
            sources[f"layers.{i}.feed_forward.gate_up.weight"] = [WeightSource(f"l{i}.mlp.gate", 0, F), WeightSource(f"l{i}.mlp.up", F, F)]
            sources[f"layers.{i}.feed_forward.down.weight"] = [WeightSource(f"l{i}.mlp.down")]
        layers.append(make_part("block", "output_norm", norm1=norm(), mixer=mixer, norm2=norm2, feed_forward=ffn))
        sources[f"layers.{i}.norm1.weight"] = [WeightSource(f"l{i}.norm1")]
    embedding = TokenEmbedding(cfg.vocab_size, h)
    head = LMHead(cfg.vocab_size, h, tied_to=embedding)
    sources["embedding.weight"] = [WeightSource("embed")]
    sources["final_norm.weight"] = [WeightSource("final.norm")]
    return DecoderModel(cfg, embedding, layers, [LayerCall(i) for i in range(len(layers))], norm(), head, sources)
