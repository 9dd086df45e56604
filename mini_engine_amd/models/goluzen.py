"""Goluzen: a pre-norm decoder whose layers each name their mixer and their feed-forward, assembled from parts.

Per layer x += mixer(norm1(x)), x += feed_forward(norm2(x)), norm weights stored around zero (`PreNormBlock`; the sums
live in the float32 stream). Mixers: softmax attention with biases, a partly rotated head with stretched positions,
unit q and k, capped scores, a window that keeps the first positions and a sink per head (`Attention`); attention
over a latent that all heads share, the latent optionally another layer's (`LatentAttention`); linear attention with
a decay per key channel (`GatedLinearAttention`). Feed-forwards: dense with the tanh form of gelu (`ActivatedMLP`), or
routed experts without gates beside a shared expert under a gate per token (`RoutedExperts`). The embedding's rows are
multiplied by a constant; a final norm, then a head with weights of its own.

Checkpoint names: `embed`, `l<i>.norm1|norm2`, `l<i>.mix.<tensor>` (`.b` behind q, k, v for biases), `l<i>.mlp.up|down`,
`l<i>.mlp.router|correction`, `l<i>.mlp.e<j>.up|down`, `l<i>.mlp.shared.up|down|sg`, `final.norm`, `head`. The inner
width of the thin matrix pair of a `gla` layer (`a1`/`a2`) is read from the tensors' shapes.
"""
from __future__ import annotations

from ..config.model_config import ConfigError, GoluzenConfig
from ..parts.base import LayerCall, make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import register_architecture
from .model import DecoderModel, WeightSource
from .sigosun import _kernel_head_size
from .tavevik import default_rank


@register_architecture("Goluzen")
def build_goluzen(cfg: GoluzenConfig, checkpoint_shapes=None) -> DecoderModel:
    h, eps = cfg.hidden_size, cfg.norm_eps
    norm = lambda: make_part("norm", "rms", size=h, eps=eps, one_plus=True)
    layers, order, sources = [], [], {}
    rotations: dict = {}                      # layers with equal rotations share one table
    for i, layer in enumerate(cfg.layers):
        m, ck, me = layer.mixer, f"l{i}.mix.", f"layers.{i}.mixer."
        call = LayerCall(i)
        if layer.kind == "attention":
            D = _kernel_head_size(m["dim"], m["vdim"])
            position = None
            if m["rot_dims"]:
                sc = m["rot_scaling"]
                key = ("half", D, m["dim"], m["rot_dims"], m["rot_base"], None if sc is None else tuple(sorted(sc.items())))
                if key not in rotations:
                    rotations[key] = make_part("position_encoding", "rotary", head_dim=D, theta=m["rot_base"], stored_dim=m["dim"],
                                               rotary_dims=m["rot_dims"], interleaved=False, exact_angles=True, scaling=sc)
                position = rotations[key]
            mixer = make_part("mixer", "attention", hidden_size=h, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"],
                              value_dim=m["vdim"], scale=m["scale"], qk_norm_eps=eps, qk_norm_weights=False, position=position,
                              window=m["window"], keep_first=m["keep_first"], score_cap=m["softcap"], sinks=True, qkv_bias=True)
            q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            sources[me + "qkv.weight"] = [WeightSource(ck + "q", 0, q), WeightSource(ck + "k", q, k), WeightSource(ck + "v", q + k, v)]
            sources[me + "qkv_bias"] = [WeightSource(ck + "q.b", 0, q), WeightSource(ck + "k.b", q, k), WeightSource(ck + "v.b", q + k, v)]
            sources[me + "sinks"] = [WeightSource(ck + "sink")]
            sources[me + "o.weight"] = [WeightSource(ck + "o")]
        elif layer.kind == "latent_attention":
            own = m["kv_from"] is None
            position = None
            if m["rot_dim"]:
                sc = m["rot_scaling"]
                key = ("pairs", m["rot_dim"], m["rot_base"], None if sc is None else tuple(sorted(sc.items())))
                if key not in rotations:
                    rotations[key] = make_part("position_encoding", "rotary", head_dim=m["rot_dim"], theta=m["rot_base"],
                                               interleaved=True, exact_angles=True, scaling=sc)
                position = rotations[key]
            H, dn, dr, nv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            mixer = make_part("mixer", "latent_attention", hidden_size=h, num_heads=H, nope_dim=dn, rot_dim=dr, value_dim=nv, rank=R,
                              scale=m["scale"], norm_eps=eps, position=position, window=m["window"], own_kv=own, output_gate=True)
            blocks = [WeightSource(ck + "q", 0, H * (dn + dr))]
            at = H * (dn + dr)
            if own:
                blocks.append(WeightSource(ck + "dkv", at, R + dr))
                at += R + dr
                sources[me + "latent_norm_weight"] = [WeightSource(ck + "dkv.norm")]
            else:
                call = LayerCall(i, cache_of=m["kv_from"])
            blocks.append(WeightSource(ck + "g", at, H * nv))
            sources[me + "in_proj.weight"] = blocks
            sources[me + "uk"] = [WeightSource(ck + "uk")]
            sources[me + "uv"] = [WeightSource(ck + "uv")]
            sources[me + "o.weight"] = [WeightSource(ck + "o")]
        else:
            rank = m["decay_rank"]
            if rank is None and checkpoint_shapes is not None:
                if ck + "a1" not in checkpoint_shapes:
                    raise ConfigError(f"layers[{i}].mixer: the checkpoint lacks {ck + 'a1'!r}, whose shape gives the pair's inner width")
                rank = checkpoint_shapes[ck + "a1"][0]
            rank = int(rank) if rank is not None else default_rank(h)
            H, dn, nv = m["heads"], m["dim"], m["vdim"]
            mixer = make_part("mixer", "gla", hidden_size=h, num_heads=H, key_dim=dn, value_dim=nv, decay_rank=rank, tau=m["tau"], norm_eps=eps)
            qk, inner = H * dn, H * nv
            sources[me + "in_proj.weight"] = [WeightSource(ck + "q", 0, qk), WeightSource(ck + "k", qk, qk), WeightSource(ck + "v", 2 * qk, inner),
                                              WeightSource(ck + "g", 2 * qk + inner, inner), WeightSource(ck + "a1", 2 * qk + 2 * inner, rank)]
            for mine, stored in (("a2.weight", "a2"), ("a2_bias", "a2.b"), ("norm_weight", "norm"), ("o.weight", "o")):
                sources[me + mine] = [WeightSource(ck + stored)]
        order.append(call)
        f = layer.mlp
        ffn = norm2 = None
        if f is not None:
            ck, me = f"l{i}.mlp.", f"layers.{i}.feed_forward."
            norm2 = norm()
            sources[f"layers.{i}.norm2.weight"] = [WeightSource(f"l{i}.norm2")]
            if f["kind"] == "dense":
                ffn = make_part("feed_forward", "dense", hidden_size=h, intermediate_size=f["ff"], activation="gelu_tanh")
                sources[me + "up.weight"] = [WeightSource(ck + "up")]
                sources[me + "down.weight"] = [WeightSource(ck + "down")]
            else:
                shared = None
                if f["shared_ff"] is not None:
                    shared = make_part("feed_forward", "dense", hidden_size=h, intermediate_size=f["shared_ff"], activation="relu2",
                                       token_gate=True)
                    sources[me + "shared.up.weight"] = [WeightSource(ck + "shared.up")]
                    sources[me + "shared.down.weight"] = [WeightSource(ck + "shared.down")]
                    sources[me + "shared.token_gate_weight"] = [WeightSource(ck + "shared.sg")]
                E, F = f["experts"], f["ff"]
                ffn = make_part("feed_forward", "moe", hidden_size=h, intermediate_size=F, num_experts=E, top=f["top"],
                                group_count=f["group_count"], group_keep=f["group_keep"], shared=shared, gated=False, scoring="sigmoid",
                                correction=True, group_top=2, normalise=False, route_scale=f["scale"], sum_outputs=True)
                sources[me + "router"] = [WeightSource(ck + "router")]
                sources[me + "correction"] = [WeightSource(ck + "correction")]
                sources[me + "gate_up"] = [WeightSource(f"{ck}e{e}.up", e * F, F) for e in range(E)]
                sources[me + "down"] = [WeightSource(f"{ck}e{e}.down", e * h, h) for e in range(E)]
        layers.append(make_part("block", "pre_norm", norm1=norm(), mixer=mixer, norm2=norm2, feed_forward=ffn))
        sources[f"layers.{i}.norm1.weight"] = [WeightSource(f"l{i}.norm1")]
    embedding = TokenEmbedding(cfg.vocab_size, h, scale=cfg.embedding_scale)
    head = LMHead(cfg.vocab_size, h)
    sources["embedding.weight"] = [WeightSource("embed")]
    sources["final_norm.weight"] = [WeightSource("final.norm")]
    sources["head.weight"] = [WeightSource("head")]
    return DecoderModel(cfg, embedding, layers, order, norm(), head, sources)
