"""The layer sizes of the Qwen3 dense models that the benchmarks and the command lines name, for runs
with random weights (no model folder at hand). The figures are those of the published config.json
files; a model folder's own config.json always wins where there is one."""
from __future__ import annotations

from .model_config import GoluzenConfig, NegosunConfig, Qwen3Config, SigosunConfig, TavevikConfig

SIZES = {
    # name: (layers, hidden, q heads, kv heads, head_dim, intermediate, vocab, tied)
    "tinyA": (2, 64, 4, 2, 16, 128, 256, True),
    "0.6b": (28, 1024, 16, 8, 128, 3072, 151936, True),
    "1.7b": (28, 2048, 16, 8, 128, 6144, 151936, True),
    "4b": (36, 2560, 32, 8, 128, 9728, 151936, True),
    "8b": (36, 4096, 32, 8, 128, 12288, 151936, False),
    "14b": (40, 5120, 40, 8, 128, 17408, 151936, False),
    "32b": (64, 5120, 64, 8, 128, 25600, 151936, False),
}


def model_config(size: str, layers: int | None = None):
    """(typed configuration of that size with `layers` layers, or all of them; the size's own layer count)."""
    L, h, Hq, Hkv, D, I, V, tied = SIZES[size]
    return Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], vocab_size=V, hidden_size=h, intermediate_size=I,
        num_hidden_layers=layers or L, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D,
        rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=tied, max_position_embeddings=40960)), L


def sigosun_config(size: str, layers: int | None = None):
    """(a Sigosun configuration whose layers resemble that size's: the same width, vocabulary, feed-forward width and
    attention heads, with `layers` layers or as many as the size has; that count). The mixers take turns: linear
    attention, attention with keys of its own, a state-space layer, linear attention, attention on the keys of the
    attention layer before it, a state-space layer; the attention layers carry the feed-forwards. Blocks of 2,048
    positions, half of each head's dimensions turning; state-space heads of 64 with a state of 128; linear
    attention with the attention layers' head size."""
    L, h, Hq, Hkv, D, I, V, _ = SIZES[size]
    n = layers or L
    attention = lambda src: {"type": "attention", "mlp": {"kind": "dense", "ff": I},
                             "mixer": dict({"heads": Hq, "kv_heads": Hkv, "dim": D, "vdim": D, "scale": D ** -0.5,
                                            "rot": {"dims": D // 2, "base": 1e6}, "mask": {"size": 2048}},
                                           **({} if src is None else {"kv_from": src}))}
    space = {"type": "mamba2", "mlp": None, "mixer": {"heads": 2 * h // 64, "vdim": 64, "state": 128, "groups": 1, "conv": 4,
                                                      "norm_groups": 1}}
    linear = {"type": "lightning", "mlp": None,
              "mixer": {"heads": Hq, "dim": D, "vdim": D, "decay": [1.0 - 2.0 ** (-5 - 8 * i / max(1, Hq - 1)) for i in range(Hq)]}}
    out, last_own = [], None
    for i in range(n):
        turn = i % 6
        if turn in (0, 3):
            out.append(linear)
        elif turn in (2, 5):
            out.append(space)
        elif turn == 1 or last_own is None:
            out.append(attention(None))
            last_own = i
        else:
            out.append(attention(last_own))
    return SigosunConfig.from_dict({"architecture": "Sigosun", "vocab": V, "width": h, "norm": {"eps": 1e-6}, "layers": out,
                                    "max_position_embeddings": 40960}), L


def negosun_config(size: str, layers: int | None = None):
    """(a Negosun configuration whose layers resemble that size's: the same width, vocabulary and attention heads, with
    `layers` layers or as many as the size has; that count). Every layer mixes its values with the first layer's and has a
    query temperature that steps every 1,024 positions. The feed-forward has 32 experts of an eighth of the size's
    feed-forward width in four groups of which two are kept, four experts per token, and a shared expert of half that
    width: a token passes as many feed-forward weights as in the dense model of that size."""
    L, h, Hq, Hkv, D, I, V, _ = SIZES[size]
    n = layers or L
    ff = max(8, I // 8)
    layer = {"type": "attention",
             "mixer": {"heads": Hq, "kv_heads": Hkv, "dim": D, "vdim": D, "scale": D ** -0.5, "v_mix": True, "q_temp": {"coef": 0.1, "every": 1024}},
             "mlp": {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": max(8, I // 2)},
                     "router": {"experts": 32, "top": 4, "groups": {"count": 4, "keep": 2}}}}
    return NegosunConfig.from_dict({"architecture": "Negosun", "vocab": V, "width": h, "norm": {"eps": 1e-6}, "residual_mult": 0.5,
                                    "logit_softcap": 30.0, "layers": [layer] * n, "max_position_embeddings": 40960}), L


def tavevik_config(size: str, layers: int | None = None):
    """(a Tavevik configuration whose layers resemble that size's: the same width, vocabulary, feed-forward width and
    attention heads, with `layers` layers or as many as the size has; that count). The two layer kinds take turns, the
    second kind first. Attention under a window of 1,024 positions, half of each head's dimensions turning; in the first
    kind 16 kept positions and a cap of 50 on the scores. Beside it a delta rule with a quarter of the attention's heads
    at its head size (half as many key heads, four taps) or a shifted-mix recurrence with heads of 64 over the model's
    width; thin pairs of 64."""
    L, h, Hq, Hkv, D, I, V, _ = SIZES[size]
    n = layers or L
    small = D < 64
    left = lambda first: dict({"heads": Hq, "kv_heads": Hkv, "dim": D, "vdim": D, "scale": D ** -0.5, "rot": {"dims": D // 2, "base": 1e6},
                               "mask": dict({"size": 1024}, **({"keep_first": 16} if first else {}))}, **({"softcap": 50.0} if first else {}))
    rank = 8 if small else 64
    delta_heads = max(2, Hq // 4)
    one = {"type": "parallel", "mlp": {"kind": "dense", "ff": I, "limit": 7.0},
           "mixer": {"left": left(True), "right": {"heads": max(1, h // (16 if small else 64)), "dim": 16 if small else 64, "decay_rank": rank},
                     "left_scale": 0.8, "right_scale": 1.1}}
    two = {"type": "parallel_2", "mlp": {"kind": "dense", "ff": I, "limit": 7.0},
           "mixer": {"left": left(False), "right": {"heads": delta_heads, "kv_heads": delta_heads // 2, "dim": D, "vdim": D, "conv": 4,
                                                    "decay_rank": rank, "gate_rank": rank},
                     "left_scale": 0.6, "right_scale": 0.9}}
    return TavevikConfig.from_dict({"architecture": "Tavevik", "vocab": V, "width": h, "norm": {"eps": 1e-6},
                                    "layers": [two if i % 2 == 0 else one for i in range(n)], "max_position_embeddings": 40960}), L


def goluzen_config(size: str, layers: int | None = None):
    """(a Goluzen configuration whose layers resemble that size's: the same width, vocabulary and attention heads, with
    `layers` layers or as many as the size has; that count). The mixers take turns: attention (a window of 1,024 positions
    with 16 kept ones, half of each head turning under positions stretched fourfold, a cap of 50, sinks), attention over a
    latent of one and a half head sizes with a rotating part of half a head size under a window of 2,048 positions,
    linear attention with a quarter of the heads and values twice as wide as keys, attention again, latent attention on
    the latent of the layer three before it, linear attention. The first layer's feed-forward is dense; the others have 32
    experts of an eighth of the size's feed-forward width in four groups of which two are kept, four experts per token,
    and a shared expert of half that width."""
    L, h, Hq, Hkv, D, I, V, _ = SIZES[size]
    n = layers or L
    small = D < 64
    attention = {"type": "attention",
                 "mixer": {"heads": Hq, "kv_heads": Hkv, "dim": D, "vdim": D, "scale": D ** -0.5, "softcap": 50.0,
                           "rot": {"dims": D // 2, "base": 1e6, "scaling": {"factor": 4.0}}, "mask": {"size": 1024, "keep_first": 16}}}
    latent = lambda src: {"type": "latent_attention",
                          "mixer": dict({"heads": Hq, "dim": D, "rot_dim": D // 2, "vdim": D, "kv_rank": 3 * D // 2, "scale": (3 * D // 2) ** -0.5,
                                         "rot": {"dims": D // 2, "base": 1e6, "scaling": {"factor": 4.0, "original": 8192, "fast": 32.0, "slow": 1.0}},
                                         "mask": {"size": 2048}}, **({} if src is None else {"kv_from": src}))}
    linear = {"type": "gla", "mixer": {"heads": max(1, Hq // 4), "dim": D, "vdim": 2 * D, "tau": 8.0, "decay_rank": 8 if small else 16}}
    moe = {"kind": "moe", "expert": {"ff": max(8, I // 8)}, "shared": {"ff": max(8, I // 2)},
           "router": {"experts": 32, "top": 4, "scale": 2.5, "groups": {"count": 4, "keep": 2}}}
    out, last_own = [], None
    for i in range(n):
        turn = i % 6
        if turn in (0, 3):
            entry = attention
        elif turn in (2, 5):
            entry = linear
        elif turn == 1 or last_own is None:
            entry, last_own = latent(None), i
        else:
            entry = latent(last_own)
        out.append(dict(entry, mlp={"kind": "dense", "ff": I} if i == 0 else moe))
    return GoluzenConfig.from_dict({"architecture": "Goluzen", "vocab": V, "width": h, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
                                    "layers": out, "max_position_embeddings": 40960}), L


DESIGNS = ("sigosun", "negosun", "tavevik", "goluzen")


def named_config(name: str, layers: int | None = None):
    """(configuration, full layer count) of a name the command lines take for random weights: a Qwen3 size
    ("0.6b"), or "<design>:<size>" for one of `DESIGNS` at that size's layer sizes."""
    design, _, size = name.rpartition(":")
    if size not in SIZES or design not in ("", "qwen3") + DESIGNS:
        raise KeyError(f"{name!r} is not one of {sorted(SIZES)}, optionally behind one of {[d + ':' for d in DESIGNS]}")
    if design == "goluzen":
        return goluzen_config(size, layers)
    if design == "negosun":
        return negosun_config(size, layers)
    if design == "tavevik":
        return tavevik_config(size, layers)
    return sigosun_config(size, layers) if design == "sigosun" else model_config(size, layers)
