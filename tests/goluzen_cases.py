"""The Goluzen design in the engine against its plain evaluation (tests/plain_goluzen.py), under every way of cutting
the work. Each case takes `env` with .device, .dtype, .tol and .runner(name, pages, slots) -> (runner, manager,
folder); the same cases run on the CPU (plain kernel twins, float32) and on the GPU (HIP kernels, float32 and
bfloat16). Pools start filled with NaN, so a read of a key or state nobody wrote poisons the logits.

The configurations are the tests' own and differ from each other in every size: the three mixers in several orders,
a latent layer that reads the latent of an earlier one under a window of its own, layers without a feed-forward,
dense and routed feed-forwards with and without groups, with and without a shared expert, windows of 5 to 300
positions with 0 to 12 kept first positions, rotations of a whole head and of a part, stretched and not, sizes that
are no whole steps of 8, single heads, one expert per token. Score scales are large, so that the softmax is peaked
and a key that is wrongly seen or missed moves the logits; sinks, biases, corrections and routers are scaled up so
that leaving one out moves them far beyond the tolerance.
"""
from __future__ import annotations

import os

import torch

import helpers
import plain_goluzen
from helpers import Driver, random_ids, rel_err
from mini_engine_amd.config.model_config import GoluzenConfig
from mini_engine_amd.weights.random_init import write_random_model


def _attention(heads, kv, dim, vdim, scale, rot=None, base=10000.0, factor=None, size=None, keep=None, cap=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
        if factor:
            m["rot"]["scaling"] = {"factor": factor}
    if size:
        m["mask"] = {"size": size}
        if keep:
            m["mask"]["keep_first"] = keep
    if cap:
        m["softcap"] = cap
    return {"type": "attention", "mixer": m}


def _latent(heads, dim, rot_dim, vdim, rank, scale, base=10000.0, yarn=None, size=None, src=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": {"dims": rot_dim, "base": base}}
    if yarn:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), yarn))
    if size:
        m["mask"] = {"size": size}
    if src is not None:
        m["kv_from"] = src
    return {"type": "latent_attention", "mixer": m}


def _gla(heads, dim, vdim, tau, rank):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": rank}}


def _moe(ff, experts, top, scale=None, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if scale is not None:
        router["scale"] = scale
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _with(layer, mlp):
    return dict(layer, mlp=mlp)


def _model(vocab, width, eps, layers, scale=None):
    d = {"architecture": "Goluzen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if scale is not None:
        d["embedding"] = {"scale": scale}
    return d


CONFIGS = {
    # linear attention first; a latent layer and, two layers on, one that reads its latent under a shorter window; grouped heads
    "mix": _model(101, 48, 1e-5, [
        _with(_gla(3, 8, 16, 8.0, 8), _dense(80)),
        _with(_latent(4, 16, 8, 24, 40, 0.9, 5000.0, (4.0, 32, 8.0, 1.0), 9), _moe(24, 8, 2, 1.5, (4, 2), 40)),
        _with(_attention(4, 2, 16, 24, 1.4, 8, 5000.0, 2.0, 7, 3, 6.0), _moe(24, 8, 3, 2.0, (2, 1), 32)),
        _with(_latent(2, 24, 8, 16, 40, 0.8, 5000.0, (4.0, 32, 8.0, 1.0), 5, src=1), _moe(16, 4, 2)),
    ], 6.0),
    # sizes in no whole steps of 8; a layer without a feed-forward; a latent read under a longer window than its owner's;
    # more kept positions than the window is long; routed experts without a shared one
    "odd": _model(97, 36, 1e-6, [
        _with(_latent(3, 12, 6, 10, 20, 1.1, 300.0, (2.0, 16, 4.0, 1.0), 6), None),
        _with(_attention(3, 3, 20, 12, 1.2, 10, 300.0, 3.0, 4, 6, 9.0), _moe(20, 6, 3, 0.7, (3, 2))),
        _with(_gla(2, 10, 14, 3.0, 5), _dense(44)),
        _with(_latent(2, 10, 6, 14, 20, 1.3, 300.0, (2.0, 16, 4.0, 1.0), 11, src=0), _moe(12, 6, 2, 1.2, (2, 2), 20)),
        _with(_attention(2, 1, 12, 20, 1.5, 12, 300.0, None, 8), _dense(40)),
    ], 4.0),
    # what a model may make equal or one: one head, one expert per token, all groups kept, nothing kept behind the window,
    # no cap, no stretch, every dimension turning, attention over everything, a temperature of one, no embedding scale
    "one": _model(64, 32, 1e-5, [
        _with(_attention(1, 1, 16, 16, 1.6, 16, 100.0), _moe(16, 4, 1, None, (2, 2), None)),
        _with(_latent(1, 8, 8, 8, 16, 1.0, 100.0), _dense(32)),
        _with(_gla(1, 16, 16, 1.0, 4), _moe(16, 2, 1)),
        _with(_attention(2, 2, 8, 8, 1.8, 4, 100.0, None, 5), None),
    ]),
    # a width in whole 16-byte pieces around sizes that are not (the kernels' vector paths beside their scalar ones in one
    # model); two latents of different sizes, each with a reader; two experts kept of two
    "mid": _model(120, 64, 1e-5, [
        _with(_latent(3, 10, 6, 14, 22, 1.0, 700.0, (3.0, 24, 6.0, 1.0), 12), _moe(24, 2, 2, 1.1, None, 16)),
        _with(_latent(2, 16, 8, 8, 24, 0.9, 900.0, None, 7), _dense(72)),
        _with(_gla(3, 6, 10, 5.0, 3), _moe(12, 9, 4, 0.9, (3, 2), 28)),
        _with(_latent(5, 10, 6, 6, 22, 1.2, 700.0, (3.0, 24, 6.0, 1.0), 30, src=0), None),
        _with(_attention(6, 2, 12, 10, 1.3, 6, 700.0, 2.5, 9, 2, 7.0), _dense(40)),
        _with(_latent(1, 16, 8, 24, 24, 1.1, 900.0, None, None, src=1), _moe(16, 4, 2, 1.3, (2, 1))),
    ], 3.0),
    # nothing but linear attention: a model without any pages
    "flat": _model(50, 24, 1e-5, [
        _with(_gla(2, 4, 6, 2.0, 3), _dense(32)),
        _with(_gla(1, 12, 8, 6.0, 4), None),
    ]),
    # long windows with few kept positions: keys hundreds of positions back
    "far": _model(80, 32, 1e-5, [
        _with(_attention(2, 1, 16, 16, 1.5, 8, 50000.0, 4.0, 300, 4, 20.0), _dense(48)),
        _with(_latent(2, 8, 8, 8, 24, 1.2, 50000.0, (4.0, 64, 16.0, 1.0), 150), _moe(16, 4, 2, 1.5, (2, 1), 16)),
        _with(_gla(2, 8, 8, 32.0, 4), None),
    ], 5.0),
    # the layer sizes of a real model (GPU only): heads of 128, a latent of 192 + 64, states of 128 x 256; every token takes
    # all 8 experts, so that no choice can fall otherwise in bfloat16 than in float32 and every row can be held to the tolerance
    "real": _model(2048, 1024, 1e-6, [
        _with(_attention(16, 8, 128, 128, 128 ** -0.5 * 4, 64, 1e6, 4.0, 256, 16, 50.0), _dense(3072)),
        _with(_latent(16, 128, 64, 128, 192, 192 ** -0.5 * 2, 1e6, (4.0, 8192, 32.0, 1.0), 384), _moe(384, 8, 8, 0.6, (2, 2), 1536)),
        _with(_gla(4, 128, 256, 8.0, 16), _moe(384, 8, 8, 0.6, (2, 2), 1536)),
        _with(_latent(16, 128, 64, 128, 192, 192 ** -0.5 * 2, 1e6, (4.0, 8192, 32.0, 1.0), 128, src=1), _moe(384, 8, 8, 0.6, None, 1536)),
    ], 8.0),
    # the same with 4 of 32 experts per token: a token whose choice hangs on two scores closer than bfloat16's rounding of the
    # router's input may choose otherwise in bfloat16 (a tenth of the rows do), so these rows are held to the tolerance in the mean
    "routed": _model(2048, 1024, 1e-6, [
        _with(_attention(16, 8, 128, 128, 128 ** -0.5 * 4, 64, 1e6, 4.0, 256, 16, 50.0), _dense(3072)),
        _with(_latent(16, 128, 64, 128, 192, 192 ** -0.5 * 2, 1e6, (4.0, 8192, 32.0, 1.0), 384), _moe(384, 32, 4, 2.5, (4, 2), 1536)),
        _with(_gla(4, 128, 256, 8.0, 16), _moe(384, 32, 4, 2.5, (4, 2), 1536)),
    ], 8.0),
}
SEEDS = {"mix": 31, "odd": 32, "one": 33, "far": 34, "real": 35, "routed": 36, "mid": 37, "flat": 38}
PAGE = {"mix": 16, "odd": 8, "one": 4, "far": 16, "real": 16, "routed": 16, "mid": 32, "flat": 16}
SMALL = ("mix", "odd", "one", "mid", "flat")


def make_folder(name: str, path: str) -> str:
    """A checkpoint of the configuration with seeded random weights in bfloat16, reshaped so that every mechanism
    shows: the latent layers' queries and keys large enough for a peaked softmax, sinks of 1 to 3, biases and
    corrections ten times as large as drawn, routers so that their logits are a few units (scores spread over the sigmoid's range), the decay's
    thin pair ten times (decays that differ from token to token), the embedding's rows of a size near the sublayers'
    outputs."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    cfg = GoluzenConfig.from_dict(CONFIGS[name])
    write_random_model(cfg, SEEDS[name], path, torch.bfloat16)
    file = os.path.join(path, "model.safetensors")
    with safe_open(file, "pt", device="cpu") as f:
        tensors = {k: f.get_tensor(k) for k in f.keys()}
    # (at the widths of a real model the drawn weights give scores of that size by themselves)
    latent = {f"l{i}." for i, layer in enumerate(cfg.layers) if layer.kind == "latent_attention" and cfg.hidden_size < 256}
    for k in tensors:
        t = tensors[k].float()
        if k.partition(".")[0] + "." in latent and k.endswith((".mix.q", ".mix.uk", ".mix.dkv")):
            t = t * {"q": 30.0, "uk": 5.0, "dkv": 8.0}[k.rsplit(".", 1)[1]]       # scores of a few units: a peaked softmax
        elif k.endswith(".sink"):
            t = 1.0 + 2.0 * torch.arange(t.numel(), dtype=torch.float32) / max(1, t.numel() - 1) if t.numel() > 1 else t + 2.0
        elif k.endswith(".b") and not k.endswith(".a2.b"):
            t = t * 10.0
        elif k.endswith(".correction"):
            t = t * 10.0
        elif k.endswith(".router") or k.endswith(".sg"):
            t = t * 2.5 / (0.02 * cfg.hidden_size ** 0.5)      # logits of a few units whatever the width
        elif k.endswith(".a2"):
            t = t * 10.0
        elif k == "embed":
            t = t * 20.0 / cfg.embedding_scale
        tensors[k] = t.to(tensors[k].dtype)
    save_file(tensors, file, metadata={"format": "pt"})
    return path


_plain: dict = {}


def plain_model(folder: str):
    if folder not in _plain:
        _plain[folder] = plain_goluzen.read_folder(folder)
    return _plain[folder]


def plain_logits(folder: str, ids: list) -> torch.Tensor:
    key = (folder, tuple(ids))
    if key not in _plain:
        cfg, w = plain_model(folder)
        _plain[key] = plain_goluzen.logits(cfg, w, ids)
    return _plain[key]


def _free_pages(manager) -> int:
    return min((manager.num_free_pages(g) for g in range(manager.num_groups)), default=1 << 30)


def _vocab(name):
    return CONFIGS[name]["vocab"]


def _check(env, folder, ids, got, what):
    ref = plain_logits(folder, ids)[: got.shape[0]]
    err = rel_err(got, ref)
    assert err <= env.tol, f"{what}: error {err:.3g} > {env.tol:g}; first bad position {helpers.first_bad_row(got, ref, env.tol)}"


def whole(env, name):
    """Each request alone and whole: one token, two, lengths around pages, windows and kept positions."""
    page = PAGE[name]
    for n in (1, 2, page, page + 1, 21, 50, 83):
        runner, manager, folder = env.runner(name, -(-n // page), 1)
        ids = random_ids(n, _vocab(name), 100 + n)
        d = Driver(runner, manager)
        d.step({"r": ids}, end=["r"])
        _check(env, folder, ids, d.result("r"), f"{name} whole n={n}")


def token_by_token(env, name):
    """A whole request decoded one token at a time from its first token, beside the same request in one step."""
    page = PAGE[name]
    n = 45
    ids = random_ids(n, _vocab(name), 200)
    runner, manager, folder = env.runner(name, 2 * -(-n // page), 2)
    d = Driver(runner, manager)
    for t in range(n):
        d.step({"r": ids[t:t + 1]})
    d.step({"w": ids})
    _check(env, folder, ids, d.result("r"), f"{name} token by token")
    _check(env, folder, ids, d.result("w"), f"{name} whole beside it")


def portions(env, name):
    """Portions of changing size, down to two tokens and one, cut inside pages, windows and the kept positions."""
    page = PAGE[name]
    n = 90
    ids = random_ids(n, _vocab(name), 300)
    for pattern in ([2, 3, 5, 8, 13, 21, 2, 2], [17, 2, 1, 1, 2, 31, 2], [page, 2, page + 1, page - 1]):
        runner, manager, folder = env.runner(name, -(-n // page), 1)
        d = Driver(runner, manager)
        pos, i = 0, 0
        while pos < n:
            c = min(pattern[i % len(pattern)], n - pos)
            d.step({"r": ids[pos:pos + c]})
            pos += c; i += 1
        _check(env, folder, ids, d.result("r"), f"{name} portions {pattern}")


def batch_against_alone(env, name):
    """Unequal requests in one batch, portions beside single tokens, against the plain evaluation of each alone; pages
    and state slots of ended requests are taken by later ones while others are live."""
    page = PAGE[name]
    V = _vocab(name)
    lens = {"a": 40, "b": 23, "c": 9, "d": 61, "e": 30, "f": 1, "g": 17}
    ids = {r: random_ids(n, V, 400 + i) for i, (r, n) in enumerate(lens.items())}
    need = lambda r: -(-lens[r] // page)
    runner, manager, folder = env.runner(name, need("a") + need("d") + need("e"), 3)
    d = Driver(runner, manager)
    waiting, live, pos = list(lens), [], {}
    patterns = {"a": [11, 2, 9], "b": [23], "c": [2, 2, 5], "d": [7, 16, 3, 20], "e": [30], "f": [1], "g": [5, 12]}
    step_no = 0
    while waiting or live:
        while waiting and len(live) < 3 and _free_pages(manager) >= need(waiting[0]) and len(manager.free_slots) > 0:
            r = waiting.pop(0)
            live.append(r); pos[r] = 0
            manager.allocate(r, 0, 0)          # takes its state slot now, pages as it goes
        parts, ended = {}, []
        for r in live:
            plan, acc, take = patterns[r], 0, 1
            for c in plan:
                if acc == pos[r]:
                    take = c
                    break
                acc += c
            take = min(take, lens[r] - pos[r])
            if (step_no + len(r)) % 5 == 4 and pos[r] > 0:
                continue                          # a request may sit a step out
            parts[r] = ids[r][pos[r]:pos[r] + take]
            pos[r] += take
            if pos[r] == lens[r]:
                ended.append(r)
        step_no += 1
        if parts:
            d.step(parts, end=ended)
            for r in ended:
                live.remove(r)
    for r in lens:
        _check(env, folder, ids[r], d.result(r), f"{name} request {r} in the batch")
    assert len(manager.free_slots) == 3


def long_decode(env, name):
    """A short prompt, then many single tokens: over page borders, many windows long, with the pages behind the windows
    given back on the way (all but those of the kept positions)."""
    page = PAGE[name]
    n = 140
    ids = random_ids(n, _vocab(name), 500)
    runner, manager, folder = env.runner(name, -(-n // page), 1)
    d = Driver(runner, manager)
    d.step({"r": ids[:6]})
    for t in range(6, n):
        d.step({"r": ids[t:t + 1]})
    _check(env, folder, ids, d.result("r"), f"{name} long decode")


def slots_start_from_zero(env, name):
    """A request that takes over the state slot and the pages of one that has ended starts from nothing."""
    page = PAGE[name]
    V = _vocab(name)
    runner, manager, folder = env.runner(name, 4, 1)
    d = Driver(runner, manager)
    for i, n in enumerate((4 * page, 3, 2 * page + 1, 1)):
        ids = random_ids(n, V, 700 + i)
        d.step({f"r{i}": ids[:n // 2 + 1]})
        if n // 2 + 1 < n:
            d.step({f"r{i}": ids[n // 2 + 1:]}, end=[f"r{i}"])
        else:
            manager.free(f"r{i}")
        _check(env, folder, ids, d.result(f"r{i}"), f"{name} request {i} in a used slot")


def window_edges(env, name="far"):
    """Windows of 300 and 150 positions with 4 kept ones: queries whose best key lies hundreds of positions back, in a
    prompt, in a portion behind a long prefix and decoded alone; around the windows' edges (positions 149-151, 299-304)
    a key must vanish exactly one position behind the window, and the kept ones never."""
    page = PAGE[name]
    n = 330
    ids = random_ids(n, _vocab(name), 600)
    runner, manager, folder = env.runner(name, 2 * -(-n // page), 2)
    d = Driver(runner, manager)
    d.step({"w": ids})
    d.step({"r": ids[:147]})
    for t in range(147, 153):
        d.step({"r": ids[t:t + 1]})
    d.step({"r": ids[153:290]})
    d.step({"r": ids[290:298]})
    for t in range(298, 306):
        d.step({"r": ids[t:t + 1]})
    d.step({"r": ids[306:]})
    _check(env, folder, ids, d.result("w"), f"{name} whole")
    _check(env, folder, ids, d.result("r"), f"{name} cut around the windows' edges")


def real_sizes(env_f32, env_bf16, name="real", every_row=True):
    """At the layer sizes of a real model: float32 against the plain evaluation on a short prompt; then a prompt of 600
    tokens whole, in portions and with its last tokens decoded, bfloat16 against float32 of the same engine: every row
    within the tolerance, or (a model whose tokens choose among experts) the rows' mean within half of it and their
    median within a quarter."""
    page = PAGE[name]
    V = _vocab(name)
    short = random_ids(40, V, 900)
    runner, manager, folder = env_f32.runner(name, 8, 1)
    d = Driver(runner, manager)
    d.step({"s": short[:33]})
    d.step({"s": short[33:34]})
    d.step({"s": short[34:]}, end=["s"])
    _check(env_f32, folder, short, d.result("s"), f"{name} short prompt in float32")
    n = 600
    ids = random_ids(n, V, 901)
    got = {}
    for env in (env_f32, env_bf16):
        runner, manager, folder = env.runner(name, 2 * -(-n // page), 2)
        d = Driver(runner, manager)
        d.step({"w": ids})
        d.step({"r": ids[:300]})
        d.step({"r": ids[300:302]})
        d.step({"r": ids[302:580]})
        for t in range(580, n):
            d.step({"r": ids[t:t + 1]})
        got[env.dtype] = (d.result("w"), d.result("r"))
    (wf, rf), (wb, rb) = got[torch.float32], got[torch.bfloat16]
    assert rel_err(rf, wf.double().cpu()) <= 1e-4, "float32: the cut request differs from the whole one"
    wide = wf.double().cpu()
    for got_b, what in ((wb, "whole"), (rb, "cut")):
        if every_row:
            assert rel_err(got_b, wide) <= env_bf16.tol, f"bfloat16 {what}"
        row_err = (got_b.double().cpu() - wide).abs().amax(-1) / wide.abs().max()
        assert float(row_err.mean()) <= env_bf16.tol / 2 and float(row_err.median()) <= env_bf16.tol / 4, f"bfloat16 {what}: rows in the mean"


ALL = [whole, token_by_token, portions, batch_against_alone, long_decode, slots_start_from_zero]


def greedy_through_the_engine(device, dtype_name, name, folder, exact: bool):
    """Greedy generation through `LLM.generate`: the scheduler admits under a token budget, cuts prompts, batches
    portions beside decoding requests, takes and gives back pages and state slots; decode steps go through the
    fixed layouts (captured as graphs on a GPU) and run one ahead."""
    from mini_engine_amd import LLM, SamplingParams
    V = _vocab(name)
    prompts = [random_ids(n, V, 800 + n) for n in (30, 12, 9, 1, 21)]
    llm = LLM(folder, dtype=dtype_name, device=device, kvcache_block_size=PAGE[name], num_kvcache_blocks=24, max_num_seqs=3,
              max_num_batched_tokens=16, max_model_len=64, poison_cache=True)
    assert llm.manager.num_state_slots == 3
    outs = llm.generate(prompts, SamplingParams(temperature=0, max_tokens=12, ignore_eos=True), use_tqdm=False)
    assert llm.runner.graphs is not None and llm.runner.graphs.replays > 0, "no decode step went through the fixed-layout path"
    llm.manager.check_invariants()
    assert len(llm.manager.free_slots) == 3 and _free_pages(llm.manager) == 24
    for p, o in zip(prompts, outs):
        seq = list(p)
        assert len(o["token_ids"]) == 12
        for tok in o["token_ids"]:
            z = plain_logits(folder, seq)[-1]
            best = int(z.argmax())
            close = not exact and float(z[best] - z[tok]) < 8e-2 * float(z.abs().max())
            assert tok == best or close, f"{name} {dtype_name}: generated {tok}, the plain evaluation gives {best}"
            seq.append(tok)
