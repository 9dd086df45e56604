"""The Tavevik design in the engine against its plain evaluation (tests/plain_tavevik.py), under every way of cutting
the work. Each case takes `env` with .device, .dtype, .tol and .runner(name, pages, slots) -> (runner, manager,
folder); the same cases run on the CPU (plain kernel twins, float32) and on the GPU (HIP kernels, float32 and
bfloat16). Pools start filled with NaN, so a read of a key or state nobody wrote poisons the logits.

The configurations are the tests' own and differ from each other in every size: both layer kinds in several orders,
layers without a feed-forward, windows of 5 to 300 positions with 0 to 12 kept first positions (more kept than the
window is long, too), rotations of a whole head and of a part, key sizes that differ from value sizes, grouped
key/value heads on both sides, states above and below a wave's 64 rows, value sizes above 64, convolutions of 1 to 4
taps, thin matrix pairs of 8 to 24. The stored q norms are scaled up so that the softmax is peaked, sinks and biases so
that leaving one out moves the logits far beyond the tolerance, the embedding's rows to the size of the sublayers' outputs.
"""
from __future__ import annotations

import os

import torch

import helpers
import plain_tavevik
from helpers import Driver, random_ids, rel_err
from mini_engine_amd.config.model_config import TavevikConfig
from mini_engine_amd.weights.random_init import write_random_model


def _left(heads, kv, dim, vdim, scale, rot, base, size, keep=None, cap=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size}}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    if keep:
        m["mask"]["keep_first"] = keep
    if cap:
        m["softcap"] = cap
    return m


def _one(left, heads, dim, rank, ls=0.7, rs=1.2, ff=None, limit=2.0):
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": heads, "dim": dim, "decay_rank": rank},
                                          "left_scale": ls, "right_scale": rs},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def _two(left, heads, kv, dim, vdim, conv, rank_a, rank_g, ls=1.3, rs=0.5, ff=None, limit=1.5):
    return {"type": "parallel_2", "mixer": {"left": left, "right": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv,
                                                                    "decay_rank": rank_a, "gate_rank": rank_g},
                                            "left_scale": ls, "right_scale": rs},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def _model(vocab, width, eps, layers):
    return {"architecture": "Tavevik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


CONFIGS = {
    # the second kind first; grouped heads on both sides; a part of each head turns; four taps
    "pair": _model(101, 48, 1e-5, [
        _two(_left(4, 2, 24, 16, 0.2, 8, 5000.0, 7), 4, 2, 20, 12, 4, 8, 16, ff=80),
        _one(_left(3, 3, 16, 24, 0.3, 16, 20000.0, 9, keep=3, cap=4.0), 3, 12, 8, ff=56, limit=0.2),
    ]),
    # three layers of the first kind and one of the second, two without feed-forward; more kept positions than the window is
    # long; a layer without a cap and without kept positions; one key head for three heads on the right; two taps
    "order": _model(77, 40, 1e-6, [
        _one(_left(2, 1, 32, 8, 0.15, 16, 1e4, 5, keep=12, cap=2.5), 5, 8, 16),
        _one(_left(4, 4, 8, 8, 0.4, 0, 1.0, 11), 2, 20, 8, ff=64),
        _two(_left(6, 2, 16, 16, 0.25, 16, 3e5, 13), 3, 1, 16, 24, 2, 24, 8),
        _one(_left(2, 2, 16, 32, 0.2, 4, 777.0, 6, keep=1, cap=30.0), 1, 40, 8, ff=48, limit=5.0),
    ]),
    # each kind alone; a convolution of one tap (no inputs to carry)
    "one": _model(64, 32, 1e-6, [_one(_left(6, 2, 16, 16, 0.25, 8, 1e4, 6, keep=2, cap=3.0), 4, 8, 8, ff=48)]),
    "two": _model(64, 32, 1e-5, [_two(_left(3, 1, 16, 32, 0.25, 16, 1e4, 5), 2, 2, 8, 16, 1, 8, 8, ff=40)]),
    # sizes in no whole steps of 8: a width of 36, thin pairs of 12 and 20, head sizes of 40 and 24, an odd vocabulary, five
    # heads on one key head, a state of 96 x 20
    "odd": _model(131, 36, 1e-5, [
        _two(_left(5, 1, 40, 24, 0.16, 10, 1234.5, 19), 3, 1, 96, 20, 3, 12, 20, ff=52),
        _one(_left(2, 1, 24, 40, 0.2, 24, 9e4, 4, keep=9), 3, 20, 12, ff=44, limit=3.0),
    ]),
    # windows of hundreds of positions: keys far back; states of 72 and 80 rows (four lanes to a column), values of 80
    "far": _model(80, 32, 1e-5, [
        _one(_left(3, 1, 32, 16, 0.2, 32, 4e5, 300, keep=4, cap=20.0), 1, 72, 8, ff=40),
        _two(_left(2, 2, 16, 16, 0.25, 8, 4e5, 150), 2, 1, 80, 80, 3, 8, 8),
    ]),
}
# the layer sizes of a real model (heads of 128 and 64, windows of 256 and 128, states of 64 x 64 and 128 x 128), few layers
CONFIGS["real"] = _model(1000, 512, 1e-6, [
    _two(_left(8, 2, 128, 128, 128 ** -0.5, 64, 1e6, 256), 4, 2, 128, 128, 4, 32, 32, ff=1024, limit=7.0),
    _one(_left(8, 4, 64, 64, 0.125, 64, 1e6, 128, keep=16, cap=50.0), 8, 64, 32, ff=1024, limit=7.0),
])
SEEDS = {"pair": 21, "order": 22, "one": 23, "two": 24, "far": 25, "real": 26, "odd": 27}
PAGE = {"pair": 8, "order": 16, "one": 16, "two": 8, "far": 16, "real": 16, "odd": 8}
SHARPEN = 3.0


def make_folder(name: str, path: str) -> str:
    """A model folder with seeded random weights; q norms scaled up by SHARPEN, sinks set to 1..3 (a softmax over a
    few peaked scores then loses a third to a half of its mass to the sink), biases ten times as large as drawn."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    write_random_model(TavevikConfig.from_dict(CONFIGS[name]), SEEDS[name], path, torch.bfloat16)
    file = os.path.join(path, "model.safetensors")
    with safe_open(file, "pt", device="cpu") as f:
        tensors = {k: f.get_tensor(k) for k in f.keys()}
    for k in tensors:
        t = tensors[k].float()
        if k.endswith(".left.q.norm"):
            t = t * SHARPEN
        elif k.endswith(".left.sink"):
            t = 1.0 + 2.0 * torch.arange(t.numel(), dtype=torch.float32) / max(1, t.numel() - 1) if t.numel() > 1 else t + 2.0
        elif k.endswith(".b") and ".left." in k:
            t = t * 10.0
        elif k == "embed":
            t = t * 20.0          # rows of a size near the sublayers' normed outputs, as in a trained model: in bfloat16 a
                                  # stream that starts a fiftieth of that size makes single positions noisy beyond any tolerance
        tensors[k] = t.to(tensors[k].dtype)
    save_file(tensors, file, metadata={"format": "pt"})
    return path


_plain: dict = {}


def plain_model(folder: str):
    if folder not in _plain:
        _plain[folder] = plain_tavevik.read_folder(folder)
    return _plain[folder]


def plain_logits(folder: str, ids: list) -> torch.Tensor:
    key = (folder, tuple(ids))
    if key not in _plain:
        cfg, w = plain_model(folder)
        _plain[key] = plain_tavevik.logits(cfg, w, ids)
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
    """Portions of changing size, down to two tokens and one, cut inside pages, windows, the kept positions and the
    convolution's reach."""
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
    """A short prompt, then many single tokens: over page borders, many windows long, far beyond the convolution's reach,
    with the pages behind the windows given back on the way (all but those of the kept positions)."""
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


def real_sizes(env_f32, env_bf16, name="real"):
    """At the layer sizes of a real model: float32 against the plain evaluation on a short prompt; then a prompt of 600
    tokens whole, in portions and with its last tokens decoded, bfloat16 against float32 of the same engine."""
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
    assert rel_err(wb, wf.double().cpu()) <= env_bf16.tol and rel_err(rb, wf.double().cpu()) <= env_bf16.tol


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
