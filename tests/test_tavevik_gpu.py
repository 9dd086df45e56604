"""Tavevik on the GPU: each new kernel against its plain twin at sizes of its own, then the engine's cuts, batches,
slot and page reuse, long decoding and window edges in float32 and bfloat16 against the plain evaluation, decode steps
replayed as graphs, greedy generation through the scheduler, and the trace program on a folder of this design."""
import pytest
import torch

import helpers
import kernel_twins as twin
import tavevik_cases as C
import test_trace_run as TR
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.kernels import ops
from mini_engine_amd.weights.loader import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 5e-5, torch.bfloat16: 1.2e-1}    # widths of 32-48 make bfloat16 noisy: the plain twins in bfloat16 differ as much (to the digit)


# The configuration of odd sizes (width 36) is ill-conditioned in bfloat16 at single positions: with the attention kernel swapped
# for the exact one, every attention output equal within one rounding (0.002), the logits of one position of 50 move by 0.14.
# Its bfloat16 runs are held to a loose bound; its float32 runs to the same one as every other configuration.
LOOSE_BF16 = {"odd": 2.5e-1}


def hip():
    return ops.HipBackend()


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    assert torch.isfinite(a).all()
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
    assert err <= tol, f"relative error {err:.3g} > {tol:g}"


@pytest.fixture(scope="module")
def tavevik_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = C.make_folder(name, str(tmp_path_factory.mktemp(f"tavevik_{name}")))
        return made[name]

    return get


def _steps_meta(q_lens, slots):
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    seq = torch.repeat_interleave(torch.arange(len(q_lens)), torch.tensor(q_lens)).to(torch.int32).to(DEV)
    return cu, seq, torch.tensor(slots, dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------ kernels against their twins

@pytest.mark.parametrize("groups", [None, (1, False), (4, False), (4, True), (16, True)],
                         ids=["rule", "one-lane", "four-lanes", "four-lanes-prepared", "sixteen-lanes-prepared"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rule,H,G,N,P", [("delta", 4, 2, 20, 12), ("delta", 2, 1, 72, 80), ("delta", 3, 3, 128, 128), ("delta", 2, 2, 64, 64),
                                          ("delta", 1, 1, 200, 7), ("bonus", 3, 3, 12, 12), ("bonus", 2, 2, 64, 64), ("bonus", 1, 1, 130, 130),
                                          ("bonus", 5, 5, 8, 8)])
def test_decay_rows_recurrence(monkeypatch, dtype, rule, H, G, N, P, groups):
    """Requests of unequal lengths from states of their own, against the token-by-token twin; then one request cut in
    three gives what it gives whole. Every form of the kernel: one, four or sixteen lanes to a state column, the tokens'
    values shaped inside the kernel or by a kernel of its own."""
    if groups:
        if groups[0] == 1 and N > 64:
            pytest.skip("a lane keeps up to 64 rows")
        monkeypatch.setattr(ops, "decay_row_groups", lambda *a: groups)
    torch.manual_seed(H * N + P)
    q_lens = [1, 90, 2, 17]
    cu, seq, slots = _steps_meta(q_lens, [2, 0, 4, 1])
    T = sum(q_lens)
    rows = torch.randn(T, 2 * G * N + H * P + H * N + H + 5, device=DEV).to(dtype)
    a = 1
    q, k = rows[:, a:a + G * N], rows[:, a + G * N:a + 2 * G * N]
    a += 2 * G * N
    v, raw, beta = rows[:, a:a + H * P], rows[:, a + H * P:a + H * P + H * N], rows[:, a + H * P + H * N:a + H * P + H * N + H]
    if rule == "delta":
        kw = dict(base=torch.randn(H * N, device=DEV) - 1, rate=torch.rand(H, device=DEV) * 3 + 0.1, beta=beta, unit_eps=1e-6, q_scale=N ** -0.5)
    else:
        kw = dict(base=torch.randn(H * N, device=DEV) - 2, bonus=torch.randn(H * N, device=DEV))
        q, k = q * 0.3, k * 0.3
    full = torch.randn(6, 3 + H * N * P, device=DEV)
    st_h, st_c = full.clone(), full.cpu().clone()
    got = hip().decay_rows_recurrence(q, k, v, raw, st_h[:, 3:], slots, cu, q_lens, H, G, N, P, rule, **kw)
    cpu = lambda t: t.cpu() if torch.is_tensor(t) else t
    want = twin.decay_rows_recurrence(q.cpu(), k.cpu(), v.cpu(), raw.cpu(), st_c[:, 3:], slots.cpu(), cu.cpu(), q_lens, H, G, N, P, rule,
                                      **{n: cpu(t) for n, t in kw.items()})
    close(got, want, 2e-5)
    close(st_h, st_c, 2e-5)
    assert torch.equal(st_h[:, :3], full[:, :3]) and torch.equal(st_h[3], full[3]) and torch.equal(st_h[5], full[5])
    st2 = full.clone()
    lo = 1
    pieces = []
    for n in (40, 1, 49):
        cu1, _, sl1 = _steps_meta([n], [0])
        cut = {n_: (t[lo:lo + n] if n_ == "beta" else t) for n_, t in kw.items()}
        pieces.append(hip().decay_rows_recurrence(q[lo:lo + n], k[lo:lo + n], v[lo:lo + n], raw[lo:lo + n], st2[:, 3:], sl1, cu1, [n],
                                                  H, G, N, P, rule, **cut))
        lo += n
    if groups and groups[1]:          # one kernel shapes every token: the same sums in the same order, however the request is cut
        assert torch.equal(torch.cat(pieces), got[1:91]) and torch.equal(st2[0], st_h[0])
    else:               # other forms for a single token than for a portion, or the shaping unrolled per place in a batch: equal within rounding
        close(torch.cat(pieces), got[1:91], 2e-6)
        close(st2[0], st_h[0], 2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [24, 256, 1000])
def test_token_shift(dtype, n):
    q_lens = [1, 30, 2, 1]
    cu, seq, slots = _steps_meta(q_lens, [3, 0, 1, 4])
    T = sum(q_lens)
    rows = torch.randn(T, n + 16, device=DEV).to(dtype)
    x = rows[:, 8:8 + n]
    mu = torch.rand(5, n, device=DEV)
    full = torch.randn(6, 7 + n, device=DEV).to(torch.bfloat16).float()
    st_h, st_c = full.clone(), full.cpu().clone()
    got = hip().token_shift(x, mu, st_h[:, 7:], slots, cu, seq)
    want = twin.token_shift(x.cpu(), mu.cpu(), st_c[:, 7:], slots.cpu(), cu.cpu(), seq.cpu())
    close(got, want, 1e-6 if dtype == torch.float32 else 8e-3)
    assert torch.equal(st_h.cpu(), st_c)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_elementwise_steps(dtype):
    tol = 1e-6 if dtype == torch.float32 else 8e-3
    rows = (torch.randn(33, 200, device=DEV) * 2).to(dtype)
    close(hip().glu_clamped(rows[:, 8:168], 1.3, 1.702), twin.glu_clamped(rows[:, 8:168], 1.3, 1.702), tol)
    close(hip().activation(rows[:, 17:150], "tanh"), twin.activation(rows[:, 17:150], "tanh"), tol)
    o, want = rows[:, :64].contiguous(), rows[:, :64].contiguous()
    hip().sigmoid_gate_(o, rows[:, 100:164])
    twin.sigmoid_gate_(want, rows[:, 100:164])
    close(o, want, tol)
    bias = torch.randn(120, device=DEV)
    close(hip().add_bias(rows[:, 40:168], bias, dtype), twin.add_bias(rows[:, 40:168], bias, dtype), tol)
    parts = torch.randn(3, 33, 128, device=DEV)
    close(hip().add_bias(parts, bias, dtype), twin.add_bias(parts, bias, dtype), tol)
    y = torch.randn(33, 64, device=DEV)
    gate = rows[:, 100:164]
    w = torch.rand(64, device=DEV) + 0.5
    close(hip().gated_rms_norm(y, gate, w, 1e-5, 4, "silu_behind", dtype), twin.gated_rms_norm(y, gate, w, 1e-5, 4, "silu_behind", dtype), tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,n", [(1, 48), (37, 1000), (300, 256), (5, 3)])
def test_weighted_sum_and_the_norm_on_it(dtype, T, n):
    torch.manual_seed(T + n)
    a = torch.randn(3, T, n, device=DEV)
    b = torch.randn(T, n, device=DEV).to(dtype)
    bias = torch.randn(n, device=DEV)
    terms = [(a, 0.6, None), (b, -1.1, bias)]
    close(hip().weighted_sum(terms), twin.weighted_sum(terms), 1e-6)
    stream, w = torch.randn(T, n, device=DEV) * 3, torch.rand(n, device=DEV) + 0.5
    lo, new = hip().weighted_sum(terms, w, 1e-5, stream, dtype)
    lo_t, new_t = twin.weighted_sum(terms, w, 1e-5, stream, dtype)
    close(new, new_t, 2e-6)
    assert lo.dtype == dtype and torch.equal(lo.float(), new.to(dtype).float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D,page,window,keep,cap,sink", [(16, 8, 6, 3, 3.0, False), (48, 16, 40, 0, None, True), (64, 16, 33, 70, 10.0, True),
                                                         (128, 16, 300, 5, 50.0, False), (96, 8, 17, 0, None, True), (128, 32, 256, 0, None, True)])
def test_attention_with_kept_keys_cap_and_sinks(dtype, D, page, window, keep, cap, sink):
    """Prompts, portions behind a prefix and single tokens in one step, against the twin that gathers exactly the keys the
    mask lets through; in bfloat16 whichever kernel the rule picks."""
    torch.manual_seed(D + window)
    Hq, Hkv = 6, 2
    ctx = [350, 40, 1, 401, 9, 333]                # two single tokens first, then prompts and portions
    new = [1, 1, 1, 401, 9, 120]
    B = len(ctx)
    pages_per = [-(-c // page) for c in ctx]
    total = sum(pages_per)
    kc = (torch.randn(total + 1, Hkv, page, D, device=DEV)).to(dtype)
    vc = (torch.randn(total + 1, Hkv, D, page, device=DEV)).to(dtype)
    bt = torch.full((B, max(pages_per)), -1, dtype=torch.int32, device=DEV)
    order = torch.randperm(total)
    at = 0
    for b, n in enumerate(pages_per):
        bt[b, :n] = order[at:at + n].to(torch.int32).to(DEV)
        at += n
    positions = torch.cat([torch.arange(c - n, c) for c, n in zip(ctx, new)]).to(torch.int32).to(DEV)
    seq = torch.cat([torch.full((n,), b) for b, n in enumerate(new)]).to(torch.int32).to(DEV)
    T = sum(new)
    q = (torch.randn(T, Hq * D, device=DEV) * 2).to(dtype)
    lens = torch.tensor(ctx, dtype=torch.int32, device=DEV)
    cu = torch.tensor([0, 401, 410, 530], dtype=torch.int32, device=DEV)
    sinks = torch.randn(Hq, device=DEV) + 1.0 if sink else None
    args = (q, kc, vc, page, bt, lens, seq, positions, cu, 3, max(ctx[:3]), D ** -0.5, window, Hq, Hkv, D)
    got = hip().paged_attention(*args, max_prefill_context=max(ctx), keep_first=keep, softcap=cap, sinks=sinks)
    want = twin.paged_attention(*args, keep_first=keep, softcap=cap, sinks=sinks)
    close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


# ------------------------------------------------------------------ the engine against the plain evaluation

class Env:
    device = DEV

    def __init__(self, folders, dtype, graphs=False):
        self.folders, self.dtype, self.tol, self.graphs, self.models = folders, dtype, TOL[dtype], graphs, {}

    def runner(self, name, pages, slots):
        folder = self.folders(name)
        self.tol = LOOSE_BF16.get(name, TOL[self.dtype]) if self.dtype == torch.bfloat16 else TOL[self.dtype]
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 1024)
        model = self.models[name]
        manager = CacheManager(pages, C.PAGE[name], ModelRunner.windows_of(model), num_state_slots=slots, enable_prefix_caching=False)
        options = dict(use_graphs=True, mixed_graphs_after=1) if self.graphs else {}
        return ModelRunner(model, manager, self.dtype, self.device, 1024, poison_cache=True, **options), manager, folder


@pytest.fixture(scope="module", params=[torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def env(request, tavevik_folders):
    return Env(tavevik_folders, request.param)


@pytest.mark.parametrize("name", ["pair", "order", "one", "two", "odd"])
@pytest.mark.parametrize("case", C.ALL, ids=lambda c: c.__name__)
def test_cuts(env, case, name):
    case(env, name)


def test_far_keys_and_window_edges(env):
    C.window_edges(env)


def test_real_layer_sizes(tavevik_folders):
    C.real_sizes(Env(tavevik_folders, torch.float32), Env(tavevik_folders, torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("case", [C.token_by_token, C.long_decode, C.batch_against_alone], ids=lambda c: c.__name__)
def test_cuts_through_captured_steps(tavevik_folders, case, dtype):
    """The same with decode steps (and small steps that come up again) replayed as graphs: state slots travel with the
    step's metadata, fresh slots are zeroed outside the graph."""
    case(Env(tavevik_folders, dtype, graphs=True), "pair")


def test_hip_libraries_are_the_ones_running(env):
    C.whole(env, "one")
    assert ops.backend().name == "hip" and any("libme_core" in p for p in ops.loaded_libraries())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["pair", "order"])
def test_greedy_generation_through_the_scheduler(tavevik_folders, dtype, name):
    C.greedy_through_the_engine(DEV, dtype, name, tavevik_folders(name), exact=dtype == "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_program_on_this_design(tavevik_folders, tmp_path, dtype):
    """bin/trace_run picks the model class by the folder's config: four live requests, portions beside single tokens,
    state slots and pages used again."""
    name = "order"
    folder = tavevik_folders(name)
    V = C.CONFIGS[name]["vocab"]
    lens = {"a": 100, "b": 64, "c": 30, "d": 77, "e": 50}
    ids = {r: helpers.random_ids(n, V, 900 + i) for i, (r, n) in enumerate(lens.items())}
    schedule = helpers.cuts_schedule({r: lens[r] for r in ("a", "b", "c", "d")}, [19, 1, 1, 2, 33, 1, 7, 1])
    steps = TR.steps_from_schedule(ids, schedule)
    last_c = max(i for i, st in enumerate(schedule) if "c" in st)
    for j, st in enumerate(helpers.cuts_schedule({"e": lens["e"]}, [5, 1, 40, 1])):
        a, b = st["e"]
        entry = {"id": "e", "tokens": ids["e"][a:b], "want": list(range(b - a))}
        i = last_c + 1 + j
        if i < len(steps):
            steps[i]["entries"].append(entry)
            if b == lens["e"]:
                steps[i]["end"].append("e")
        else:
            steps.append({"step": i, "entries": [entry], "end": ["e"] if b == lens["e"] else []})
    out = str(tmp_path / "o")
    TR.replay(folder, dtype, steps, out, max_tokens=TR.most_live_tokens(steps), page=C.PAGE[name])
    for r, g in TR.collect(steps, out, V).items():
        err = helpers.rel_err(g, C.plain_logits(folder, ids[r]))
        assert err <= TOL[getattr(torch, dtype)], f"{dtype} request {r}: {err:.3g}"


def test_offline_workload_row_with_random_weights(tmp_path, capsys):
    """The offline workload through the command line, on this design at a tiny size with random weights."""
    import json
    from mini_engine_amd import cli
    rc = cli.main(["--random-weights", "tavevik:tinyA", "--num-seqs", "6", "--max-prompt", "40", "--max-output", "8",
                   "--max-model-len", "64", "--max-num-seqs", "4", "--budget", "32", "--tokens-out", "-",
                   "--out", str(tmp_path / "bench.jsonl")])
    assert rc == 0
    lines = capsys.readouterr().out.strip().splitlines()
    row = json.loads(lines[-1])
    tokens = [json.loads(line) for line in lines[-7:-1]]
    assert [len(t) for t in tokens] == [8] * 6 and all(0 <= t < 256 for ts in tokens for t in ts)
    assert row["num_seqs"] == 6 and row["output_tokens"] == 48 and row["throughput_tok_s"] > 0
