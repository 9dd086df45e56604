"""Goluzen on the GPU: each new kernel (and each new form of an older one) against its plain twin at sizes of its own,
then the engine's cuts, batches, slot and page reuse, long decoding and window edges in float32 and bfloat16 against
the plain evaluation, decode steps replayed as graphs, greedy generation through the scheduler, and the trace program
on a folder of this design."""
import pytest
import torch

import goluzen_cases as C
import helpers
import kernel_twins as twin
import test_trace_run as TR
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.kernels import ops
from mini_engine_amd.parts.rotary import RotaryEmbedding
from mini_engine_amd.weights.loader import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 5e-5, torch.bfloat16: 1.2e-1}    # widths of 32-48 make bfloat16 noisy


def hip():
    return ops.HipBackend()


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    assert torch.isfinite(a).all()
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
    assert err <= tol, f"relative error {err:.3g} > {tol:g}"


@pytest.fixture(scope="module")
def goluzen_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = C.make_folder(name, str(tmp_path_factory.mktemp(f"goluzen_{name}")))
        return made[name]

    return get


def _steps_meta(q_lens, slots):
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    return cu, torch.tensor(slots, dtype=torch.int32, device=DEV)


def _cpu(t):
    return t.cpu() if torch.is_tensor(t) else t


# ------------------------------------------------------------------ kernels against their twins

@pytest.mark.parametrize("groups", [None, (1, False), (4, False), (4, True), (16, True)],
                         ids=["rule", "one-lane", "four-lanes", "four-lanes-prepared", "sixteen-lanes-prepared"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,N,P", [(3, 8, 16), (2, 10, 14), (4, 128, 256), (1, 200, 7), (2, 64, 64)])
def test_gated_rule_of_the_decay_rows_recurrence(monkeypatch, dtype, H, N, P, groups):
    """Requests of unequal lengths from states of their own, against the token-by-token twin; then one request cut in
    three gives what it gives whole."""
    if groups:
        if groups[0] == 1 and N > 64:
            pytest.skip("a lane keeps up to 64 rows")
        monkeypatch.setattr(ops, "decay_row_groups", lambda *a: groups)
    torch.manual_seed(H * N + P)
    q_lens = [1, 90, 2, 17]
    cu, slots = _steps_meta(q_lens, [2, 0, 4, 1])
    T = sum(q_lens)
    rows = torch.randn(T, 3 * H * N + H * P + 5, device=DEV).to(dtype)
    q, k, raw, v = rows[:, 1:1 + H * N] * 0.3, rows[:, 1 + H * N:1 + 2 * H * N] * 0.3, rows[:, 1 + 2 * H * N:1 + 3 * H * N], rows[:, 1 + 3 * H * N:1 + 3 * H * N + H * P]
    kw = dict(base=torch.randn(H * N, device=DEV) + 2, rate=torch.full((H,), 1 / 3.0, device=DEV), q_scale=N ** -0.5)
    full = torch.randn(6, 3 + H * N * P, device=DEV)
    st_h, st_c = full.clone(), full.cpu().clone()
    got = hip().decay_rows_recurrence(q, k, v, raw, st_h[:, 3:], slots, cu, q_lens, H, H, N, P, "gated", **kw)
    want = twin.decay_rows_recurrence(q.cpu(), k.cpu(), v.cpu(), raw.cpu(), st_c[:, 3:], slots.cpu(), cu.cpu(), q_lens, H, H, N, P, "gated",
                                      **{n: _cpu(t) for n, t in kw.items()})
    close(got, want, 2e-5)
    close(st_h, st_c, 2e-5)
    assert torch.equal(st_h[:, :3], full[:, :3]) and torch.equal(st_h[3], full[3]) and torch.equal(st_h[5], full[5])
    st2 = full.clone()
    parts = []
    for lo, hi in ((1, 40), (40, 41), (41, 91)):
        cu1, slots1 = _steps_meta([hi - lo], [0])
        parts.append(hip().decay_rows_recurrence(q[lo:hi], k[lo:hi], v[lo:hi], raw[lo:hi], st2[:, 3:], slots1, cu1, [hi - lo], H, H, N, P, "gated", **kw))
    close(torch.cat(parts), got[1:91], 1e-5)
    close(st2[0], st_h[0], 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,n,groups,keep,top,group_top", [(50, 12, 40, 3, 2, 3, 2), (3, 10, 256, 5, 2, 3, 2), (200, 32, 64, 4, 2, 4, 2),
                                                              (7, 6, 36, 3, 2, 3, 2), (33, 4, 16, 1, 1, 1, 1), (64, 64, 128, 8, 8, 6, 2),
                                                              (20, 16, 24, 16, 5, 5, 2)])
def test_router_with_sigmoid_scores_a_correction_and_groups_by_their_best_two(dtype, T, E, n, groups, keep, top, group_top):
    """The choice and the weights against the twin, through the kernel of its own and, for few tokens, inside the kernel
    that orders the pairs. The router's rows are drawn so that no two choice scores of a token come close."""
    torch.manual_seed(T + E)
    x = torch.randn(T, n, device=DEV).to(dtype)
    router = torch.randn(E, n, device=DEV) * 2.0 * n ** -0.5
    correction = torch.randn(E, device=DEV) * 0.6 - 0.8            # most choice scores are negative
    rule = ops.RouteRule("sigmoid", correction, group_top=group_top, normalise=False, scale=1.7)
    ids, weights = hip().moe_route(x, router, top, groups, keep, rule)
    want_ids, want_w = twin.moe_route(x.cpu(), router.cpu(), top, groups, keep, ops.RouteRule("sigmoid", correction.cpu(), group_top, False, 1.7))
    z = torch.sigmoid(x.float() @ router.t()) + correction
    gap = (z.sort(-1).values.diff(dim=-1)).amin(-1).cpu()
    sure = gap > 1e-4                                             # a token with two nearly equal scores may go either way
    assert sure.float().mean() > 0.6
    assert torch.equal(ids.cpu()[sure], want_ids[sure])
    close(weights.cpu()[sure], want_w[sure], 2e-3 if dtype == torch.bfloat16 else 1e-5)
    F, hidden = 24, 40
    up = (torch.randn(E, F, n, device=DEV) * 0.2).to(dtype)
    down = (torch.randn(E, hidden, F, device=DEV) * 0.2).to(dtype)
    got = hip().route_and_run_experts(x, router, top, groups, keep, up, down, rule=rule, gated=False)
    want = twin.routed_experts(x.cpu(), ids.cpu(), weights.cpu(), up.cpu(), down.cpu(), gated=False)
    close(got.sum(0), want.sum(0), 3e-2 if dtype == torch.bfloat16 else 2e-5)
    # the softmax rule that other designs use, through the same kernels
    ids0, w0 = hip().moe_route(x, router, top, groups, keep)
    want0 = twin.moe_route(x.cpu(), router.cpu(), top, groups, keep)
    s = torch.softmax(x.float() @ router.t(), -1)
    sure0 = (s.sort(-1).values.diff(dim=-1)).amin(-1).cpu() > 1e-5
    assert torch.equal(ids0.cpu()[sure0], want0[0][sure0])
    close(w0.cpu()[sure0], want0[1][sure0], 2e-3 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("rows", [None, 16, 64, 128], ids=["simple", "rows16", "rows64", "rows128"])
@pytest.mark.parametrize("T,E,top,K,F,N", [(5, 16, 2, 256, 80, 192), (300, 8, 3, 64, 40, 72), (700, 32, 4, 128, 384, 128), (40, 6, 2, 40, 24, 36)])
def test_experts_without_a_gate(rows, T, E, top, K, F, N):
    """relu(W_up x)^2 through W_down, in every tile size of the matrix-core kernels and in the one-wave-per-output form, in
    float32 too."""
    torch.manual_seed(T + K)
    for dtype in ((torch.bfloat16,) if rows else (torch.float32, torch.bfloat16)):
        x = torch.randn(T, K, device=DEV).to(dtype)
        up = (torch.randn(E, F, K, device=DEV) * K ** -0.5).to(dtype)
        down = (torch.randn(E, N, F, device=DEV) * F ** -0.5).to(dtype)
        ids = torch.stack([torch.randperm(E, device=DEV)[:top] for _ in range(T)]).to(torch.int32)
        weights = torch.rand(T, top, device=DEV) + 0.5
        got = hip().routed_experts(x, ids, weights, up, down, force_simple=rows is None, tile_rows=rows, gated=False)
        want = twin.routed_experts(x.cpu(), ids.cpu(), weights.cpu(), up.cpu(), down.cpu(), gated=False)
        close(got, want, 2e-2 if dtype == torch.bfloat16 else 2e-5)
        gu = (torch.randn(E, 2 * F, K, device=DEV) * K ** -0.5).to(dtype)          # the gated form still runs beside it
        close(hip().routed_experts(x, ids, weights, gu, down, force_simple=rows is None, tile_rows=rows),
              twin.routed_experts(x.cpu(), ids.cpu(), weights.cpu(), gu.cpu(), down.cpu()), 2e-2 if dtype == torch.bfloat16 else 2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,dn,dr,nv,R,page", [(5, 24, 8, 40, 72, 16), (3, 12, 6, 10, 20, 8), (16, 128, 64, 128, 192, 16), (1, 8, 8, 8, 16, 4),
                                               (2, 24, 0, 16, 40, 16)])
def test_latent_prepare_and_the_products_per_head(dtype, H, dn, dr, nv, R, page):
    """The latent's norm, both rotations and the page writes against the twin, with tokens of several requests at scattered
    slots and one slot below zero; then the two products per head, on views inside wider rows."""
    torch.manual_seed(H + R)
    T, D = 37, -(-(R + dr) // 16) * 16
    table = None
    if dr:
        enc = RotaryEmbedding(dr, 5000.0, interleaved=True, scaling={"kind": "yarn", "factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0})
        enc.finalize(DEV, dtype, 512)
        table = enc.table
    q_off, kv_off = 0, H * (dn + dr)
    rows = torch.randn(T, kv_off + R + dr + 5, device=DEV).to(dtype)
    w = torch.rand(R, device=DEV) + 0.5
    pos = torch.randint(0, 512, (T,), device=DEV, dtype=torch.int32)
    slots = torch.randperm(10 * page, device=DEV)[:T].to(torch.int32)
    slots[5] = -1
    kc = torch.full((11, 1, page, D), 7.0, device=DEV, dtype=dtype)
    vc = torch.full((11, 1, D, page), 7.0, device=DEV, dtype=dtype)
    kc2, vc2 = kc.cpu().clone(), vc.cpu().clone()
    qa = hip().latent_prepare(rows, q_off, kv_off, H, dn, dr, R, D, w, 1e-5, table, pos, slots, kc, vc, page)
    want = twin.latent_prepare(rows.cpu(), q_off, kv_off, H, dn, dr, R, D, w.cpu(), 1e-5, _cpu(table), pos.cpu(), slots.cpu(), kc2, vc2, page)
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    close(qa.view(T, H, D)[:, :, R:], want.view(T, H, D)[:, :, R:], tol)
    close(kc, kc2, tol)
    close(vc, vc2, tol)
    read = hip().latent_prepare(rows, q_off, None, H, dn, dr, R, D, None, 1e-5, table, pos, None, None, None, page)     # a layer that only reads
    assert torch.equal(read.view(T, H, D)[:, :, R:], qa.view(T, H, D)[:, :, R:])
    uk_t = (torch.randn(H, R, dn, device=DEV) * dn ** -0.5).to(dtype)
    x = rows[:, :kv_off].view(T, H, dn + dr)[:, :, :dn]
    hip().heads_linear(x, uk_t, qa.view(T, H, D)[:, :, :R])
    ref = torch.einsum("thk,hnk->thn", x.float(), uk_t.float())
    close(qa.view(T, H, D)[:, :, :R], ref, tol)
    close(qa.view(T, H, D)[:, :, R:], want.view(T, H, D)[:, :, R:], tol)          # the neighbours are untouched
    uv = (torch.randn(H, nv, R, device=DEV) * R ** -0.5).to(dtype)
    o = torch.randn(T, H * D, device=DEV).to(dtype)
    heads = torch.empty(T, H * nv, device=DEV, dtype=dtype)
    hip().heads_linear(o.view(T, H, D)[:, :, :R], uv, heads.view(T, H, nv))
    close(heads.view(T, H, nv), torch.einsum("thk,hnk->thn", o.view(T, H, D)[:, :, :R].float(), uv.float()), tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_steps(dtype):
    torch.manual_seed(9)
    a, b = torch.randn(3, 50, 72, device=DEV), torch.randn(50, 72, device=DEV).to(dtype)
    wide = torch.randn(50, 11, device=DEV).to(dtype)
    got = hip().weighted_sum([(a, 1.0, None), (b, 1.0, None, wide[:, 4:5])])
    close(got, twin.weighted_sum([(a.cpu(), 1.0, None), (b.cpu(), 1.0, None, wide.cpu()[:, 4:5])]), 1e-5)
    x = (torch.randn(33, 100, device=DEV) * 3).to(dtype)
    close(hip().activation(x[:, 10:70], "gelu_tanh"), torch.nn.functional.gelu(x[:, 10:70].float(), approximate="tanh"), 1e-2 if dtype == torch.bfloat16 else 1e-6)
    table = torch.randn(64, 36, device=DEV).to(dtype)
    idx = torch.tensor([3, 0, 63, 3], dtype=torch.int32, device=DEV)
    rows = hip().gather_rows(table, idx, scale=7.0)
    assert rows.dtype == torch.float32 and torch.equal(rows, table[idx.long()].float() * 7.0)


# ------------------------------------------------------------------ the engine against the plain evaluation

class Env:
    device = DEV

    def __init__(self, folders, dtype, graphs=False):
        self.folders, self.dtype, self.tol, self.graphs, self.models = folders, dtype, TOL[dtype], graphs, {}

    def runner(self, name, pages, slots):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 1024)
        model = self.models[name]
        manager = CacheManager(pages, C.PAGE[name], ModelRunner.windows_of(model), num_state_slots=slots, enable_prefix_caching=False)
        options = dict(use_graphs=True, mixed_graphs_after=1) if self.graphs else {}
        return ModelRunner(model, manager, self.dtype, self.device, 1024, poison_cache=True, **options), manager, folder


@pytest.fixture(scope="module", params=[torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def env(request, goluzen_folders):
    return Env(goluzen_folders, request.param)


@pytest.mark.parametrize("name", C.SMALL)
@pytest.mark.parametrize("case", C.ALL, ids=lambda c: c.__name__)
def test_cuts(env, case, name):
    case(env, name)


def test_far_keys_and_window_edges(env):
    C.window_edges(env)


def test_real_layer_sizes(goluzen_folders):
    C.real_sizes(Env(goluzen_folders, torch.float32), Env(goluzen_folders, torch.bfloat16))


def test_real_layer_sizes_with_a_choice_of_experts(goluzen_folders):
    C.real_sizes(Env(goluzen_folders, torch.float32), Env(goluzen_folders, torch.bfloat16), "routed", every_row=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("case", [C.token_by_token, C.long_decode, C.batch_against_alone], ids=lambda c: c.__name__)
def test_cuts_through_captured_steps(goluzen_folders, case, dtype):
    """The same with decode steps (and small steps that come up again) replayed as graphs: state slots travel with the
    step's metadata, fresh slots are zeroed outside the graph."""
    case(Env(goluzen_folders, dtype, graphs=True), "mix")


def test_hip_libraries_are_the_ones_running(env):
    C.whole(env, "one")
    assert ops.backend().name == "hip" and any("libme_core" in p for p in ops.loaded_libraries())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mix", "odd"])
def test_greedy_generation_through_the_scheduler(goluzen_folders, dtype, name):
    C.greedy_through_the_engine(DEV, dtype, name, goluzen_folders(name), exact=dtype == "float32")


@pytest.mark.parametrize("name", ["mix", "mid", "flat"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_program_on_this_design(goluzen_folders, tmp_path, dtype, name):
    """bin/trace_run picks the model class by the folder's config: four live requests, portions beside single tokens,
    state slots and pages used again; also on a model that keeps no pages at all."""
    folder = goluzen_folders(name)
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
    rc = cli.main(["--random-weights", "goluzen:tinyA", "--num-seqs", "6", "--max-prompt", "40", "--max-output", "8",
                   "--max-model-len", "64", "--max-num-seqs", "4", "--budget", "32", "--tokens-out", "-",
                   "--out", str(tmp_path / "bench.jsonl")])
    assert rc == 0
    lines = capsys.readouterr().out.strip().splitlines()
    row = json.loads(lines[-1])
    tokens = [json.loads(line) for line in lines[-7:-1]]
    assert [len(t) for t in tokens] == [8] * 6 and all(0 <= t < 256 for ts in tokens for t in ts)
    assert row["num_seqs"] == 6 and row["output_tokens"] == 48 and row["throughput_tok_s"] > 0
