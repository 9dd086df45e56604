"""Tavevik on the CPU: configuration, checkpoint layout, and the engine's bookkeeping for it (pages with kept first
positions, state slots, batches, cuts, the scheduler) with the plain twins of the kernels in float32, against the plain
evaluation; each twin against the plain function of its mechanism; and the plain evaluation with one mechanism taken
out, which must be far off (so that the random weights cannot hide a fault of that mechanism)."""
import copy
import json

import pytest
import torch

import kernel_twins as twin
import plain_tavevik as P
import tavevik_cases as C
from mini_engine_amd.cache.manager import CacheManager, first_kept, pinned_prefix
from mini_engine_amd.config.model_config import ConfigError, TavevikConfig, load_model_config
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.registry import build_model
from mini_engine_amd.weights.loader import load_model


@pytest.fixture(scope="module")
def tavevik_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = C.make_folder(name, str(tmp_path_factory.mktemp(f"tavevik_{name}")))
        return made[name]

    return get


class Env:
    device, dtype, tol = "cpu", torch.float32, 4e-5      # float32 sums against float64: the sharpened softmax and the recurrences leave 2e-5

    def __init__(self, folders):
        self.folders, self.models = folders, {}

    def runner(self, name, pages, slots):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 512)
        model = self.models[name]
        manager = CacheManager(pages, C.PAGE[name], ModelRunner.windows_of(model), num_state_slots=slots, enable_prefix_caching=False)
        return ModelRunner(model, manager, self.dtype, self.device, 512, poison_cache=True), manager, folder


def test_config_reads_back_and_refuses_what_it_cannot_run(tmp_path):
    for name, raw in C.CONFIGS.items():
        cfg = TavevikConfig.from_dict(raw)
        assert TavevikConfig.from_dict(cfg.to_dict()) == cfg
        assert len(cfg.layers) == len(raw["layers"]) and cfg.vocab_size == raw["vocab"]
    with open(tmp_path / "config.json", "w") as f:
        json.dump(C.CONFIGS["pair"], f)
    assert isinstance(load_model_config(str(tmp_path)), TavevikConfig)          # chosen by the file's architecture name
    for spoil in (lambda c: c["layers"][0].update(type="parallel_3"),
                  lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3),
                  lambda c: c["layers"][0]["mixer"]["right"].pop("conv"),
                  lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=7),
                  lambda c: c["layers"][1]["mlp"].pop("limit"),
                  lambda c: c["layers"][1]["mixer"].pop("right")):
        bad = copy.deepcopy(C.CONFIGS["pair"])
        spoil(bad)
        with pytest.raises(ConfigError):
            TavevikConfig.from_dict(bad)


def test_model_is_assembled_from_the_config(tavevik_folders):
    model = build_model(TavevikConfig.from_dict(C.CONFIGS["pair"]))
    plan = model.cache_plan()
    assert plan.call_group == [0, 1] and plan.call_writes == [True, True]
    # the delta rule's matrices and its convolutions' inputs; the shifted mixer's matrices and the previous token's input
    assert plan.state_needs[0].shape == (4 * 20 * 12 + (2 * 2 * 20 + 4 * 12) * 3,) and plan.state_needs[1].shape == (3 * 12 * 12 + 48,)
    assert ModelRunner.windows_of(model) == [7, (("window", 9), ("first", 3))]
    names = {src.name for sources in model.weight_sources.values() for src in sources}
    assert {"embed", "final.norm", "l0.mix.left.q.b", "l0.mix.left.sink", "l0.mix.left.o.b", "l0.mix.right.q.conv", "l0.mix.right.a1",
            "l0.mix.right.g2", "l0.mix.right.A_log", "l1.mix.left.g", "l1.mix.right.mu.w", "l1.mix.right.w2", "l1.mix.right.u",
            "l1.mlp.gate", "l0.norm2"} <= names
    assert "head" not in names and "l1.mix.left.sink" not in names and "l0.mix.left.g" not in names
    # the thin pairs' inner widths come from the checkpoint's shapes when the file does not name them
    raw = copy.deepcopy(C.CONFIGS["pair"])
    for layer in raw["layers"]:
        layer["mixer"]["right"].pop("decay_rank", None)
        layer["mixer"]["right"].pop("gate_rank", None)
    folder = tavevik_folders("pair")
    with open(folder + "/config.json") as f:
        kept = f.read()
    try:
        with open(folder + "/config.json", "w") as f:
            json.dump(raw, f)
        loaded = load_model(folder, "cpu", torch.float32, 64)
        assert loaded.layers[0].mixer.right.decay_rank == 8 and loaded.layers[0].mixer.right.gate_rank == 16
        assert loaded.layers[1].mixer.right.decay_rank == 8
    finally:
        with open(folder + "/config.json", "w") as f:
            f.write(kept)


def test_pages_of_kept_positions_stay():
    from mini_engine_amd.parts import CacheNeed
    rule = CacheNeed.keys_and_values(2, 16, window=9, keep_first=3).keep()
    assert rule == (("window", 9), ("first", 3)) and pinned_prefix(rule) == 3 and pinned_prefix(9) == 0 and pinned_prefix(None) == 0
    assert [first_kept(rule, n) for n in (0, 8, 9, 30)] == [0, 0, 1, 22]
    manager = CacheManager(8, 4, [rule], num_state_slots=1, enable_prefix_caching=False)
    assert manager.allocate("r", 0, 21) and manager.block_table("r") == [0, 1, 2, 3, 4, 5]
    # the next token stands at 21 and sees keys from 13 on: pages 1 and 2 (positions 4-11) go, page 0 (positions 0-3) stays
    assert manager.allocate("r", 21, 1) and manager.block_table("r") == [0, -1, -1, 3, 4, 5]
    assert manager.allocate("r", 22, 9) and manager.block_table("r") == [0, -1, -1, 3, 4, 5, 6, 7] and manager.num_free_pages(0) == 2
    assert manager.allocate("r", 31, 1) and manager.block_table("r") == [0, -1, -1, -1, -1, 5, 6, 7] and manager.num_free_pages(0) == 4
    manager.check_invariants()
    manager.free("r")
    assert manager.num_free_pages(0) == 8
    # more kept positions than a page: both pages that hold any of them stay
    manager = CacheManager(8, 4, [(("window", 2), ("first", 5))], enable_prefix_caching=False)
    assert manager.allocate("s", 0, 20) and manager.allocate("s", 20, 1)
    assert manager.block_table("s") == [0, 1, -1, -1, 4, 5]


# ---------------------------------------------------------------- each twin against the plain function of its mechanism

def _meta(q_lens, slots):
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    seq = torch.tensor([b for b, n in enumerate(q_lens) for _ in range(n)], dtype=torch.int32)
    return cu, torch.tensor(slots, dtype=torch.int32), seq


def test_delta_rule_twin_in_steps_against_the_plain_loop():
    torch.manual_seed(0)
    T, H, G, N, Pv = 23, 4, 2, 6, 5
    m = {"heads": H, "kv_heads": G, "dim": N, "vdim": Pv, "conv": 1}
    width = 16
    h = torch.randn(T, width, dtype=torch.float64)
    w = {"x.q": torch.randn(G * N, width).double(), "x.k": torch.randn(G * N, width).double(), "x.v": torch.randn(H * Pv, width).double(),
         "x.q.conv": torch.ones(G * N, 1).double(), "x.k.conv": torch.ones(G * N, 1).double(), "x.v.conv": torch.ones(H * Pv, 1).double(),
         "x.b": torch.randn(H, width).double(), "x.a1": torch.randn(3, width).double(), "x.a2": torch.randn(H * N, 3).double(),
         "x.dt_bias": torch.randn(H * N).double(), "x.A_log": torch.randn(H).double(), "x.norm": torch.ones(Pv).double(),
         "x.g1": torch.zeros(3, width).double(), "x.g2": torch.zeros(H * Pv, 3).double(), "x.o": torch.eye(H * Pv).double()}
    want = P.delta_rule(m, w, "x.", h, 1e-5)                 # unit rms per head, half a gate
    silu = lambda z: z * torch.sigmoid(z)
    q, k, v = silu(h @ w["x.q"].T).float(), silu(h @ w["x.k"].T).float(), silu(h @ w["x.v"].T).float()
    raw, beta = ((h @ w["x.a1"].T) @ w["x.a2"].T).float(), (h @ w["x.b"].T).float()
    state = torch.zeros(3, H * N * Pv)
    ys = []
    for lo, hi in ((0, 9), (9, 10), (10, 12), (12, 23)):     # the state carries over the cuts
        cu, slots, _ = _meta([hi - lo], [1])
        ys.append(twin.decay_rows_recurrence(q[lo:hi], k[lo:hi], v[lo:hi], raw[lo:hi], state, slots, cu, [hi - lo], H, G, N, Pv, "delta",
                                             base=w["x.dt_bias"].float(), rate=torch.exp(w["x.A_log"].float()), beta=beta[lo:hi],
                                             unit_eps=1e-6, q_scale=N ** -0.5))
    y = torch.cat(ys).double().view(T, H, Pv)
    got = (P.unit_rms(y, 1e-5) * 0.5).reshape(T, H * Pv)
    assert float((got - want).abs().max()) < 1e-4 * float(want.abs().max())
    assert float(state[0].abs().max()) == 0 and float(state[2].abs().max()) == 0


def test_shifted_mixer_twins_in_steps_against_the_plain_loop():
    torch.manual_seed(1)
    T, H, N, width = 19, 3, 5, 12
    m = {"heads": H, "dim": N}
    h = torch.randn(T, width, dtype=torch.float64)
    w = {f"x.mu.{s}": torch.rand(width).double() for s in "rkvgw"}
    for s in "rkvg":
        w["x." + s] = torch.randn(H * N, width).double() * 0.5
    w.update({"x.w1": torch.randn(4, width).double(), "x.w2": torch.randn(H * N, 4).double(), "x.w0": torch.randn(H * N).double() - 2,
              "x.u": torch.randn(H, N).double()})
    want, _ = P.shifted_mix(m, w, "x.", h)
    mu = torch.stack([w[f"x.mu.{s}"] for s in "rkvgw"]).float()
    state = torch.zeros(2, H * N * N + width)
    ys = []
    for lo, hi in ((0, 1), (1, 8), (8, 10), (10, 19)):
        cu, slots, seq = _meta([hi - lo], [0])
        mixes = twin.token_shift(h[lo:hi].float(), mu, state[:, H * N * N:], slots, cu, seq).double()
        r, k, v = (mixes[i] @ w["x." + s].T for i, s in enumerate("rkv"))
        raw = torch.tanh(mixes[4] @ w["x.w1"].T) @ w["x.w2"].T
        ys.append(twin.decay_rows_recurrence(r.float(), k.float(), v.float(), raw.float(), state[:, : H * N * N], slots, cu, [hi - lo],
                                             H, H, N, N, "bonus", base=w["x.w0"].float(), bonus=w["x.u"].float().reshape(-1)))
    got = torch.cat(ys).double().view(T, H, N)
    assert float((got - want).abs().max()) < 1e-4 * float(want.abs().max())
    assert torch.equal(state[0, H * N * N:], h[-1].float())


def test_attention_twin_with_kept_keys_cap_and_sinks_against_the_plain_mask():
    """One request in pages, queries at chosen positions; one key is made to stand out so that the softmax shows whether
    it was seen: just inside and just outside the window, among the kept positions and right behind them."""
    torch.manual_seed(2)
    n, D, page, window, keep = 40, 8, 4, 6, 3
    k = torch.randn(n, 1, D)
    v = torch.randn(n, 1, D)
    kc, vc = torch.full((10, 1, page, D), float("nan")), torch.full((10, 1, D, page), float("nan"))
    slots = torch.arange(n, dtype=torch.int32)
    twin.write_pages(k, v, slots, kc, vc, page)
    bt = torch.arange(10, dtype=torch.int32)[None]
    sinks = torch.tensor([0.7, -0.3])
    for pos in (0, 2, 5, 6, 8, 9, 20, 39):
        for far in (0, 2, 3, pos - window, pos - window + 1, pos):
            if not 0 <= far <= pos:
                continue
            q = torch.randn(1, 2 * D)
            q[0, :D] = 4.0 * k[far, 0]                       # head 0 points at key `far`
            args = (q, kc, vc, page, bt, torch.tensor([pos + 1], dtype=torch.int32), torch.zeros(1, dtype=torch.int32),
                    torch.tensor([pos], dtype=torch.int32), None, 1, pos + 1, 0.5, window, 2, 1, D)
            got = twin.paged_attention(*args, keep_first=keep, softcap=3.0, sinks=sinks).double().view(2, D)
            for head in range(2):
                js = [j for j in range(pos + 1) if P.visible(pos, j, window, keep)]
                s = (k[js, 0].double() @ q[0, head * D:(head + 1) * D].double()) * 0.5
                s = 3.0 * torch.tanh(s / 3.0)
                e = torch.exp(s - s.max())
                want = ((e / (e.sum() + torch.exp(sinks[head].double() - s.max())))[:, None] * v[js, 0].double()).sum(0)
                assert float((got[head] - want).abs().max()) < 1e-5


def test_small_twins():
    gu = torch.randn(7, 10) * 3
    g, u = torch.clamp(gu[:, :5], max=1.5), torch.clamp(gu[:, 5:], -1.5, 1.5)
    assert torch.allclose(twin.glu_clamped(gu, 1.5, 1.702), g * torch.sigmoid(1.702 * g) * (u + 1), atol=1e-6)
    a, b = torch.randn(2, 5, 6), torch.randn(5, 6)
    bias = torch.randn(6)
    s = twin.weighted_sum([(a, 0.5, None), (b, -2.0, bias)])
    assert torch.allclose(s, 0.5 * a.sum(0) - 2.0 * (b + bias), atol=1e-6)
    stream, w = torch.randn(5, 6), torch.rand(6)
    lo, new = twin.weighted_sum([(a, 0.5, None), (b, -2.0, bias)], w, 1e-5, stream, torch.float32)
    assert torch.allclose(new, stream + w * s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + 1e-5), atol=1e-6)
    assert torch.allclose(twin.add_bias(a, bias[:4], torch.float32)[:, 4:], a.sum(0)[:, 4:])


# ---------------------------------------------------------------- a mechanism left out must show

@pytest.mark.parametrize("spoil", ["keep_first", "softcap", "sink", "bias", "gate", "window", "bonus", "limit", "scales", "shift"])
def test_the_weights_show_a_mechanism_that_is_left_out(tavevik_folders, spoil):
    folder = tavevik_folders("pair")
    cfg, w = P.read_folder(folder)
    ids = C.random_ids(40, 101, 5)
    ref = P.logits(cfg, w, ids)
    cfg, w = copy.deepcopy(cfg), dict(w)
    left1, left0 = cfg["layers"][1]["mixer"]["left"], cfg["layers"][0]["mixer"]["left"]
    if spoil == "keep_first":
        left1["mask"].pop("keep_first")
    elif spoil == "softcap":
        left1.pop("softcap")
    elif spoil == "sink":
        w["l0.mix.left.sink"] = w["l0.mix.left.sink"] - 30.0
    elif spoil == "bias":
        w["l0.mix.left.k.b"] = torch.zeros_like(w["l0.mix.left.k.b"])
    elif spoil == "gate":
        w["l1.mix.left.g"] = torch.zeros_like(w["l1.mix.left.g"])
    elif spoil == "window":
        left0["mask"]["size"] += 1
    elif spoil == "bonus":
        w["l1.mix.right.u"] = torch.zeros_like(w["l1.mix.right.u"])
    elif spoil == "limit":
        cfg["layers"][1]["mlp"]["limit"] = 100.0
    elif spoil == "scales":
        m = cfg["layers"][0]["mixer"]
        m["left_scale"], m["right_scale"] = m["right_scale"], m["left_scale"]
    elif spoil == "shift":
        w["l1.mix.right.mu.k"] = torch.zeros_like(w["l1.mix.right.mu.k"])
    off = P.logits(cfg, w, ids)
    assert float((off - ref).abs().max() / ref.abs().max()) > 1e-3, f"leaving out {spoil} does not show in the logits"


# ---------------------------------------------------------------- the engine against the plain evaluation

@pytest.mark.parametrize("name", ["pair", "order", "one", "two", "odd"])
@pytest.mark.parametrize("case", C.ALL, ids=lambda c: c.__name__)
def test_cuts(tavevik_folders, plain_backend, case, name):
    case(Env(tavevik_folders), name)


def test_far_keys_and_window_edges(tavevik_folders, plain_backend):
    C.window_edges(Env(tavevik_folders))


@pytest.mark.parametrize("name", ["pair", "order"])
def test_greedy_generation_through_the_scheduler(tavevik_folders, plain_backend, name):
    C.greedy_through_the_engine("cpu", "float32", name, tavevik_folders(name), exact=True)


def test_command_line_on_a_folder_of_this_design(tavevik_folders, plain_backend, tmp_path):
    """`python -m mini_engine_amd.cli --model DIR`: the folder's config picks the model class; prompts in, greedy tokens out."""
    from mini_engine_amd import cli
    import helpers
    folder = tavevik_folders("pair")
    prompts = [helpers.random_ids(n, 101, 950 + n) for n in (3, 19, 41)]
    path = tmp_path / "prompts.jsonl"
    path.write_text("\n".join(json.dumps(p) for p in prompts) + "\n")
    out = tmp_path / "tokens.jsonl"
    rc = cli.main(["--model", folder, "--prompts", str(path), "--tokens-out", str(out), "--temperature", "0", "--max-output", "6",
                   "--dtype", "float32", "--device", "cpu", "--num-kv-blocks", "64", "--block-size", "8", "--budget", "16",
                   "--max-num-seqs", "2", "--max-model-len", "128", "--out", str(tmp_path / "rows.jsonl")])
    assert rc == 0
    got = [json.loads(line) for line in open(out)]
    for p, g in zip(prompts, got):
        seq = list(p)
        assert len(g) == 6
        for tok in g:
            assert tok == int(C.plain_logits(folder, seq)[-1].argmax())
            seq.append(tok)


def test_launch_rule_of_the_recurrence():
    from mini_engine_amd.kernels import ops
    for N in range(1, 257):
        for P_ in (1, 16, 64, 80, 128):
            for B, H in ((1, 1), (4, 16), (64, 32)):
                rg, prepared = ops.decay_row_groups(B, H, N, P_)
                assert not prepared and rg in (1, 4) and (rg == 4 or N <= 64)
                rg, prepared = ops.decay_row_groups(B, H, N, P_, 700)
                assert prepared and rg in (4, 16) and (rg == 4 or B * H * -(-P_ // 4) <= 4096)
