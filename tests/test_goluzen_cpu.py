"""Goluzen on the CPU: configuration, checkpoint layout, and the engine's bookkeeping for it (two page groups of which
one is shared by a reading layer, kept first positions, state slots, batches, cuts, the scheduler) with the plain twins
of the kernels in float32, against the plain evaluation; each new twin against the plain function of its mechanism;
and the plain evaluation with one mechanism taken out, which must be far off (so that the random weights cannot hide
a fault of that mechanism)."""
import copy
import json
import math

import pytest
import torch

import goluzen_cases as C
import kernel_twins as twin
import plain_goluzen as P
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.config.model_config import ConfigError, GoluzenConfig, load_model_config
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.kernels import ops
from mini_engine_amd.parts.rotary import RotaryEmbedding
from mini_engine_amd.registry import build_model
from mini_engine_amd.weights.loader import load_model


@pytest.fixture(scope="module")
def goluzen_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = C.make_folder(name, str(tmp_path_factory.mktemp(f"goluzen_{name}")))
        return made[name]

    return get


class Env:
    device, dtype, tol = "cpu", torch.float32, 4e-5      # float32 sums against float64

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
        cfg = GoluzenConfig.from_dict(raw)
        assert GoluzenConfig.from_dict(cfg.to_dict()) == cfg
        assert len(cfg.layers) == len(raw["layers"]) and cfg.vocab_size == raw["vocab"]
    with open(tmp_path / "config.json", "w") as f:
        json.dump(C.CONFIGS["mix"], f)
    assert isinstance(load_model_config(str(tmp_path)), GoluzenConfig)          # chosen by the file's architecture name
    for spoil in (lambda c: c["layers"][0].update(type="gla2"),
                  lambda c: c["layers"][2]["mixer"].update(kv_heads=3),
                  lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7),
                  lambda c: c["layers"][3]["mixer"].update(kv_from=2),           # not a latent layer
                  lambda c: c["layers"][3]["mixer"].update(kv_rank=32),          # another latent than its source's
                  lambda c: c["layers"][1]["mixer"].update(kv_from=1),           # not an earlier layer
                  lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
                  lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3),
                  lambda c: c["layers"][0]["mixer"].pop("tau"),
                  lambda c: c["layers"][0]["mlp"].update(kind="glu")):
        bad = copy.deepcopy(C.CONFIGS["mix"])
        spoil(bad)
        with pytest.raises(ConfigError):
            GoluzenConfig.from_dict(bad)


def test_model_is_assembled_from_the_config(goluzen_folders):
    model = build_model(GoluzenConfig.from_dict(C.CONFIGS["mix"]))
    plan = model.cache_plan()
    # the latent layers share one group, and the second of them reads the first one's pages
    assert plan.call_group == [None, 0, 1, 0] and plan.call_writes == [False, True, True, False]
    assert plan.state_needs[0].shape == (3 * 8 * 16,) and plan.state_needs[1:] == [None, None, None]
    assert ModelRunner.windows_of(model) == [(("window", 5), ("window", 9)), (("window", 7), ("first", 3))]   # owner and reader: the looser holds
    assert plan.group_needs[0].tensors[0].shape[0] == 1 and plan.group_needs[0].tensors[0].shape[2] == 48       # one head of rank + rotating part
    odd = build_model(GoluzenConfig.from_dict(C.CONFIGS["odd"]))
    assert ModelRunner.windows_of(odd)[0] == (("window", 6), ("window", 11))          # here the reader's window is the longer one
    assert odd.layers[0].feed_forward is None and odd.layers[3].feed_forward.shared is not None and odd.layers[1].feed_forward.shared is None
    names = {src.name for sources in model.weight_sources.values() for src in sources}
    assert {"embed", "head", "final.norm", "l0.mix.a1", "l0.mix.a2.b", "l0.mix.norm", "l0.mlp.up", "l1.mix.dkv", "l1.mix.dkv.norm",
            "l1.mix.uk", "l1.mix.g", "l1.mlp.e7.up", "l1.mlp.correction", "l1.mlp.shared.sg", "l2.mix.q.b", "l2.mix.sink", "l3.mix.uv",
            "l3.norm2"} <= names
    assert "l3.mix.dkv" not in names and "l3.mlp.shared.up" not in names and "l1.mlp.e0.gate" not in names
    # the thin pair's inner width comes from the checkpoint's shapes when the file does not name it
    raw = copy.deepcopy(C.CONFIGS["mix"])
    raw["layers"][0]["mixer"].pop("decay_rank")
    folder = goluzen_folders("mix")
    with open(folder + "/config.json") as f:
        kept = f.read()
    try:
        with open(folder + "/config.json", "w") as f:
            json.dump(raw, f)
        assert load_model(folder, "cpu", torch.float32, 64).layers[0].mixer.decay_rank == 8
    finally:
        with open(folder + "/config.json", "w") as f:
            f.write(kept)


# ---------------------------------------------------------------- each twin against the plain function of its mechanism

def _meta(q_lens, slots):
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    return cu, torch.tensor(slots, dtype=torch.int32)


def test_gated_rule_twin_in_steps_against_the_plain_loop():
    torch.manual_seed(0)
    T, H, N, Pv, width, rank = 23, 3, 6, 5, 16, 4
    m = {"heads": H, "dim": N, "vdim": Pv, "tau": 3.0}
    h = torch.randn(T, width, dtype=torch.float64)
    w = {"x.q": torch.randn(H * N, width).double(), "x.k": torch.randn(H * N, width).double() * 0.5, "x.v": torch.randn(H * Pv, width).double(),
         "x.a1": torch.randn(rank, width).double(), "x.a2": torch.randn(H * N, rank).double(), "x.a2.b": torch.randn(H * N).double() + 1,
         "x.norm": torch.ones(Pv).double(), "x.g": torch.zeros(H * Pv, width).double(), "x.o": torch.eye(H * Pv).double()}
    w["x.g"] = torch.randn(H * Pv, width).double()
    want = P.gated_linear_attention(h, w, "x.", m, 1e-5)
    q, k, v = (h @ w["x.q"].T).float(), (h @ w["x.k"].T).float(), (h @ w["x.v"].T).float()
    raw = ((h @ w["x.a1"].T) @ w["x.a2"].T).float()
    state = torch.zeros(3, H * N * Pv)
    ys = []
    for lo, hi in ((0, 9), (9, 10), (10, 12), (12, 23)):     # the state carries over the cuts
        cu, slots = _meta([hi - lo], [1])
        ys.append(twin.decay_rows_recurrence(q[lo:hi], k[lo:hi], v[lo:hi], raw[lo:hi], state, slots, cu, [hi - lo], H, H, N, Pv, "gated",
                                             base=w["x.a2.b"].float(), rate=torch.full((H,), 1 / 3.0), q_scale=N ** -0.5))
    y = torch.cat(ys)
    g = (h @ w["x.g"].T).float()
    got = twin.gated_rms_norm(y, g, torch.ones(H * Pv), 1e-5, H, "silu_behind", torch.float32).double()
    assert float((got - want).abs().max()) < 1e-4 * float(want.abs().max())
    assert float(state[0].abs().max()) == 0 and float(state[2].abs().max()) == 0


def test_router_twin_against_the_plain_choice():
    """Sigmoid scores, a correction that changes the choice but not the weights, groups scored by their two best (which is not
    the order of their best), choice scores below zero, weights that are not brought to sum one."""
    torch.manual_seed(3)
    T, E, n = 50, 12, 10
    x = torch.randn(T, n)
    router = torch.randn(E, n)
    correction = torch.randn(E) * 0.8 - 0.9              # most choice scores are negative
    for groups, keep, top in ((3, 2, 3), (4, 1, 2), (2, 1, 6), (1, 1, 5), (6, 6, 4), (12, 5, 5)):
        r = {"experts": E, "top": top, "scale": 1.7, "groups": {"count": groups, "keep": keep}}
        ids, weights = P.choose_experts((x @ router.T).double(), correction.double(), r)
        rule = ops.RouteRule("sigmoid", correction, group_top=2, normalise=False, scale=1.7)
        got_ids, got_w = twin.moe_route(x, router, top, groups, keep, rule)
        assert torch.equal(got_ids.long(), ids)
        assert torch.allclose(got_w.double(), weights, atol=1e-6)
    # one group differs when groups go by their best expert only
    z = torch.tensor([[3.0, -3.0, 2.0, 2.0]])
    rule2, rule1 = ops.RouteRule("sigmoid", None, 2, False, 1.0), ops.RouteRule("sigmoid", None, 1, False, 1.0)
    eye = torch.eye(4)
    assert twin.moe_route(z, eye, 1, 2, 1, rule2)[0].tolist() == [[2]] and twin.moe_route(z, eye, 1, 2, 1, rule1)[0].tolist() == [[0]]


def test_rotation_tables_against_the_plain_rates():
    for dims, base, sc in ((8, 5000.0, (4.0, 32, 8.0, 1.0)), (12, 80000.0, (8.0, 512, 20.0, 2.0)), (6, 300.0, (2.0, 16, 4.0, 1.0))):
        scaling = dict(zip(("factor", "original", "fast", "slow"), sc))
        enc = RotaryEmbedding(dims, base, interleaved=True, scaling=dict(scaling, kind="yarn"))
        enc.finalize("cpu", torch.float32, 40)
        f, mult = P.yarn_frequencies(dims, base, scaling)
        a = torch.arange(40, dtype=torch.float64)[:, None] * f[None, :]
        want = torch.stack((a.cos(), a.sin()), -1) * mult
        assert float((enc.table.double() - want).abs().max()) < 1e-6 and mult > 1.0
        assert len(set((f * base ** (2 * torch.arange(dims // 2, dtype=torch.float64) / dims)).round(decimals=6).tolist())) > 1       # a ramp, not one factor
    enc = RotaryEmbedding(16, 3000.0, rotary_dims=8, stored_dim=12, scaling={"kind": "linear", "factor": 2.5})
    enc.finalize("cpu", torch.float32, 10)
    f = P.linear_frequencies(8, 3000.0, 2.5)
    assert torch.allclose(enc.table[:, :4, 1].double(), torch.sin(torch.arange(10, dtype=torch.float64)[:, None] * f), atol=1e-7)
    assert torch.equal(enc.table[:, 4:, 0], torch.ones(10, 4)) and torch.equal(enc.table[:, 4:, 1], torch.zeros(10, 4))


def test_latent_twins_against_the_plain_heads():
    """Queries carried into the latent's space against keys and values made head by head; a window whose edge is made to show
    by a key that the query points at."""
    torch.manual_seed(5)
    T, H, dn, dr, nv, R, width, page, window = 30, 3, 6, 4, 5, 10, 12, 4, 7
    m = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": nv, "kv_rank": R, "scale": 1.3, "rot": {"dims": dr, "base": 50.0}, "mask": {"size": window}}
    h = torch.randn(T, width, dtype=torch.float64)
    w = {"x.q": torch.randn(H * (dn + dr), width).double(), "x.dkv": torch.randn(R + dr, width).double(), "x.dkv.norm": torch.rand(R).double() + 0.5,
         "x.uk": torch.randn(H * dn, R).double(), "x.uv": torch.randn(H * nv, R).double(), "x.g": torch.randn(H * nv, width).double(),
         "x.o": torch.eye(H * nv).double()}
    want = P.latent_attention(h, w, "x.", m, 1e-5, P.latent_of(h, w, "x.", m, 1e-5))
    enc = RotaryEmbedding(dr, 50.0, interleaved=True, exact_angles=True)
    enc.finalize("cpu", torch.float32, 64)
    D = 16
    rows = torch.cat((h @ w["x.q"].T, h @ w["x.dkv"].T), 1).float()
    kc, vc = torch.full((9, 1, page, D), float("nan")), torch.full((9, 1, D, page), float("nan"))
    pos = torch.arange(T, dtype=torch.int32)
    qa = twin.latent_prepare(rows, 0, H * (dn + dr), H, dn, dr, R, D, w["x.dkv.norm"].float(), 1e-5, enc.table, pos, pos, kc, vc, page)
    uk_t = w["x.uk"].float().view(H, dn, R).transpose(1, 2).contiguous()
    twin.heads_linear(rows[:, :H * (dn + dr)].view(T, H, dn + dr)[:, :, :dn], uk_t, qa.view(T, H, D)[:, :, :R])
    bt = torch.arange(9, dtype=torch.int32)[None]
    o = twin.paged_attention(qa, kc, vc, page, bt, torch.tensor([T], dtype=torch.int32), torch.zeros(T, dtype=torch.int32), pos,
                             torch.tensor([0, T], dtype=torch.int32), 0, 0, 1.3, window, H, 1, D, max_prefill_context=T)
    heads = torch.empty(T, H * nv)
    twin.heads_linear(o.view(T, H, D)[:, :, :R], w["x.uv"].float().view(H, nv, R), heads.view(T, H, nv))
    got = (heads.double() * torch.sigmoid(h @ w["x.g"].T))
    assert float((got - want).abs().max()) < 2e-5 * float(want.abs().max())
    wider = P.latent_attention(h, w, "x.", dict(m, mask={"size": window + 1}), 1e-5, P.latent_of(h, w, "x.", m, 1e-5))
    assert float((wider - want).abs().max()) > 1e-2 * float(want.abs().max())           # the edge shows


def test_small_twins():
    a, b, gate = torch.randn(2, 5, 6), torch.randn(5, 6), torch.randn(5, 3)
    s = twin.weighted_sum([(a, 1.0, None), (b, 1.0, None, gate[:, 1:2])])
    assert torch.allclose(s, a.sum(0) + b * torch.sigmoid(gate[:, 1:2]), atol=1e-6)
    x = torch.randn(4, 7) * 2
    assert torch.allclose(twin.activation(x, "gelu_tanh").double(), P.gelu_tanh(x.double()), atol=1e-6)
    assert torch.allclose(twin.activation(x, "gelu_tanh"), torch.nn.functional.gelu(x, approximate="tanh"), atol=1e-6)
    table = torch.randn(9, 5).bfloat16()
    rows = twin.gather_rows(table, torch.tensor([3, 0, 8], dtype=torch.int32), scale=7.0)
    assert rows.dtype == torch.float32 and torch.equal(rows, table[[3, 0, 8]].float() * 7.0)


# ---------------------------------------------------------------- a mechanism left out must show

@pytest.mark.parametrize("spoil", ["keep_first", "softcap", "sink", "bias", "window", "stretch", "unit", "latent_window", "yarn", "latent_norm",
                                   "gate", "own_latent", "tau", "decay_bias", "correction", "groups", "route_scale", "shared_gate", "gelu",
                                   "embedding_scale", "one_plus"])
def test_the_weights_show_a_mechanism_that_is_left_out(goluzen_folders, spoil):
    folder = goluzen_folders("mix")
    cfg, w = P.read_folder(folder)
    ids = C.random_ids(40, 101, 5)
    ref = P.logits(cfg, w, ids)
    cfg, w = copy.deepcopy(cfg), dict(w)
    gla, lat, att, lat2 = (layer["mixer"] for layer in cfg["layers"])
    if spoil == "keep_first":
        att["mask"].pop("keep_first")
    elif spoil == "softcap":
        att.pop("softcap")
    elif spoil == "sink":
        w["l2.mix.sink"] = w["l2.mix.sink"] - 30.0
    elif spoil == "bias":
        w["l2.mix.k.b"] = torch.zeros_like(w["l2.mix.k.b"])
    elif spoil == "window":
        att["mask"]["size"] += 1
    elif spoil == "stretch":
        att["rot"].pop("scaling")
    elif spoil == "unit":
        w["l2.mix.q"], w["l2.mix.q.b"] = w["l2.mix.q"] * 2.0, w["l2.mix.q.b"] * 2.0      # unit root mean square per head undoes this
    elif spoil == "latent_window":
        lat2["mask"]["size"] += 1
    elif spoil == "yarn":
        lat["rot"].pop("scaling"); lat2["rot"].pop("scaling")
    elif spoil == "latent_norm":
        w["l1.mix.dkv.norm"] = torch.ones_like(w["l1.mix.dkv.norm"]) * 1.3
    elif spoil == "gate":
        w["l1.mix.g"] = torch.zeros_like(w["l1.mix.g"])
    elif spoil == "own_latent":
        lat2.pop("kv_from")
        w["l3.mix.dkv"], w["l3.mix.dkv.norm"] = w["l1.mix.dkv"] * 0.9, w["l1.mix.dkv.norm"]
    elif spoil == "tau":
        gla["tau"] = 1.0
    elif spoil == "decay_bias":
        w["l0.mix.a2.b"] = torch.zeros_like(w["l0.mix.a2.b"])
    elif spoil == "correction":
        w["l1.mlp.correction"] = torch.zeros_like(w["l1.mlp.correction"])
    elif spoil == "groups":
        cfg["layers"][2]["mlp"]["router"].pop("groups")
    elif spoil == "route_scale":
        cfg["layers"][1]["mlp"]["router"]["scale"] = 1.0
    elif spoil == "shared_gate":
        w["l1.mlp.shared.sg"] = torch.zeros_like(w["l1.mlp.shared.sg"])
    elif spoil == "gelu":
        w["l0.mlp.up"] = -w["l0.mlp.up"]                     # an even activation would not notice
    elif spoil == "embedding_scale":
        cfg["embedding"]["scale"] = 1.0
    elif spoil == "one_plus":
        w["l2.norm1"] = w["l2.norm1"] - 1.0
    if spoil == "unit":
        off = P.logits(cfg, w, ids)
        ref = P.logits(*P.read_folder(folder), ids)
        assert float((off - ref).abs().max() / ref.abs().max()) < 1e-4
        return
    off = P.logits(cfg, w, ids)
    assert float((off - ref).abs().max() / ref.abs().max()) > 1e-3, f"leaving out {spoil} does not show in the logits"


# ---------------------------------------------------------------- the engine against the plain evaluation

@pytest.mark.parametrize("name", C.SMALL)
@pytest.mark.parametrize("case", C.ALL, ids=lambda c: c.__name__)
def test_cuts(goluzen_folders, plain_backend, case, name):
    case(Env(goluzen_folders), name)


def test_far_keys_and_window_edges(goluzen_folders, plain_backend):
    C.window_edges(Env(goluzen_folders))


@pytest.mark.parametrize("name", ["mix", "odd"])
def test_greedy_generation_through_the_scheduler(goluzen_folders, plain_backend, name):
    C.greedy_through_the_engine("cpu", "float32", name, goluzen_folders(name), exact=True)


def test_command_line_on_a_folder_of_this_design(goluzen_folders, plain_backend, tmp_path):
    """`python -m mini_engine_amd.cli --model DIR`: the folder's config picks the model class; prompts in, greedy tokens out."""
    from mini_engine_amd import cli
    import helpers
    folder = goluzen_folders("mix")
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


def test_named_sizes_build():
    from mini_engine_amd.config.sizes import named_config
    cfg, full = named_config("goluzen:tinyA")
    model = build_model(cfg)
    assert [layer.kind for layer in cfg.layers] == ["attention", "latent_attention"] and full == 2 and model.layers[1].feed_forward.num_experts == 32
    cfg, _ = named_config("goluzen:0.6b", 8)
    plan = build_model(cfg).cache_plan()
    assert plan.call_writes == [True, True, False, True, False, False, True, True] and math.prod(plan.state_needs[2].shape) == 4 * 128 * 256
