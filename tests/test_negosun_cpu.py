"""Negosun on the CPU: configuration, checkpoint layout, each mechanism's twin against the plain evaluation's function,
and the engine's bookkeeping for the design (pages, batches, cuts, the scheduler) with the plain twins of the kernels in
float32, against the plain evaluation."""
import json

import pytest
import torch

import kernel_twins as twin
import negosun_cases as N
import plain_negosun as P
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.config.model_config import ConfigError, NegosunConfig, load_model_config
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.registry import build_model
from mini_engine_amd.weights.loader import load_model


@pytest.fixture(scope="module")
def negosun_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = N.make_folder(name, str(tmp_path_factory.mktemp(f"negosun_{name}")))
        return made[name]

    return get


class Env:
    device, dtype, tol = "cpu", torch.float32, 2e-5

    def __init__(self, folders):
        self.folders, self.models = folders, {}

    def runner(self, name, pages, slots=0):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 512)
        model = self.models[name]
        manager = CacheManager(pages, N.PAGE[name], ModelRunner.windows_of(model), num_state_slots=0, enable_prefix_caching=False)
        return ModelRunner(model, manager, self.dtype, self.device, 512, poison_cache=True), manager, folder


def test_config_reads_back_and_refuses_what_it_cannot_run(tmp_path):
    for name, raw in N.CONFIGS.items():
        cfg = NegosunConfig.from_dict(raw)
        assert NegosunConfig.from_dict(cfg.to_dict()) == cfg
        assert len(cfg.layers) == len(raw["layers"]) and cfg.vocab_size == raw["vocab"]
    with open(tmp_path / "config.json", "w") as f:
        json.dump(N.CONFIGS["trio"], f)
    assert isinstance(load_model_config(str(tmp_path)), NegosunConfig)           # chosen by the file's architecture name
    for path, value in ((("layers", 2, "mixer", "vdim"), 40),                      # 1 x 40 value dimensions beside 2 x 40
                        (("layers", 0, "mlp", "router", "groups", "count"), 4),    # 9 experts in 4 groups
                        (("layers", 0, "mlp", "router", "top"), 7),                # more than the two kept groups hold
                        (("layers", 0, "mixer", "heads"), 3),                      # 3 heads on 2 key heads
                        (("layers", 1, "type"), "mamba2")):
        bad = json.loads(json.dumps(N.CONFIGS["trio"]))
        at = bad
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError):
            NegosunConfig.from_dict(bad)
    bad = json.loads(json.dumps(N.CONFIGS["trio"]))
    del bad["layers"][0]["mixer"]["scale"]
    with pytest.raises(ConfigError, match="scale"):
        NegosunConfig.from_dict(bad)


def test_model_is_assembled_from_the_config():
    model = build_model(NegosunConfig.from_dict(N.CONFIGS["late"]))
    plan = model.cache_plan()
    assert plan.call_writes == [True] * 4 and len(plan.group_needs) == 4            # four layers of unlike head sizes: four page groups
    assert [layer.mixer.value_mix for layer in model.layers] == [None, "first", None, "blend"]
    assert [layer.feed_forward is None for layer in model.layers] == [False, False, True, False]
    assert model.layers[1].feed_forward.shared is not None and model.layers[0].feed_forward.shared is None
    assert model.head.tied_to is model.embedding and model.head.softcap == 30.0
    names = {src.name for sources in model.weight_sources.values() for src in sources}
    assert {"embed", "final.norm", "l0.mix.q.b", "l0.mix.k.norm", "l3.mix.vmix", "l1.mlp.e8.down", "l1.mlp.shared.up", "l1.mlp.router",
            "l0.ls1", "l0.ls2", "l2.ls1", "l1.norm2"} <= names
    assert not ({"l1.mix.vmix", "l2.ls2", "l2.norm2", "head"} & names) and "l1.mix.vmix" in model.optional_sources


# ---------------------------------------------------------------- each mechanism: the twin against the plain function

def test_router_twin_against_the_plain_choice():
    torch.manual_seed(3)
    for E, top, groups in ((6, 2, {"count": 3, "keep": 2}), (8, 1, {"count": 4, "keep": 1}), (5, 5, None), (12, 3, {"count": 2, "keep": 1}),
                           (9, 2, {"count": 1, "keep": 1})):
        w = torch.randn(E, 20, dtype=torch.float64)
        for _ in range(40):
            u = torch.randn(20, dtype=torch.float64)
            scores = torch.softmax(w @ u, 0)
            chosen = P.choose(scores, top, groups)
            ids, wt = twin.moe_route(u[None], w, top, groups["count"] if groups else 1, groups["keep"] if groups else 1)
            assert ids[0].tolist() == chosen
            assert torch.allclose(wt[0].double(), scores[chosen] / scores[chosen].sum(), atol=1e-6)
    # ties go to the lower index, in groups and in experts
    ids, wt = twin.moe_route(torch.zeros(1, 4), torch.ones(6, 4), 2, 3, 1)
    assert ids[0].tolist() == [0, 1] and P.choose(torch.full((6,), 1 / 6), 2, {"count": 3, "keep": 1}) == [0, 1]


def test_experts_twin_against_the_plain_sum():
    torch.manual_seed(4)
    E, top, F, h, T = 5, 2, 12, 16, 7
    w = {"m.router": torch.randn(E, h, dtype=torch.float64)}
    for e in range(E):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"] = (torch.randn(F, h, dtype=torch.float64), torch.randn(F, h, dtype=torch.float64),
                                                                 torch.randn(h, F, dtype=torch.float64))
    x = torch.randn(T, h, dtype=torch.float64)
    ids, wt = twin.moe_route(x, w["m.router"], top)
    gate_up = torch.stack([torch.cat((w[f"m.e{e}.gate"], w[f"m.e{e}.up"])) for e in range(E)])
    down = torch.stack([w[f"m.e{e}.down"] for e in range(E)])
    got = twin.routed_experts(x, ids, wt, gate_up, down).sum(0)
    want = torch.stack([P.experts(w, "m", {"router": {"experts": E, "top": top}}, x[t]) for t in range(T)])
    assert torch.allclose(got.double(), want, rtol=1e-4, atol=1e-4)


def test_prologue_twin_against_the_plain_projection():
    """Bias, the norm over all heads at once, the temperature's steps and the blend of values, heads padded to 16 slots."""
    torch.manual_seed(5)
    Hq, Hkv, n, nv, D, T, eps = 3, 2, 10, 6, 16, 9, 1e-5
    mixer = {"q_temp": {"coef": 0.7, "every": 4}}
    w = {"q": torch.randn(Hq * n, 8, dtype=torch.float64), "k": torch.randn(Hkv * n, 8, dtype=torch.float64), "v": torch.randn(Hkv * nv, 8, dtype=torch.float64)}
    for name, size in (("q", Hq * n), ("k", Hkv * n), ("v", Hkv * nv)):
        w[name + ".b"] = torch.randn(size, dtype=torch.float64)
        w[name + ".norm"] = torch.rand(size, dtype=torch.float64) + 0.5
    u = torch.randn(T, 8, dtype=torch.float64)
    first = torch.randn(T, Hkv * nv)
    lam = torch.tensor(0.3)

    def slots(block, heads, size):           # [T, heads * size] -> [T, heads * D] with zeros behind every head
        return torch.cat((block.view(T, heads, size), block.new_zeros(T, heads, D - size)), 2).reshape(T, heads * D)

    rows = torch.cat((slots(u @ w["q"].T, Hq, n), slots(u @ w["k"].T, Hkv, n), slots(u @ w["v"].T, Hkv, nv)), 1).float()
    one = lambda name, heads, size: slots(w[name][None].expand(T, -1), heads, size)[0].float()
    bias = torch.cat((one("q.b", Hq, n), one("k.b", Hkv, n), one("v.b", Hkv, nv)))
    positions = torch.tensor([0, 2, 3, 4, 6, 7, 8, 11, 40], dtype=torch.int32)
    kc, vc = torch.zeros(T, Hkv, 1, D), torch.zeros(T, Hkv, D, 1)
    q = twin.qkv_prepare_store(rows, bias, one("q.norm", Hq, n), one("k.norm", Hkv, n), eps, Hq * n, Hkv * n, (0.7, 4), positions,
                               torch.arange(T, dtype=torch.int32), kc, vc, Hq, Hkv, D, 1, nv, 2, lam, first)
    for t in range(T):
        want_q = P.project(w, "q", u[t], eps, True) * P.temperature(mixer, int(positions[t]))
        want_k = P.project(w, "k", u[t], eps, True)
        want_v = 0.7 * P.project(w, "v", u[t], eps, False) + 0.3 * first[t].double()
        assert torch.allclose(q[t].view(Hq, D)[:, :n].reshape(-1).double(), want_q, atol=1e-5)
        assert torch.allclose(kc[t, :, 0, :n].reshape(-1).double(), want_k, atol=1e-5)
        assert torch.allclose(vc[t, :, :nv, 0].reshape(-1).double(), want_v, atol=1e-5)
    assert P.temperature(mixer, 2) == 1.0 and P.temperature(mixer, 3) > 1.0            # position 3 is the first of the second step


def test_block_sum_twin():
    torch.manual_seed(6)
    T, n = 4, 10
    stream, a, b, c = torch.randn(T, n), torch.randn(T, n), torch.randn(2, T, n), torch.randn(T, n)
    s1, s2, w1, w2 = torch.rand(n), torch.rand(n), torch.rand(n) + 0.5, torch.rand(n) + 0.5
    new, y1, y2 = twin.scaled_sum_norm(stream, [(a, s1), (b, s2), (c, s2)], 0.45, w1, w2, 1e-5, torch.float32)
    want = stream.double() + 0.45 * (s1 * a + s2 * (b.sum(0) + c)).double()
    assert torch.allclose(new.double(), want, atol=1e-6)
    for t in range(T):
        assert torch.allclose(y1[t].double(), P.unit_rms(want[t], 1e-5) * w1, atol=1e-6)
        assert torch.allclose(y2[t].double(), P.unit_rms(want[t], 1e-5) * w2, atol=1e-6)


# ---------------------------------------------------------------- the engine

@pytest.mark.parametrize("name", ["trio", "solo", "late"])
@pytest.mark.parametrize("case", N.ALL, ids=lambda c: c.__name__)
def test_cuts(negosun_folders, plain_backend, case, name):
    case(Env(negosun_folders), name)


def test_far_keys_and_temperature_steps(negosun_folders, plain_backend):
    N.far_keys(Env(negosun_folders))


def test_a_lost_mechanism_shows(negosun_folders, plain_backend):
    """The tests' weights make every mechanism matter: the plain evaluation without one of them is far from the engine."""
    env = Env(negosun_folders)
    runner, manager, folder = env.runner("trio", 8)
    ids = N.random_ids(40, 97, 77)
    d = N.Driver(runner, manager)
    d.step({"r": ids})
    got = d.result("r")
    cfg, w = P.read_folder(folder)
    assert N.rel_err(got, P.logits(cfg, w, ids)) <= env.tol
    for what in ("bias", "temperature", "mix", "scale", "groups", "shared", "cap"):
        c, v = json.loads(json.dumps(cfg)), dict(w)
        if what == "bias":
            v = {k: (t * 0 if k.endswith(".b") else t) for k, t in w.items()}
        elif what == "temperature":
            c["layers"][0]["mixer"].pop("q_temp")
        elif what == "mix":
            c["layers"][2]["mixer"]["v_mix"] = False
        elif what == "scale":
            v = {k: (t * 0 + 1 if k.endswith(".ls2") else t) for k, t in w.items()}
        elif what == "groups":
            c["layers"][0]["mlp"]["router"].pop("groups")
        elif what == "shared":
            c["layers"][0]["mlp"].pop("shared")
        else:
            c.pop("logit_softcap")
        assert N.rel_err(got, P.logits(c, v, ids)) > 10 * env.tol, f"the plain evaluation without its {what} is as close as with it"


@pytest.mark.parametrize("name", ["trio", "late"])
def test_greedy_generation_through_the_scheduler(negosun_folders, plain_backend, name):
    N.greedy_through_the_engine("cpu", "float32", name, negosun_folders(name), exact=True)


def test_command_line_on_a_folder_of_this_design(negosun_folders, plain_backend, tmp_path):
    """`python -m mini_engine_amd.cli --model DIR`: the folder's config picks the model class; prompts in, greedy tokens out."""
    from mini_engine_amd import cli
    import helpers
    folder = negosun_folders("trio")
    prompts = [helpers.random_ids(n, 97, 950 + n) for n in (3, 19, 41)]
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
            assert tok == int(N.plain_logits(folder, seq)[-1].argmax())
            seq.append(tok)


def test_launch_rules_of_the_routed_experts():
    """Whatever the step: tiles of a size the kernels are built for, small ones while experts get few rows, and the tile
    count the launches are sized by holds every expert's tiles however the pairs fall; the kernel that orders the pairs
    chooses only for steps and expert counts that fit its one workgroup."""
    from mini_engine_amd.kernels import ops
    import random
    rng = random.Random(1)
    for _ in range(3000):
        T, top, E = rng.choice((1, 2, 7, 64, 65, 300, 2048, 16384)), rng.choice((1, 2, 4, 8)), rng.choice((2, 8, 32, 60, 256))
        top = min(top, E)
        rows = ops.expert_tile_rows(T, top, E)
        assert rows in (16, 64, 128)
        assert rows == 16 or T * top > 16 * E and (rows == 64 or T * top >= 128 * E)
        # the worst split of the pairs over the experts: every expert that has pairs ends in a tile that is not full
        counts = [0] * E
        for _ in range(T * top if T * top < 200 else 200):
            counts[rng.randrange(E)] += max(1, T * top // 200)
        counts[0] += T * top - sum(counts) if sum(counts) <= T * top else 0
        if sum(counts) == T * top:
            assert sum(-(-c // rows) for c in counts) <= T * top // rows + min(E, T * top)
    assert ops.moe_sort_chooses(1, 32, 4) and ops.moe_sort_chooses(64, 256, 8)
    assert not ops.moe_sort_chooses(65, 32, 4) and not ops.moe_sort_chooses(4, 1024, 1)
