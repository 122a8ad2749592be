"""Negosun on the GPU: the engine's cuts, batches, page reuse, long decoding, far keys and temperature steps in float32
and bfloat16 against the plain evaluation, decode steps replayed as graphs, greedy generation through the scheduler, the
trace program and the command line on a folder of this design. (Its kernels against their twins:
test_negosun_kernels_gpu.py.)"""
import pytest
import torch

import helpers
import negosun_cases as N
import test_trace_run as TR
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.kernels import ops
from mini_engine_amd.weights.loader import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 3e-5, torch.bfloat16: 8e-2}      # widths of 32-48 make bfloat16 noisy


@pytest.fixture(scope="module")
def negosun_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = N.make_folder(name, str(tmp_path_factory.mktemp(f"negosun_{name}")))
        return made[name]

    return get


class Env:
    def __init__(self, folders, dtype, graphs=False):
        self.folders, self.dtype, self.tol, self.models, self.graphs = folders, dtype, TOL[dtype], {}, graphs
        self.device = DEV

    def runner(self, name, pages, slots=0):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 1024)
        model = self.models[name]
        manager = CacheManager(pages, N.PAGE[name], ModelRunner.windows_of(model), num_state_slots=0, enable_prefix_caching=False)
        options = dict(use_graphs=True, mixed_graphs_after=1) if self.graphs else {}
        return ModelRunner(model, manager, self.dtype, self.device, 1024, poison_cache=True, **options), manager, folder


@pytest.fixture(scope="module", params=[torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def env(request, negosun_folders):
    return Env(negosun_folders, request.param)


@pytest.mark.parametrize("name", ["trio", "solo", "late"])
@pytest.mark.parametrize("case", N.ALL, ids=lambda c: c.__name__)
def test_cuts(env, case, name):
    case(env, name)


def test_far_keys_and_temperature_steps(env):
    N.far_keys(env)


@pytest.mark.parametrize("case", [N.whole, N.portions, N.batch_against_alone], ids=lambda c: c.__name__)
def test_mid_sizes(env, case):
    """Heads of 64 without padding, 64 experts of which six are used, the tiled expert kernels in bfloat16."""
    case(env, "mid")


def test_real_layer_sizes(negosun_folders):
    N.real_sizes(Env(negosun_folders, torch.float32), Env(negosun_folders, torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("case", [N.token_by_token, N.long_decode, N.batch_against_alone], ids=lambda c: c.__name__)
def test_cuts_through_captured_steps(negosun_folders, case, dtype):
    """The same with decode steps (and small steps that come up again) replayed as graphs: what one layer leaves for the
    others inside a step (the first mixing layer's values) lives inside the graph."""
    case(Env(negosun_folders, dtype, graphs=True), "trio")


def test_hip_libraries_are_the_ones_running(env):
    N.whole(env, "solo")
    assert ops.backend().name == "hip" and any("libme_core" in p for p in ops.loaded_libraries())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["trio", "late"])
def test_greedy_generation_through_the_scheduler(negosun_folders, dtype, name):
    N.greedy_through_the_engine(DEV, dtype, name, negosun_folders(name), exact=dtype == "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_program_on_this_design(negosun_folders, tmp_path, dtype):
    """bin/trace_run picks the model class by the folder's config: four live requests, portions beside single tokens,
    pages used again."""
    name = "trio"
    folder = negosun_folders(name)
    V = N.CONFIGS[name]["vocab"]
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
    TR.replay(folder, dtype, steps, out, max_tokens=TR.most_live_tokens(steps), page=N.PAGE[name])
    for r, g in TR.collect(steps, out, V).items():
        err = helpers.rel_err(g, N.plain_logits(folder, ids[r]))
        assert err <= TOL[getattr(torch, dtype)], f"{dtype} request {r}: {err:.3g}"


def test_offline_workload_row_with_random_weights(tmp_path, capsys):
    """The offline workload through the command line, on this design at a tiny size with random weights."""
    import json
    from mini_engine_amd import cli
    rc = cli.main(["--random-weights", "negosun:tinyA", "--num-seqs", "6", "--max-prompt", "40", "--max-output", "8",
                   "--max-model-len", "64", "--max-num-seqs", "4", "--budget", "32", "--tokens-out", "-",
                   "--out", str(tmp_path / "bench.jsonl")])
    assert rc == 0
    lines = capsys.readouterr().out.strip().splitlines()
    row = json.loads(lines[-1])
    tokens = [json.loads(line) for line in lines[-7:-1]]
    assert [len(t) for t in tokens] == [8] * 6 and all(0 <= t < 256 for ts in tokens for t in ts)
    assert row["num_seqs"] == 6 and row["output_tokens"] == 48 and row["throughput_tok_s"] > 0
