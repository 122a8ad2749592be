"""Sigosun on the CPU: configuration, checkpoint layout, and the engine's bookkeeping for it (pages, state slots,
batches, cuts, the scheduler) with the plain twins of the kernels in float32, against the plain evaluation."""
import json
import os

import pytest
import torch

import sigosun_cases as S
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.config.model_config import ConfigError, SigosunConfig, load_model_config
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.parts.rotary import RotaryEmbedding
from mini_engine_amd.registry import build_model
from mini_engine_amd.weights.loader import load_model


@pytest.fixture(scope="module")
def sigosun_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = S.make_folder(name, str(tmp_path_factory.mktemp(f"sigosun_{name}")))
        return made[name]

    return get


class Env:
    device, dtype, tol = "cpu", torch.float32, 2e-5

    def __init__(self, folders):
        self.folders, self.models = folders, {}

    def runner(self, name, pages, slots):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 512)
        model = self.models[name]
        manager = CacheManager(pages, S.PAGE[name], ModelRunner.windows_of(model), num_state_slots=slots, enable_prefix_caching=False)
        return ModelRunner(model, manager, self.dtype, self.device, 512, poison_cache=True), manager, folder


def test_config_reads_back_and_refuses_what_it_cannot_run(tmp_path):
    for name, raw in S.CONFIGS.items():
        cfg = SigosunConfig.from_dict(raw)
        assert SigosunConfig.from_dict(cfg.to_dict()) == cfg
        assert len(cfg.layers) == len(raw["layers"]) and cfg.vocab_size == raw["vocab"]
    with open(tmp_path / "config.json", "w") as f:
        json.dump(S.CONFIGS["mix"], f)
    assert isinstance(load_model_config(str(tmp_path)), SigosunConfig)          # chosen by the file's architecture name
    bad = json.loads(json.dumps(S.CONFIGS["mix"]))
    bad["layers"][3]["mixer"]["kv_from"] = 2                                    # not an attention layer
    with pytest.raises(ConfigError):
        SigosunConfig.from_dict(bad)
    bad = json.loads(json.dumps(S.CONFIGS["mix"]))
    bad["layers"][2]["mixer"]["decay"] = [0.5]
    with pytest.raises(ConfigError):
        SigosunConfig.from_dict(bad)
    bad = json.loads(json.dumps(S.CONFIGS["mix"]))
    del bad["layers"][0]["mixer"]["state"]
    with pytest.raises(ConfigError, match="state"):
        SigosunConfig.from_dict(bad)


def test_model_is_assembled_from_the_config():
    model = build_model(SigosunConfig.from_dict(S.CONFIGS["mix"]))
    plan = model.cache_plan()
    assert plan.call_group == [None, 0, None, 0, None] and plan.call_writes == [False, True, False, False, False]
    assert [s is not None for s in plan.state_needs] == [True, False, True, False, True]
    assert plan.state_needs[0].shape == (4 * 20 * 12 + (48 + 2 * 2 * 20) * 3,)       # matrices, then the convolution's inputs
    names = {src.name for sources in model.weight_sources.values() for src in sources}
    assert {"embed", "head", "final.norm", "l0.mix.in", "l0.mix.conv.b", "l1.mix.k.norm", "l1.mix.g", "l2.mix.norm", "l3.mix.q",
            "l0.mlp.up", "l1.norm2"} <= names
    assert not any(n.startswith("l3.mix.k") or n.startswith("l3.mix.v") or n.startswith("l2.mlp") for n in names)


def test_pages_behind_a_block_are_given_back():
    """A block mask keeps the pages of the block the next token falls into; a group that another layer reads under a
    mask of its own keeps what the loosest of the rules needs."""
    from mini_engine_amd.cache.manager import first_kept
    from mini_engine_amd.parts import CacheNeed
    assert first_kept(5, 3) == 0 and first_kept(5, 12) == 8
    assert [first_kept((("chunk", 7),), n) for n in (0, 6, 7, 13, 14)] == [0, 0, 7, 7, 14]
    assert [first_kept((("chunk", 7), ("chunk", 10)), n) for n in (9, 10, 13, 14, 20, 21)] == [0, 7, 7, 10, 14, 20]
    assert first_kept((("chunk", 8), ("window", 3)), 17) == 15
    need = CacheNeed.keys_and_values(2, 16, chunk=7)
    assert need.keep() == (("chunk", 7),) and CacheNeed.keys_and_values(2, 16, window=9).keep() == 9
    assert CacheNeed.keys_and_values(2, 16).keep() is None
    import dataclasses
    assert dataclasses.replace(need, readers=(("chunk", 10),)).keep() == (("chunk", 7), ("chunk", 10))
    assert dataclasses.replace(need, readers=(("all", 0),)).keep() is None          # a reader that sees every key
    model = build_model(SigosunConfig.from_dict(S.CONFIGS["mix"]))
    assert ModelRunner.windows_of(model) == [(("chunk", 7), ("chunk", 10))]
    manager = CacheManager(8, 8, ModelRunner.windows_of(model), num_state_slots=1, enable_prefix_caching=False)
    assert manager.allocate("r", 0, 30) and manager.block_table("r") == [0, 1, 2, 3]
    assert manager.allocate("r", 30, 1) and manager.block_table("r") == [-1, -1, -1, 3]     # blocks start at 28 and 30: keys from 28 on
    assert manager.allocate("r", 31, 10) and manager.block_table("r")[:3] == [-1, -1, -1] and manager.num_free_pages(0) == 5
    manager.check_invariants()


def test_head_order_of_rotations():
    assert RotaryEmbedding(16, 1e4).head_order() is None
    assert RotaryEmbedding(8, 1e4, interleaved=True).head_order() == [0, 2, 4, 6, 1, 3, 5, 7]
    # 4 of 10 stored dimensions turn, in 16 slots: the pairs half a head apart, the rest behind them, empty slots last
    order = RotaryEmbedding(16, 1e4, rotary_dims=4, interleaved=True, stored_dim=10).head_order()
    assert order == [0, 2, 4, 5, 6, 7, 8, 9, 1, 3, -1, -1, -1, -1, -1, -1]
    r = RotaryEmbedding(16, 100.0, rotary_dims=4, interleaved=True, stored_dim=10, exact_angles=True)
    r.finalize("cpu", torch.float32, 8)
    assert torch.equal(r.table[:, 2:, 0], torch.ones(8, 6)) and torch.equal(r.table[:, 2:, 1], torch.zeros(8, 6))
    assert abs(float(r.table[3, 1, 1]) - float(torch.sin(torch.tensor(3 * 100.0 ** -0.5, dtype=torch.float64)))) < 1e-7


@pytest.mark.parametrize("name", ["mix", "odd", "att", "ssm", "lin"])
@pytest.mark.parametrize("case", S.ALL, ids=lambda c: c.__name__)
def test_cuts(sigosun_folders, plain_backend, case, name):
    case(Env(sigosun_folders), name)


def test_far_keys_and_block_edges(sigosun_folders, plain_backend):
    S.far_keys(Env(sigosun_folders))


@pytest.mark.parametrize("name", ["mix", "lin"])
def test_greedy_generation_through_the_scheduler(sigosun_folders, plain_backend, name):
    S.greedy_through_the_engine("cpu", "float32", name, sigosun_folders(name), exact=True)


def test_command_line_on_a_folder_of_this_design(sigosun_folders, plain_backend, tmp_path, capsys):
    """`python -m mini_engine_amd.cli --model DIR`: the folder's config picks the model class; prompts in, greedy tokens out."""
    from mini_engine_amd import cli
    import helpers
    folder = sigosun_folders("mix")
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
            assert tok == int(S.plain_logits(folder, seq)[-1].argmax())
            seq.append(tok)


def test_launch_rules_of_the_recurrence():
    """Whatever the step, the spans cover the longest request, keep 64 tokens or more in whole batches of the kernel's 8,
    and stay within one launch; the rows a wave keeps are a size the kernel is built for and cover N."""
    from mini_engine_amd.kernels import ops
    import random
    rng = random.Random(0)
    for _ in range(2000):
        q_lens = [rng.choice((1, 2, 17, 63, 64, 127, 128, 129, 700, 5000, 40000)) for _ in range(rng.randint(1, 40))]
        waves = rng.choice((1, 4, 64, 128, 1024))
        span, spans = ops.recurrence_spans(q_lens, waves)
        if spans == 1:
            assert span == 0 and (max(q_lens) < 128 or -(-sum(q_lens) // max(1, 4096 // waves)) >= max(q_lens))
        else:
            assert span >= 64 and span % 8 == 0 and spans * span >= max(q_lens) and (spans - 1) * span < max(q_lens)
            assert spans * 4 <= 65535
    for N in list(range(1, 300)) + [512, 1000, 4096]:
        rows = ops.recurrence_rows_per_wave(N)
        assert rows in (16, 32, 48, 64) and -(-N // rows) * rows >= N and -(-N // rows) * rows - N < rows
