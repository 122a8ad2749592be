"""The Sigosun design in the engine against its plain evaluation (tests/plain_sigosun.py), under every way of
cutting the work. Each case takes `env` with .device, .dtype, .tol and .runner(name, pages, slots) -> (runner,
manager, folder); the same cases run on the CPU (plain kernel twins, float32) and on the GPU (HIP kernels, float32
and bfloat16). Pools start filled with NaN, so a read of a key or state nobody wrote poisons the logits.

The configurations are the tests' own and differ from each other in every size: key and value sizes that differ,
heads that are not powers of two, rotations of part of a head, block masks of 5 to 300 positions, one and several
groups, state sizes above and below a wave's 64 rows, value sizes above 64, convolutions of 2 to 4 taps, layers
with and without feed-forward, a layer on another layer's keys with a mask of its own. The stored q norms are
scaled up so that the softmax is peaked: a key that is wrongly seen or wrongly hidden then moves the logits far
beyond the tolerance, also among hundreds of keys.
"""
from __future__ import annotations

import json
import os

import torch

import helpers
import plain_sigosun
from helpers import Driver, random_ids, rel_err
from mini_engine_amd.config.model_config import SigosunConfig
from mini_engine_amd.weights.random_init import write_random_model


def _att(heads, kv, dim, vdim, scale, rot, base, mask, kv_from=None, ff=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": mask}}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _ssm(heads, vdim, state, groups, conv, norm_groups, ff=None):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _lin(heads, dim, vdim, decay, ff=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _model(vocab, width, eps, layers):
    return {"architecture": "Sigosun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


CONFIGS = {
    # every mixer, in an order of its own; key size 24 against value size 40, 8 of 24 dimensions turn, no grouping of
    # heads; the layer on layer 1's keys has a mask of another size and no feed-forward; two groups, two norm groups
    "mix": _model(97, 48, 1e-5, [
        _ssm(4, 12, 20, 2, 4, 2, ff=80),
        _att(4, 4, 24, 40, 0.3, 8, 5000.0, 7, ff=56),
        _lin(3, 10, 20, [0.5, 0.93, 0.998]),
        _att(4, 4, 24, 40, 0.2, 8, 5000.0, 10, kv_from=1),
        _ssm(2, 8, 16, 1, 2, 1),
    ]),
    # attention first, its keys larger than its values, five query heads on one key head, an odd vocabulary; three groups
    # and three norm groups; a feed-forward behind the linear attention; the reader's mask is the smaller one
    "odd": _model(301, 72, 1e-6, [
        _att(5, 1, 48, 32, 0.17, 16, 30000.0, 33),
        _lin(2, 40, 24, [0.7, 0.99], ff=100),
        _ssm(6, 20, 24, 3, 2, 3),
        _att(5, 1, 48, 32, 0.21, 16, 30000.0, 9, kv_from=0, ff=64),
    ]),
    # each mechanism alone
    "att": _model(64, 32, 1e-6, [_att(9, 3, 16, 16, 0.25, 16, 10000.0, 5, ff=48)]),
    "ssm": _model(64, 36, 1e-5, [_ssm(3, 80, 70, 1, 3, 1)]),          # value size above 64, state above 64 rows, a width that is no multiple of 8
    "lin": _model(64, 24, 1e-5, [_lin(2, 72, 8, [0.8, 0.9995])]),     # key size above 64: two slices of the state
    # long blocks: keys far back among hundreds; 1 key head for 3 query heads; key size 32 against value size 16
    "far": _model(80, 32, 1e-5, [_att(3, 1, 32, 16, 0.2, 32, 400000.0, 300, ff=40), _lin(1, 16, 16, [0.9985]),
                                 _att(3, 1, 32, 16, 0.2, 32, 400000.0, 64, kv_from=0, ff=40)]),
}
# the layer sizes of a real model (heads of 128, a state of 128 x 64, four taps), few layers: the kernel forms that
# the small widths above never reach
CONFIGS["real"] = _model(1000, 512, 1e-6, [
    _lin(4, 128, 128, [0.9, 0.97, 0.99, 0.9975]),
    _att(8, 2, 128, 128, 128 ** -0.5, 64, 1e6, 256, ff=1024),
    _ssm(16, 64, 128, 1, 4, 1),
    _att(8, 2, 128, 128, 128 ** -0.5, 64, 1e6, 100, kv_from=1, ff=1024),
])
SEEDS = {"real": 16, "odd": 17, "mix": 11, "att": 12, "ssm": 13, "lin": 14, "far": 15}
PAGE = {"real": 16, "odd": 16, "mix": 8, "att": 16, "ssm": 16, "lin": 8, "far": 16}
SHARPEN = 3.0


def make_folder(name: str, path: str) -> str:
    """A model folder with seeded random weights, the q norms scaled up by SHARPEN."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    write_random_model(SigosunConfig.from_dict(CONFIGS[name]), SEEDS[name], path, torch.bfloat16)
    file = os.path.join(path, "model.safetensors")
    with safe_open(file, "pt", device="cpu") as f:
        tensors = {k: f.get_tensor(k) for k in f.keys()}
    for k in tensors:
        if k.endswith(".mix.q.norm"):
            tensors[k] = (tensors[k].float() * SHARPEN).to(tensors[k].dtype)
    save_file(tensors, file, metadata={"format": "pt"})
    return path


_plain: dict = {}


def plain_logits(folder: str, ids: list) -> torch.Tensor:
    key = (folder, tuple(ids))
    if key not in _plain:
        if folder not in _plain:
            _plain[folder] = plain_sigosun.read_folder(folder)
        cfg, w = _plain[folder]
        _plain[key] = plain_sigosun.logits(cfg, w, ids)
    return _plain[key]


def _free_pages(manager) -> int:
    """Free pages of the scarcest group; a model without attention has no pages at all."""
    return min((manager.num_free_pages(g) for g in range(manager.num_groups)), default=1 << 30)


def _vocab(name):
    return CONFIGS[name]["vocab"]


def _check(env, folder, ids, got, what):
    ref = plain_logits(folder, ids)[: got.shape[0]]
    err = rel_err(got, ref)
    assert err <= env.tol, f"{what}: error {err:.3g} > {env.tol:g}; first bad position {helpers.first_bad_row(got, ref, env.tol)}"


def whole(env, name):
    """Each request alone and whole: one token, lengths around pages, around the masks' edges and the kernels' tiles."""
    page = PAGE[name]
    for n in (1, 2, page, page + 1, 21, 50, 83):
        runner, manager, folder = env.runner(name, -(-n // page), 1)
        ids = random_ids(n, _vocab(name), 100 + n)
        d = Driver(runner, manager)
        d.step({"r": ids}, end=["r"])
        _check(env, folder, ids, d.result("r"), f"{name} whole n={n}")


def token_by_token(env, name):
    """A whole request decoded one token at a time from its first token, against the same request in one step."""
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
    """Portions of changing size, down to two tokens and one, cut inside pages, blocks of the masks and the
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
            plan = patterns[r]
            done_prompt = sum(plan)
            if pos[r] < done_prompt:
                acc = 0
                for c in plan:
                    if acc == pos[r]:
                        take = c
                        break
                    acc += c
            else:
                take = 1
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
    """A short prompt, then many single tokens: over page borders, over several blocks of the masks, far beyond the
    convolution's reach."""
    page = PAGE[name]
    n = 140
    ids = random_ids(n, _vocab(name), 500)
    runner, manager, folder = env.runner(name, -(-n // page), 1)
    d = Driver(runner, manager)
    d.step({"r": ids[:6]})
    for t in range(6, n):
        d.step({"r": ids[t:t + 1]})
    _check(env, folder, ids, d.result("r"), f"{name} long decode")


def far_keys(env, name="far"):
    """Blocks of 300 positions: queries whose best key lies hundreds of positions back, in a prompt, in a portion
    behind a long prefix and decoded alone; around the block's edge (positions 299, 300, 301) the keys before it
    must vanish."""
    page = PAGE[name]
    n = 330
    ids = random_ids(n, _vocab(name), 600)
    runner, manager, folder = env.runner(name, 2 * -(-n // page), 2)
    d = Driver(runner, manager)
    d.step({"w": ids})
    d.step({"r": ids[:290]})
    d.step({"r": ids[290:298]})
    for t in range(298, 304):
        d.step({"r": ids[t:t + 1]})
    d.step({"r": ids[304:]})
    _check(env, folder, ids, d.result("w"), f"{name} whole")
    _check(env, folder, ids, d.result("r"), f"{name} cut around the block's edge")


def real_sizes(env_f32, env_bf16, name="real"):
    """At the layer sizes of a real model: float32 against the plain evaluation on a short prompt; then a prompt of 700
    tokens (spans of the recurrence side by side, several blocks of both masks) whole, in portions and with its
    last tokens decoded, bfloat16 against float32 of the same engine."""
    page = PAGE[name]
    V = _vocab(name)
    short = random_ids(40, V, 900)
    runner, manager, folder = env_f32.runner(name, 8, 1)
    d = Driver(runner, manager)
    d.step({"s": short[:33]})
    d.step({"s": short[33:34]})
    d.step({"s": short[34:]}, end=["s"])
    _check(env_f32, folder, short, d.result("s"), f"{name} short prompt in float32")
    n = 700
    ids = random_ids(n, V, 901)
    got = {}
    for env in (env_f32, env_bf16):
        runner, manager, folder = env.runner(name, 2 * -(-n // page), 2)
        d = Driver(runner, manager)
        d.step({"w": ids})
        d.step({"r": ids[:300]})
        d.step({"r": ids[300:302]})
        d.step({"r": ids[302:680]})
        for t in range(680, n):
            d.step({"r": ids[t:t + 1]})
        got[env.dtype] = (d.result("w"), d.result("r"))
    (wf, rf), (wb, rb) = got[torch.float32], got[torch.bfloat16]
    assert rel_err(rf, wf.double().cpu()) <= 1e-4, "float32: the cut request differs from the whole one"
    assert rel_err(wb, wf.double().cpu()) <= env_bf16.tol and rel_err(rb, wf.double().cpu()) <= env_bf16.tol


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
    assert len(llm.manager.free_slots) == 3 and _free_pages(llm.manager) in (24, 1 << 30)
    for p, o in zip(prompts, outs):
        seq = list(p)
        assert len(o["token_ids"]) == 12
        for tok in o["token_ids"]:
            z = plain_logits(folder, seq)[-1]
            best = int(z.argmax())
            close = not exact and float(z[best] - z[tok]) < 8e-2 * float(z.abs().max())
            assert tok == best or close, f"{name} {dtype_name}: generated {tok}, the plain evaluation gives {best}"
            seq.append(tok)
