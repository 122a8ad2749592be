"""The Negosun design in the engine against its plain evaluation (tests/plain_negosun.py), under every way of cutting
the work. Each case takes `env` with .device, .dtype, .tol and .runner(name, pages) -> (runner, manager, folder); the
same cases run on the CPU (plain kernel twins, float32) and on the GPU (HIP kernels, float32 and bfloat16). Pools start
filled with NaN, so a read of a key nobody wrote poisons the logits.

The configurations are the tests' own and differ from each other, and from layer to layer, in every size: key and value
sizes that differ, several key/value heads, layers with and without a feed-forward, with and without a temperature,
value mixing that starts at the first layer or later, groups of experts of which one or two are kept, all experts
chosen, with and without a shared expert, with and without a cap on the logits. The stored weights are changed so
that a fault shows: q norms scaled up (a peaked softmax: a key wrongly seen or hidden moves the logits far beyond the
tolerance, also among hundreds of keys), biases and routers scaled up (a lost bias matters, and expert choices are no
close calls).
"""
from __future__ import annotations

import os

import torch

import helpers
import plain_negosun
from helpers import Driver, random_ids, rel_err
from mini_engine_amd.config.model_config import NegosunConfig
from mini_engine_amd.weights.random_init import write_random_model


def _layer(heads, kv, dim, vdim, scale, temp=None, v_mix=False, moe=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m, "mlp": moe}


def _moe(experts, top, ff, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def _model(vocab, width, eps, mult, cap, layers):
    d = {"architecture": "Negosun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}
    if cap is not None:
        d["logit_softcap"] = cap
    return d


CONFIGS = {
    # three unlike layers: two key/value heads of 24 against values of 40, then no feed-forward and no temperature, then one
    # key/value head with values of 80 and every expert chosen; two of three groups kept; temperatures that step every 5 and 16
    "trio": _model(97, 48, 1e-5, 0.45, 9.0, [
        _layer(4, 2, 24, 40, 0.3, temp=(0.7, 5), v_mix=True, moe=_moe(9, 3, 40, groups=(3, 2), shared=56)),
        _layer(2, 2, 16, 40, 0.4, v_mix=True),
        _layer(6, 1, 32, 80, 0.2, temp=(0.3, 16), v_mix=True, moe=_moe(4, 4, 24)),
    ]),
    # one layer alone: no mixing, no temperature, no cap, multiplier 1; one expert per token out of the best of four groups
    "solo": _model(64, 40, 1e-6, 1.0, None, [_layer(3, 3, 16, 16, 0.25, moe=_moe(8, 1, 48, groups=(4, 1), shared=24))]),
    # mixing starts at the second layer and skips the third; odd sizes (a width and feed-forwards that are no multiples of 8)
    "late": _model(301, 36, 1e-6, 0.8, 30.0, [
        _layer(2, 1, 20, 12, 0.3, temp=(1.0, 3), moe=_moe(5, 2, 20)),
        _layer(4, 4, 8, 6, 0.5, v_mix=True, moe=_moe(9, 3, 12, groups=(3, 1), shared=10)),
        _layer(2, 2, 16, 16, 0.3),
        _layer(3, 1, 48, 24, 0.15, temp=(0.2, 7), v_mix=True, moe=_moe(2, 1, 28)),
    ]),
    # long contexts: three query heads on one key head, the temperature steps every 64 positions
    "far": _model(80, 32, 1e-5, 0.5, 20.0, [
        _layer(3, 1, 32, 16, 0.2, temp=(0.5, 64), v_mix=True, moe=_moe(4, 2, 40, groups=(2, 1))),
        _layer(3, 1, 32, 16, 0.2, temp=(0.5, 64), v_mix=True, moe=_moe(4, 2, 40, shared=16)),
    ]),
}
# mid sizes: heads of 64 on the matrix-core attention kernels without padding, 64 experts in eight groups of which three are
# kept, six per token, rows in whole 16-byte pieces (the tiled expert kernels in bfloat16); layers that differ
CONFIGS["mid"] = _model(1000, 256, 1e-6, 0.7, 12.0, [
    _layer(8, 4, 64, 64, 0.125, temp=(0.4, 32), v_mix=True, moe=_moe(64, 6, 32, groups=(8, 3), shared=64)),
    _layer(4, 2, 64, 128, 0.125, v_mix=True),
    _layer(8, 4, 64, 64, 0.125, temp=(0.4, 32), v_mix=True, moe=_moe(24, 2, 48, groups=(4, 1))),
    _layer(8, 8, 32, 32, 0.2, v_mix=True, moe=_moe(10, 3, 40, shared=16)),
])
# the layer sizes of a real model (heads of 128, experts of 256 in four groups), two layers: the kernel forms that the
# small widths above never reach
CONFIGS["real"] = _model(1000, 512, 1e-6, 0.6, 25.0, [
    _layer(8, 2, 128, 128, 128 ** -0.5, temp=(0.1, 256), v_mix=True, moe=_moe(16, 4, 256, groups=(4, 2), shared=512)),
    _layer(8, 2, 128, 128, 128 ** -0.5, temp=(0.1, 256), v_mix=True, moe=_moe(16, 4, 256, groups=(4, 2), shared=512)),
])
SEEDS = {"trio": 21, "solo": 22, "late": 23, "far": 24, "real": 25, "mid": 26}
PAGE = {"trio": 8, "solo": 16, "late": 16, "far": 16, "real": 16, "mid": 16}
SHARPEN, BIAS_UP, ROUTER_UP = 3.0, 15.0, 40.0


def make_folder(name: str, path: str) -> str:
    """A model folder with seeded random weights: q norms, biases and routers scaled up (see the module text)."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    write_random_model(NegosunConfig.from_dict(CONFIGS[name]), SEEDS[name], path, torch.bfloat16)
    file = os.path.join(path, "model.safetensors")
    with safe_open(file, "pt", device="cpu") as f:
        tensors = {k: f.get_tensor(k) for k in f.keys()}
    for k in tensors:
        up = SHARPEN if k.endswith(".mix.q.norm") else BIAS_UP if k.endswith(".b") else ROUTER_UP if k.endswith(".router") else None
        if up:
            tensors[k] = (tensors[k].float() * up).to(tensors[k].dtype)
    save_file(tensors, file, metadata={"format": "pt"})
    return path


_plain: dict = {}


def plain_logits(folder: str, ids: list) -> torch.Tensor:
    key = (folder, tuple(ids))
    if key not in _plain:
        if folder not in _plain:
            _plain[folder] = plain_negosun.read_folder(folder)
        cfg, w = _plain[folder]
        _plain[key] = plain_negosun.logits(cfg, w, ids)
    return _plain[key]


def _free_pages(manager) -> int:
    return min(manager.num_free_pages(g) for g in range(manager.num_groups))


def _vocab(name):
    return CONFIGS[name]["vocab"]


def _check(env, folder, ids, got, what):
    ref = plain_logits(folder, ids)[: got.shape[0]]
    err = rel_err(got, ref)
    assert err <= env.tol, f"{what}: error {err:.3g} > {env.tol:g}; first bad position {helpers.first_bad_row(got, ref, env.tol)}"


def whole(env, name):
    """Each request alone and whole: one token, lengths around pages and around the temperature's steps."""
    page = PAGE[name]
    for n in (1, 2, page, page + 1, 21, 50, 83):
        runner, manager, folder = env.runner(name, -(-n // page))
        ids = random_ids(n, _vocab(name), 100 + n)
        d = Driver(runner, manager)
        d.step({"r": ids}, end=["r"])
        _check(env, folder, ids, d.result("r"), f"{name} whole n={n}")


def token_by_token(env, name):
    """A whole request decoded one token at a time from its first token, beside the same request in one step."""
    page = PAGE[name]
    n = 45
    ids = random_ids(n, _vocab(name), 200)
    runner, manager, folder = env.runner(name, 2 * -(-n // page))
    d = Driver(runner, manager)
    for t in range(n):
        d.step({"r": ids[t:t + 1]})
    d.step({"w": ids})
    _check(env, folder, ids, d.result("r"), f"{name} token by token")
    _check(env, folder, ids, d.result("w"), f"{name} whole beside it")


def portions(env, name):
    """Portions of changing size, down to two tokens and one, cut inside pages and between the temperature's steps."""
    page = PAGE[name]
    n = 90
    ids = random_ids(n, _vocab(name), 300)
    for pattern in ([2, 3, 5, 8, 13, 21, 2, 2], [17, 2, 1, 1, 2, 31, 2], [page, 2, page + 1, page - 1]):
        runner, manager, folder = env.runner(name, -(-n // page))
        d = Driver(runner, manager)
        pos, i = 0, 0
        while pos < n:
            c = min(pattern[i % len(pattern)], n - pos)
            d.step({"r": ids[pos:pos + c]})
            pos += c; i += 1
        _check(env, folder, ids, d.result("r"), f"{name} portions {pattern}")


def batch_against_alone(env, name):
    """Unequal requests in one batch, portions beside single tokens, against the plain evaluation of each alone; the pages
    of ended requests are taken by later ones while others are live."""
    page = PAGE[name]
    V = _vocab(name)
    lens = {"a": 40, "b": 23, "c": 9, "d": 61, "e": 30, "f": 1, "g": 17}
    ids = {r: random_ids(n, V, 400 + i) for i, (r, n) in enumerate(lens.items())}
    need = lambda r: -(-lens[r] // page)
    runner, manager, folder = env.runner(name, need("a") + need("d") + need("e"))
    d = Driver(runner, manager)
    waiting, live, pos = list(lens), [], {}
    patterns = {"a": [11, 2, 9], "b": [23], "c": [2, 2, 5], "d": [7, 16, 3, 20], "e": [30], "f": [1], "g": [5, 12]}
    reserved = {}
    step_no = 0
    while waiting or live:
        while waiting and len(live) < 3 and _free_pages(manager) - sum(reserved.values()) >= need(waiting[0]):
            r = waiting.pop(0)
            live.append(r); pos[r] = 0
            reserved[r] = need(r)              # pages are taken as the request goes: the rest stays spoken for
        parts, ended = {}, []
        for r in live:
            plan = patterns[r]
            if pos[r] < sum(plan):
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
            reserved[r] = need(r) - -(-pos[r] // page)
            if pos[r] == lens[r]:
                ended.append(r)
        step_no += 1
        if parts:
            d.step(parts, end=ended)
            for r in ended:
                live.remove(r); reserved.pop(r)
    for r in lens:
        _check(env, folder, ids[r], d.result(r), f"{name} request {r} in the batch")


def long_decode(env, name):
    """A short prompt, then many single tokens: over page borders and over many steps of the temperature."""
    page = PAGE[name]
    n = 140
    ids = random_ids(n, _vocab(name), 500)
    runner, manager, folder = env.runner(name, -(-n // page))
    d = Driver(runner, manager)
    d.step({"r": ids[:6]})
    for t in range(6, n):
        d.step({"r": ids[t:t + 1]})
    _check(env, folder, ids, d.result("r"), f"{name} long decode")


def far_keys(env, name="far"):
    """330 positions: queries whose best key lies hundreds of positions back, in a prompt, in a portion behind a long
    prefix and decoded alone; the temperature changes at positions 63, 127, 191, 255 and 319, in a prompt and under
    single tokens (319 is decoded alone)."""
    page = PAGE[name]
    n = 330
    ids = random_ids(n, _vocab(name), 600)
    runner, manager, folder = env.runner(name, 2 * -(-n // page))
    d = Driver(runner, manager)
    d.step({"w": ids})
    d.step({"r": ids[:250]})
    d.step({"r": ids[250:258]})
    d.step({"r": ids[258:316]})
    for t in range(316, 323):
        d.step({"r": ids[t:t + 1]})
    d.step({"r": ids[323:]})
    _check(env, folder, ids, d.result("w"), f"{name} whole")
    _check(env, folder, ids, d.result("r"), f"{name} cut and decoded around a step of the temperature")


def real_sizes(env_f32, env_bf16, name="real"):
    """At the layer sizes of a real model: float32 against the plain evaluation on a short prompt; then a prompt of 700
    tokens (experts with several tiles of rows, many pages) whole, in portions and with its last tokens decoded,
    bfloat16 against float32 of the same engine."""
    page = PAGE[name]
    V = _vocab(name)
    short = random_ids(40, V, 900)
    runner, manager, folder = env_f32.runner(name, 8)
    d = Driver(runner, manager)
    d.step({"s": short[:33]})
    d.step({"s": short[33:34]})
    d.step({"s": short[34:]}, end=["s"])
    _check(env_f32, folder, short, d.result("s"), f"{name} short prompt in float32")
    n = 700
    ids = random_ids(n, V, 901)
    got = {}
    for env in (env_f32, env_bf16):
        runner, manager, folder = env.runner(name, 2 * -(-n // page))
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
    # bfloat16 rounds the router's input: a token whose expert scores nearly tie may go another way there, so the bulk is compared
    for g, what in ((wb, "whole"), (rb, "cut")):
        err = (g.double() - wf.double().cpu()).abs().amax(-1) / wf.double().abs().max()
        assert float(err.median()) <= env_bf16.tol / 4 and float((err > env_bf16.tol).float().mean()) <= 0.03, \
            f"bfloat16 {what}: median {float(err.median()):.3g}, {int((err > env_bf16.tol).sum())} positions beyond {env_bf16.tol}"


def pages_used_again(env, name):
    """A request that takes over the pages of one that has ended sees nothing of it."""
    page = PAGE[name]
    V = _vocab(name)
    runner, manager, folder = env.runner(name, 4)
    d = Driver(runner, manager)
    for i, n in enumerate((4 * page, 3, 2 * page + 1, 1)):
        ids = random_ids(n, V, 700 + i)
        d.step({f"r{i}": ids[:n // 2 + 1]})
        if n // 2 + 1 < n:
            d.step({f"r{i}": ids[n // 2 + 1:]}, end=[f"r{i}"])
        else:
            manager.free(f"r{i}")
        _check(env, folder, ids, d.result(f"r{i}"), f"{name} request {i} on used pages")


ALL = [whole, token_by_token, portions, batch_against_alone, long_decode, pages_used_again]


def greedy_through_the_engine(device, dtype_name, name, folder, exact: bool):
    """Greedy generation through `LLM.generate`: the scheduler admits under a token budget, cuts prompts, batches
    portions beside decoding requests, takes and gives back pages; decode steps go through the fixed layouts (captured
    as graphs on a GPU) and run one ahead."""
    from mini_engine_amd import LLM, SamplingParams
    V = _vocab(name)
    prompts = [random_ids(n, V, 800 + n) for n in (30, 12, 9, 1, 21)]
    llm = LLM(folder, dtype=dtype_name, device=device, kvcache_block_size=PAGE[name], num_kvcache_blocks=24, max_num_seqs=3,
              max_num_batched_tokens=16, max_model_len=64, poison_cache=True)
    outs = llm.generate(prompts, SamplingParams(temperature=0, max_tokens=12, ignore_eos=True), use_tqdm=False)
    assert llm.runner.graphs is not None and llm.runner.graphs.replays > 0, "no decode step went through the fixed-layout path"
    llm.manager.check_invariants()
    assert _free_pages(llm.manager) == 24
    for p, o in zip(prompts, outs):
        seq = list(p)
        assert len(o["token_ids"]) == 12
        for tok in o["token_ids"]:
            z = plain_logits(folder, seq)[-1]
            best = int(z.argmax())
            close = not exact and float(z[best] - z[tok]) < 8e-2 * float(z.abs().max())
            assert tok == best or close, f"{name} {dtype_name}: generated {tok}, the plain evaluation gives {best}"
            seq.append(tok)
