"""Sigosun on the GPU: each new kernel against its plain twin at sizes of its own, then the engine's cuts, batches,
slot reuse, long decoding and block edges in float32 and bfloat16 against the plain evaluation, decode steps replayed as
graphs, greedy generation through the scheduler, and the trace program on a folder of this design."""
import pytest
import torch

import helpers
import kernel_twins as twin
import sigosun_cases as S
import test_trace_run as TR
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.kernels import ops
from mini_engine_amd.weights.loader import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 3e-5, torch.bfloat16: 8e-2}      # widths of 24-48 make bfloat16 noisy: the plain twins in bfloat16 differ by up to 5e-2 too


def hip():
    return ops.HipBackend()


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    assert torch.isfinite(a).all()
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
    assert err <= tol, f"relative error {err:.3g} > {tol:g}"


@pytest.fixture(scope="module")
def sigosun_folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = S.make_folder(name, str(tmp_path_factory.mktemp(f"sigosun_{name}")))
        return made[name]

    return get


# ------------------------------------------------------------------ kernels against their twins

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,n,parts", [(1, 48, 1), (37, 1000, 1), (300, 256, 4), (5, 3, 1), (64, 4096, 2)])
def test_add_rms_norm(dtype, T, n, parts):
    torch.manual_seed(T + n)
    stream = torch.randn(T, n, device=DEV) * 4
    w = 1 + torch.randn(n, device=DEV) * 0.1
    y = torch.randn(parts, T, n, device=DEV) if parts > 1 else (torch.randn(T, n, device=DEV) * 2).to(dtype)
    lo, new = hip().add_rms_norm(y, w, 1e-5, stream, dtype)
    lo_t, new_t = twin.add_rms_norm(y, w, 1e-5, stream, dtype)
    close(new, new_t, 1e-6)
    assert lo.dtype == dtype
    close(lo, lo_t, 1e-6 if dtype == torch.float32 else 4e-3)
    assert torch.equal(lo.float(), new.to(dtype).float())              # the rounded stream is the stream, rounded once


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["silu", "relu2"])
def test_activation_of_a_row_view(dtype, kind):
    rows = (torch.randn(33, 200, device=DEV) * 3).to(dtype)
    view = rows[:, 17:150]
    close(hip().activation(view, kind), twin.activation(view, kind), 1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_gate(dtype):
    T, H, D = 19, 5, 48
    o = torch.randn(T, H * D, device=DEV).to(dtype)
    rows = (torch.randn(T, 64, device=DEV) * 3).to(dtype)
    want = o.clone()
    twin.head_gate(want, rows[:, 40:45], H, D)
    hip().head_gate(o, rows[:, 40:45], H, D)
    close(o, want, 1e-6 if dtype == torch.float32 else 4e-3)


def _steps_meta(q_lens, slots):
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    seq = torch.repeat_interleave(torch.arange(len(q_lens)), torch.tensor(q_lens)).to(torch.int32).to(DEV)
    return cu, seq, torch.tensor(slots, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,C", [(2, 40), (4, 300), (3, 7), (1, 16)])
def test_causal_conv_continues_from_its_state(dtype, taps, C):
    """Requests of 1, 2, taps - 1, taps and many tokens in one step, each from a state of its own; then the same
    tokens cut in two steps give the same as in one."""
    torch.manual_seed(taps * C)
    q_lens = [1, 2, max(1, taps - 1), taps, 77]
    cu, seq, slots = _steps_meta(q_lens, [3, 0, 5, 1, 2])
    T = sum(q_lens)
    rows = torch.randn(T, C + 9, device=DEV).to(dtype)
    x = rows[:, 4:4 + C]
    w, b = torch.randn(C, taps, device=DEV), torch.randn(C, device=DEV)
    full = torch.randn(7, 11 + C * (taps - 1), device=DEV)
    st_h, st_t = full.clone(), full.clone()
    got = hip().causal_conv(x, w, b, st_h[:, 11:], slots, cu, q_lens)
    want = twin.causal_conv(x.cpu(), w.cpu(), b.cpu(), (st_c := st_t.cpu())[:, 11:], slots.cpu(), cu.cpu(), q_lens)
    close(got, want, 1e-6 if dtype == torch.float32 else 8e-3)
    close(st_h, st_c, 1e-6)
    assert torch.equal(st_h[:, :11], full[:, :11]) and torch.equal(st_h[4], full[4]) and torch.equal(st_h[6], full[6])
    # the last request again (77 tokens: three blocks of a thread's 32), cut after 5 tokens
    st2 = full.clone()
    cu1, seq1, sl1 = _steps_meta([5], [2])
    first = hip().causal_conv(x[T - 77:T - 72], w, b, st2[:, 11:], sl1, cu1, [5])
    cu2, seq2, _ = _steps_meta([72], [2])
    rest = hip().causal_conv(x[T - 72:], w, b, st2[:, 11:], sl1, cu2, [72])
    assert torch.equal(torch.cat((first, rest)), got[T - 77:]) and torch.equal(st2[2], st_h[2])


@pytest.mark.parametrize("columns", [1, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,N,P,selective", [(4, 2, 20, 12, True), (3, 3, 10, 20, False), (2, 1, 70, 80, True),
                                               (2, 2, 130, 8, False), (5, 1, 48, 48, True), (8, 8, 64, 64, False)])
def test_linear_recurrence(monkeypatch, dtype, H, G, N, P, selective, columns):
    """Requests of unequal lengths from states of their own, against the token-by-token twin; 300 tokens are cut into
    spans that run side by side (the launch rule says so), which must give what one pass gives. Both forms of the
    kernel: one state column per lane, and two (blocks of one head, or two heads of a group)."""
    monkeypatch.setattr(ops, "RECURRENCE_COLUMNS", columns)
    assert ops.recurrence_columns([300], H, G, P, 1) == (1 if columns == 1 or (P <= 64 and (H // G) % 2) else 2)
    silu = not selective and H == 3
    torch.manual_seed(H * N + P)
    q_lens = [1, 300, 2, 17]
    cu, seq, slots = _steps_meta(q_lens, [2, 0, 4, 1])
    T = sum(q_lens)
    rows = torch.randn(T, 2 * G * N + H * P + H + 5, device=DEV).to(dtype)
    q, k = rows[:, 1:1 + G * N], rows[:, 1 + G * N:1 + 2 * G * N]
    v = rows[:, 1 + 2 * G * N:1 + 2 * G * N + H * P]
    kw = {}
    if selective:
        kw = dict(dt=rows[:, 1 + 2 * G * N + H * P:1 + 2 * G * N + H * P + H], dt_bias=torch.randn(H, device=DEV) - 2,
                  rate=torch.rand(H, device=DEV) * 4 + 0.2, skip=torch.randn(H, device=DEV))
    else:
        kw = dict(decay=torch.tensor([0.5, 0.9, 0.99, 0.999, 0.8, 0.95, 0.7, 0.9999][:H], device=DEV), silu=silu)
    full = torch.randn(6, 3 + H * N * P, device=DEV)
    st_h, st_c = full.clone(), full.cpu().clone()
    assert ops.recurrence_spans(q_lens, 1)[1] > 1
    y = hip().linear_recurrence(q, k, v, st_h[:, 3:], slots, cu, q_lens, H, G, N, P, **kw)
    y = y.sum(0) if y.dim() == 3 else y
    cpu = {n: (t.cpu() if torch.is_tensor(t) else t) for n, t in kw.items()}
    want = twin.linear_recurrence(q.cpu(), k.cpu(), v.cpu(), st_c[:, 3:], slots.cpu(), cu.cpu(), q_lens, H, G, N, P, **cpu)
    tol = 2e-5 if dtype == torch.float32 else 2e-5        # the inputs are exact in both; only the sums' order differs
    close(y, want, tol)
    close(st_h, st_c, tol)
    assert torch.equal(st_h[:, :3], full[:, :3]) and torch.equal(st_h[3], full[3]) and torch.equal(st_h[5], full[5])
    # token by token from the same start: decoding continues what a prompt left
    st1 = full.clone()
    one = [hip().linear_recurrence(q[t:t + 1], k[t:t + 1], v[t:t + 1], st1[:, 3:], slots[3:4], torch.tensor([0, 1], dtype=torch.int32, device=DEV),
                                   [1], H, G, N, P, **{n: (a[t:t + 1] if n == "dt" else a) for n, a in kw.items()}) for t in range(T - 17, T)]
    one = torch.cat([o.sum(0) if o.dim() == 3 else o for o in one])
    close(one, want[T - 17:], tol)
    close(st1[1], st_c[1], tol)
    # five requests with one token each (the kernel of pure decode steps), slots in an order of their own
    st5, st5c = full.clone(), full.cpu().clone()
    cu5, _, sl5 = _steps_meta([1] * 5, [4, 0, 2, 5, 1])
    kw5 = {n: (a[:5] if n == "dt" else a) for n, a in kw.items()}
    got5 = hip().linear_recurrence(q[:5], k[:5], v[:5], st5[:, 3:], sl5, cu5, [1] * 5, H, G, N, P, **kw5)
    assert got5.dim() == 2
    want5 = twin.linear_recurrence(q[:5].cpu(), k[:5].cpu(), v[:5].cpu(), st5c[:, 3:], sl5.cpu(), cu5.cpu(), [1] * 5, H, G, N, P,
                                   **{n: (t.cpu() if torch.is_tensor(t) else t) for n, t in kw5.items()})
    close(got5, want5, tol)
    close(st5, st5c, tol)
    assert torch.equal(st5[3], full[3]) and torch.equal(st5[:, :3], full[:, :3])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind,groups,parts", [("silu_before", 1, 1), ("silu_before", 4, 2), ("sigmoid_behind", 1, 3)])
def test_gated_rms_norm(dtype, kind, groups, parts):
    T, n = 23, 96
    y = torch.randn(parts, T, n, device=DEV) if parts > 1 else torch.randn(T, n, device=DEV)
    rows = (torch.randn(T, n + 40, device=DEV) * 2).to(dtype)
    w = torch.rand(n, device=DEV) + 0.5
    got = hip().gated_rms_norm(y, rows[:, 8:8 + n], w, 1e-5, groups, kind, dtype)
    close(got, twin.gated_rms_norm(y, rows[:, 8:8 + n], w, 1e-5, groups, kind, dtype), 1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk", [5, 32, 100, 257])
def test_attention_under_a_block_mask(dtype, chunk):
    """Prompts from their start, a portion behind a prefix and single tokens, at positions on both sides of block
    edges; one key per request is made to dominate, so a key wrongly seen or hidden shows."""
    torch.manual_seed(chunk)
    Hq, Hkv, D, page = 8, 2, 64, 16
    starts, q_lens = [chunk - 1, chunk, 2 * chunk + 3, 0, chunk - 3], [1, 1, 1, 2 * chunk + 9, 7]
    B, T = len(starts), sum(q_lens)
    ctx = [s + q for s, q in zip(starts, q_lens)]
    MB = -(-max(ctx) // page)
    pages = B * MB
    k_cache = torch.full((pages + 1, Hkv, page, D), float("nan"), device=DEV, dtype=dtype)
    v_cache = torch.full((pages + 1, Hkv, D, page), float("nan"), device=DEV, dtype=dtype)
    perm = torch.randperm(pages)
    bt = torch.full((B, MB), -1, dtype=torch.int32)
    for b in range(B):
        n = -(-ctx[b] // page)
        bt[b, :n] = perm[b * MB:b * MB + n].to(torch.int32)
        keys = torch.randn(n * page, Hkv, D)
        keys[(starts[b] // chunk) * chunk - 1 if starts[b] >= chunk else 0] *= 6          # just outside (or the first key)
        keys[(starts[b] // chunk) * chunk] *= 6                                             # just inside
        vals = torch.randn(n * page, Hkv, D)
        for i in range(n):
            k_cache[bt[b, i]] = keys[i * page:(i + 1) * page].transpose(0, 1).to(dtype)
            v_cache[bt[b, i]] = vals[i * page:(i + 1) * page].permute(1, 2, 0).to(dtype)
    bt = bt.to(DEV)
    q = torch.randn(T, Hq * D, device=DEV).to(dtype)
    cu, seq, _ = _steps_meta(q_lens, [0] * B)
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, q_lens)]).to(torch.int32).to(DEV)
    ctx_t = torch.tensor(ctx, dtype=torch.int32, device=DEV)
    prefill_cu = (cu[3:] - cu[3]).contiguous()
    args = (q, k_cache, v_cache, page, bt, ctx_t, seq, positions, prefill_cu, 3, max(ctx[:3]), 0.11, None, Hq, Hkv, D)
    got = hip().paged_attention(*args, max_prefill_context=max(ctx[3:]), chunk=chunk)
    want = twin.paged_attention(*args, chunk=chunk)
    close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)
    if dtype == torch.bfloat16:          # the other implementation of single tokens
        again = hip().paged_attention(*args, max_prefill_context=max(ctx[3:]), chunk=chunk, decode_as_prefill=True)
        close(again, want, 2e-2)


# ------------------------------------------------------------------ the engine

class Env:
    def __init__(self, folders, dtype, graphs=False):
        self.folders, self.dtype, self.tol, self.models, self.graphs = folders, dtype, TOL[dtype], {}, graphs
        self.device = DEV

    def runner(self, name, pages, slots):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 1024)
        model = self.models[name]
        manager = CacheManager(pages, S.PAGE[name], ModelRunner.windows_of(model), num_state_slots=slots, enable_prefix_caching=False)
        options = dict(use_graphs=True, mixed_graphs_after=1) if self.graphs else {}
        return ModelRunner(model, manager, self.dtype, self.device, 1024, poison_cache=True, **options), manager, folder


@pytest.fixture(scope="module", params=[torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def env(request, sigosun_folders):
    return Env(sigosun_folders, request.param)


@pytest.mark.parametrize("name", ["mix", "odd", "att", "ssm", "lin"])
@pytest.mark.parametrize("case", S.ALL, ids=lambda c: c.__name__)
def test_cuts(env, case, name):
    case(env, name)


def test_far_keys_and_block_edges(env):
    S.far_keys(env)


def test_real_layer_sizes(sigosun_folders):
    S.real_sizes(Env(sigosun_folders, torch.float32), Env(sigosun_folders, torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("case", [S.token_by_token, S.long_decode, S.batch_against_alone], ids=lambda c: c.__name__)
def test_cuts_through_captured_steps(sigosun_folders, case, dtype):
    """The same with decode steps (and small steps that come up again) replayed as graphs: state slots travel with the
    step's metadata, fresh slots are zeroed outside the graph."""
    env = Env(sigosun_folders, dtype, graphs=True)
    case(env, "mix")


def test_hip_libraries_are_the_ones_running(env):
    S.whole(env, "att")
    assert ops.backend().name == "hip" and any("libme_core" in p for p in ops.loaded_libraries())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mix", "lin"])
def test_greedy_generation_through_the_scheduler(sigosun_folders, dtype, name):
    S.greedy_through_the_engine(DEV, dtype, name, sigosun_folders(name), exact=dtype == "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_program_on_this_design(sigosun_folders, tmp_path, dtype):
    """bin/trace_run picks the model class by the folder's config: four live requests, portions beside single tokens,
    state slots and pages used again."""
    name = "mix"
    folder = sigosun_folders(name)
    V = S.CONFIGS[name]["vocab"]
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
    TR.replay(folder, dtype, steps, out, max_tokens=TR.most_live_tokens(steps), page=S.PAGE[name])
    for r, g in TR.collect(steps, out, V).items():
        err = helpers.rel_err(g, S.plain_logits(folder, ids[r]))
        assert err <= TOL[getattr(torch, dtype)], f"{dtype} request {r}: {err:.3g}"


def test_offline_workload_row_with_random_weights(tmp_path, capsys):
    """The offline workload through the command line, on this design at a tiny size with random weights."""
    import json
    from mini_engine_amd import cli
    rc = cli.main(["--random-weights", "sigosun:tinyA", "--num-seqs", "6", "--max-prompt", "40", "--max-output", "8",
                   "--max-model-len", "64", "--max-num-seqs", "4", "--budget", "32", "--tokens-out", "-",
                   "--out", str(tmp_path / "bench.jsonl")])
    assert rc == 0
    lines = capsys.readouterr().out.strip().splitlines()
    row = json.loads(lines[-1])
    tokens = [json.loads(line) for line in lines[-7:-1]]
    assert [len(t) for t in tokens] == [8] * 6 and all(0 <= t < 256 for ts in tokens for t in ts)
    assert row["num_seqs"] == 6 and row["output_tokens"] == 48 and row["throughput_tok_s"] > 0
