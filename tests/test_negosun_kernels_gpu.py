"""The kernels behind parallel blocks, attention with biases and whole-projection norms, and routed experts, each
against its plain twin at sizes of its own."""
import pytest
import torch

import kernel_twins as twin
from mini_engine_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def hip():
    return ops.HipBackend()


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    assert a.shape == b.shape and torch.isfinite(a).all()
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
    assert err <= tol, f"relative error {err:.3g} > {tol:g}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,n", [(1, 48), (37, 1000), (5, 3), (64, 4096), (300, 352)])
def test_scaled_sum_and_two_norms(dtype, T, n):
    torch.manual_seed(T + n)
    w1, w2 = 1 + torch.randn(n, device=DEV) * 0.1, 1 + torch.randn(n, device=DEV) * 0.1
    s1, s2 = torch.rand(n, device=DEV), torch.rand(n, device=DEV) + 0.5
    stream = torch.randn(T, n, device=DEV) * 3
    rows = (torch.randn(T, n, device=DEV) * 2).to(dtype)
    partials = torch.randn(3, T, n, device=DEV)
    more = torch.randn(1, T, n, device=DEV)
    tol = 1e-6 if dtype == torch.float32 else 4e-3
    for terms, a, b, base in (([(rows, s1), (partials, s2), (more, s2)], w1, w2, stream),
                              ([(partials, None)], w1, None, stream),
                              ([], w1, w2, stream),
                              ([], w1, w2, rows),                       # rows in the compute dtype start a stream
                              ([(rows, s1)], None, None, stream)):
        new, y1, y2 = hip().scaled_sum_norm(base, terms, 0.45, a, b, 1e-5, dtype)
        new_t, y1_t, y2_t = twin.scaled_sum_norm(base, terms, 0.45, a, b, 1e-5, dtype)
        assert new.dtype == torch.float32
        close(new, new_t, 1e-6)
        for y, y_t in ((y1, y1_t), (y2, y2_t)):
            assert (y is None) == (y_t is None)
            if y is not None:
                assert y.dtype == dtype
                close(y, y_t, tol)
    assert hip().scaled_sum_norm(stream, [], 1.0, w1, None, 1e-5, dtype)[0] is stream        # nothing to add: the stream stays


def test_softcap():
    z = torch.randn(7, 301, device=DEV) * 40
    want = 11.0 * torch.tanh(z / 11.0)
    view = z[:, :300]                                # rows with a stride
    hip().softcap_(view, 11.0)
    close(view, want[:, :300], 1e-6)
    assert torch.equal(z[:, 300], (want * 0 + z)[:, 300])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,D,n,nv,page", [(5, 1, 48, 40, 24, 16), (6, 3, 16, 10, 16, 8), (8, 2, 128, 128, 128, 16), (3, 3, 32, 24, 20, 4)])
def test_qkv_prologue(dtype, Hq, Hkv, D, n, nv, page):
    """Bias, norm over the stored dimensions of all heads at once, temperature by position, value mixing, page writes.
    Heads are laid out in D slots with zeros beyond their stored sizes n (keys) and nv (values)."""
    torch.manual_seed(Hq * D + page)
    T, pages = 45, 16
    width = (Hq + 2 * Hkv) * D
    mask = torch.zeros(Hq + 2 * Hkv, D, device=DEV)
    mask[:Hq + Hkv, :n] = 1
    mask[Hq + Hkv:, :nv] = 1
    mask = mask.view(-1)
    rows = torch.randn(T, width + 8, device=DEV)
    rows[:, :width] *= mask
    bias = torch.randn(width, device=DEV) * mask
    qw, kw = torch.rand(Hq * D, device=DEV) + 0.5, torch.rand(Hkv * D, device=DEV) + 0.5
    positions = torch.randint(0, 1000, (T,), device=DEV, dtype=torch.int32)
    scattered = torch.randperm(pages * page, device=DEV)[:T].to(torch.int32)
    scattered[3] = -1
    # a prompt's portions: 24 consecutive places from the start of a page (three groups of 8 tokens, which the kernel writes
    # with vector stores, over a page's border), then runs that start inside a page or at a token that starts no group
    runs = torch.cat([torch.arange(a, a + n) for a, n in ((5 * page, 24), (3, 9), (12 * page, 10))])
    portions = torch.cat((runs, torch.full((T - runs.numel(),), -1))).to(torch.int32).to(DEV)
    lam = torch.tensor(0.3, device=DEV)
    cases = ((0, None, True), (1, (0.5, 7), True), (2, (0.25, 96), True), (2, None, False))
    for slots, (mix, temperature, normed) in ((s, c) for s in (scattered, portions) for c in cases):
        got, want = [], []
        for be, keep in ((hip(), got), (twin, want)):
            kc = torch.zeros(pages, Hkv, page, D, device=DEV, dtype=dtype)
            vc = torch.zeros(pages, Hkv, D, page, device=DEV, dtype=dtype)
            vf = torch.randn(T, Hkv * nv, device=DEV, generator=torch.Generator(DEV).manual_seed(5)) if mix else None
            q = be.qkv_prepare_store(rows, bias, qw if normed else None, kw if normed else None, 1e-6, Hq * n, Hkv * n, temperature,
                                     positions, slots, kc, vc, Hq, Hkv, D, page, nv, mix, lam if mix == 2 else None, vf)
            keep += [q, kc, vc] + ([vf] if mix else [])
        tol = 2e-6 if dtype == torch.float32 else 4e-3
        assert got[0].dtype == dtype
        for a, b in zip(got, want):
            close(a, b, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,count,keep,n", [(12, 3, 3, 2, 96), (8, 8, 1, 1, 64), (60, 6, 5, 2, 200), (256, 8, 8, 4, 2048), (3, 1, 3, 1, 30),
                                                 (128, 4, 1, 1, 7168)])
def test_router(dtype, E, top, count, keep, n):
    torch.manual_seed(E + n)
    for T in (1, 5, 67):
        x = torch.randn(T, n, device=DEV).to(dtype)
        router = torch.randn(E, n, device=DEV) * (3.0 / n ** 0.5)
        ids, w = hip().moe_route(x, router, top, count, keep)
        ids_t, w_t = twin.moe_route(x.cpu().double(), router.cpu().double(), top, count, keep)
        assert torch.equal(ids.cpu(), ids_t), "another choice of experts"
        close(w, w_t, 2e-5)
        per = E // count
        assert (torch.div(ids, per, rounding_mode="floor").cpu().sort(-1).values.diff(dim=-1) >= 0).all()
        assert all(len(set(row)) == top for row in ids.tolist())
        if count > 1:
            assert all(len({e // per for e in row}) <= keep for row in ids.tolist())


@pytest.mark.parametrize("dtype,simple", [(torch.float32, True), (torch.bfloat16, True), (torch.bfloat16, 16), (torch.bfloat16, 64), (torch.bfloat16, 128)])
@pytest.mark.parametrize("E,top,F,K,T", [(12, 2, 48, 160, 45), (4, 1, 40, 72, 300), (8, 3, 200, 136, 1), (32, 4, 256, 512, 700), (5, 5, 24, 64, 3),
                                          (64, 6, 1408, 2048, 130)])
def test_routed_experts(dtype, simple, E, top, F, K, T):
    """The kernels on tiles of 128, 64 and 16 rows, and the one-wave-per-element kernels against the plain loop: experts without tokens, experts with
    more than one tile, one token, sizes that are no multiples of the tiles."""
    torch.manual_seed(E * top + T)
    x = torch.randn(T, K, device=DEV).to(dtype)
    gate_up = (torch.randn(E, 2 * F, K, device=DEV) * K ** -0.5).to(dtype)
    down = (torch.randn(E, K, F, device=DEV) * F ** -0.5).to(dtype)
    ids = torch.stack([torch.randperm(E, device=DEV)[:top] for _ in range(T)]).to(torch.int32)
    if E > 2 and T > 1:
        ids[ids == 1] = 0 if top == 1 else ids[ids == 1]          # top 1: expert 1 gets nobody
    w = torch.rand(T, top, device=DEV)
    got = hip().routed_experts(x, ids, w, gate_up, down, force_simple=simple is True, tile_rows=None if simple is True else simple)
    want = twin.routed_experts(x, ids, w, gate_up, down)
    assert got.shape == (top, T, K) and got.dtype == torch.float32
    close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2)
    if dtype == torch.bfloat16:
        close(got.sum(0), want.sum(0), 1e-2)


@pytest.mark.parametrize("E,top,count,keep,F,K", [(12, 3, 3, 2, 48, 160), (32, 4, 4, 2, 384, 1024), (256, 8, 8, 4, 64, 512), (512, 2, 1, 1, 16, 64)])
def test_route_and_run_experts(E, top, count, keep, F, K):
    """Few tokens: the kernel that orders the pairs makes the choice itself (up to the expert count that fits it); the
    result is that of the two operations one after the other."""
    torch.manual_seed(E + K)
    router = torch.randn(E, K, device=DEV) * (3.0 / K ** 0.5)
    gate_up = (torch.randn(E, 2 * F, K, device=DEV) * K ** -0.5).bfloat16()
    down = (torch.randn(E, K, F, device=DEV) * F ** -0.5).bfloat16()
    for T in (1, 7, 64, 65):
        x = torch.randn(T, K, device=DEV).bfloat16()
        got = hip().route_and_run_experts(x, router, top, count, keep, gate_up, down)
        ids, w = hip().moe_route(x, router, top, count, keep)
        want = hip().routed_experts(x, ids, w, gate_up, down)
        assert torch.equal(got, want), f"T={T}: the fused choice differs from the separate one"
    assert ops.moe_sort_chooses(64, 256, 8) and not ops.moe_sort_chooses(65, 32, 1) and not ops.moe_sort_chooses(8, 512, 1)
