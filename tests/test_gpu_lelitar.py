"""GPU tests of the Lelitar family: every HIP kernel against the fp32
reference of the same op, then the engine (paged latent pool, varlen and
decode paths, captured decode graph) against the plain oracle."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.gpu

import lelitar_oracle as O  # noqa: E402

from agentainer_amd import ops  # noqa: E402
from agentainer_amd.ops import reference as ref  # noqa: E402


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    assert torch.cuda.is_available(), "needs a GPU"
    assert ops.latent_available(), "latent extension must be built in-tree"
    torch.backends.cuda.matmul.allow_tf32 = False


def _tol(dtype):
    return dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(
        rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W,groups", [(256, 2), (96, 3), (130, 1), (1024, 4)])
def test_residual_grouped_rmsnorm(dtype, W, groups):
    g = torch.Generator().manual_seed(W)
    T = 37
    x = torch.randn(T, W, generator=g) * 3
    a = torch.randn(T, W, generator=g).to(dtype)
    b = torch.randn(T, W, generator=g).to(dtype)
    w1 = torch.rand(W, generator=g) + 0.5
    w2 = torch.rand(W, generator=g) + 0.5
    for use_a, use_b, two in [(False, False, True), (True, True, True),
                              (True, False, False)]:
        xr = x.clone()
        outs_r = [torch.empty(T, W, dtype=dtype) for _ in range(2 if two else 1)]
        ws = [w1, w2][:len(outs_r)]
        ref.residual_grouped_rmsnorm(xr, a if use_a else None,
                                     b if use_b else None, 0.37, ws, outs_r,
                                     groups, 1e-5)
        xd = x.cuda()
        outs_d = [torch.empty(T, W, dtype=dtype, device="cuda") for _ in outs_r]
        ops.residual_grouped_rmsnorm(
            xd, a.cuda() if use_a else None, b.cuda() if use_b else None, 0.37,
            [w.cuda() for w in ws], outs_d, groups, 1e-5)
        torch.testing.assert_close(xd.cpu(), xr, rtol=1e-6, atol=1e-6)
        for od, orr in zip(outs_d, outs_r):
            torch.testing.assert_close(od.cpu().float(), orr.float(),
                                       **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_latent_norm_append(dtype):
    g = torch.Generator().manual_seed(1)
    T, qr, kvr, Rp, extra, PS, P = 19, 48, 40, 64, 24, 4, 9
    proj = torch.randn(T, qr + kvr + extra, generator=g).to(dtype)
    wq = torch.rand(qr, generator=g) + 0.5
    wkv = torch.rand(kvr, generator=g) + 0.5
    slots = torch.randperm(P * PS, generator=g)[:T]
    slots[3] = -1
    cache_r = torch.full((P, PS, Rp), 7.0, dtype=dtype)
    cq_r = torch.empty(T, qr, dtype=dtype)
    ref.latent_norm_append(proj, 0, qr, qr, kvr, wq, wkv, 1e-5, cq_r, cache_r,
                           slots)
    cache_d = torch.full((P, PS, Rp), 7.0, dtype=dtype, device="cuda")
    cq_d = torch.empty(T, qr, dtype=dtype, device="cuda")
    ops.latent_norm_append(proj.cuda(), 0, qr, qr, kvr, wq.cuda(), wkv.cuda(),
                           1e-5, cq_d, cache_d, slots.cuda())
    torch.testing.assert_close(cq_d.cpu().float(), cq_r.float(), **_tol(dtype))
    torch.testing.assert_close(cache_d.cpu().float(), cache_r.float(),
                               **_tol(dtype))


def _attn_case(dtype, H, Rp, PS, window, lens, ctxs, seed, simple):
    """Varlen batch: sequence b has ctxs[b] cached tokens + lens[b] new."""
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    n_pages = sum(-(-(c + l) // PS) for c, l in zip(ctxs, lens)) + 1
    cache = (torch.randn(n_pages, PS, Rp, generator=g) * 0.7).to(dtype)
    perm = (torch.randperm(n_pages - 1, generator=g) + 1).tolist()
    width = max(-(-(c + l) // PS) for c, l in zip(ctxs, lens))
    pt = torch.zeros(B, width, dtype=torch.int32)
    for b in range(B):
        n = -(-(ctxs[b] + lens[b]) // PS)
        pt[b, :n] = torch.tensor([perm.pop() for _ in range(n)])
    T = sum(lens)
    q = (torch.randn(H, T, Rp, generator=g) * 0.5).to(dtype)
    starts = torch.tensor([sum(lens[:b]) for b in range(B)], dtype=torch.int32)
    qlens = torch.tensor(lens, dtype=torch.int32)
    seq = torch.tensor([c + l for c, l in zip(ctxs, lens)], dtype=torch.int32)
    out_r = torch.zeros(H, T, Rp, dtype=dtype)
    ref.latent_window_attention(out_r, q, cache, pt, seq, starts, qlens, 0.11,
                                window)
    out_d = torch.zeros(H, T, Rp, dtype=dtype, device="cuda")
    old = ops.LATENT_SIMPLE
    ops.LATENT_SIMPLE = simple
    try:
        ops.latent_window_attention(out_d, q.cuda(), cache.cuda(), pt.cuda(),
                                    seq.cuda(), starts.cuda(), qlens.cuda(),
                                    0.11, window, max_qlen=max(lens))
    finally:
        ops.LATENT_SIMPLE = old
    torch.testing.assert_close(out_d.cpu().float(), out_r.float(),
                               **_tol(dtype))


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("H,Rp,PS,window", [
    (6, 128, 16, 100), (3, 64, 16, 5), (1, 32, 4, 1), (5, 96, 8, 33),
    (20, 160, 16, 70), (2, 512, 16, 40), (70, 64, 16, 17)])
def test_latent_attention_varlen_bf16(simple, H, Rp, PS, window):
    _attn_case(torch.bfloat16, H, Rp, PS, window, lens=[70, 1, 2, 33, 1],
               ctxs=[0, 150, 31, 64, 0], seed=H * 1000 + Rp, simple=simple)


@pytest.mark.parametrize("H,Rp,PS,window", [
    (6, 128, 16, 100), (3, 40, 4, 5), (2, 12, 16, 1), (5, 96, 8, 33)])
def test_latent_attention_varlen_fp32(H, Rp, PS, window):
    _attn_case(torch.float32, H, Rp, PS, window, lens=[70, 1, 2, 33, 1],
               ctxs=[0, 150, 31, 64, 0], seed=H * 1000 + Rp, simple=False)


@pytest.mark.parametrize("dtype,Rp", [
    (torch.bfloat16, 64), (torch.bfloat16, 128), (torch.bfloat16, 256),
    (torch.bfloat16, 512), (torch.float32, 64), (torch.float32, 128)])
@pytest.mark.parametrize("H,window,lens", [
    (4, 20, [37, 0, 1, 64]),
    (4, 200, [300, 0, 1, 130, 64, 257]),       # key span cut into slices
    (70, 1000, [640, 33, 0, 129]),             # heads span several row tiles
    (17, 77, [78, 0, 77, 500])])               # window edge inside a slice
def test_latent_attention_decode_rows(dtype, Rp, H, window, lens):
    """Decode form: no query_starts/lens; a row with seq_len <= 0 is a pad
    row and must come back as zeros."""
    g = torch.Generator().manual_seed(5)
    PS = 16
    seq = torch.tensor(lens, dtype=torch.int32)
    B = len(lens)
    width = max(-(-n // PS) for n in lens)
    n_pages = sum(-(-n // PS) for n in lens) + 1
    cache = (torch.randn(n_pages, PS, Rp, generator=g) * 0.7).to(dtype)
    perm = (torch.randperm(n_pages - 1, generator=g) + 1).tolist()
    pt = torch.zeros(B, width, dtype=torch.int32)
    for b, n in enumerate(lens):
        k = -(-n // PS)
        pt[b, :k] = torch.tensor([perm.pop() for _ in range(k)],
                                 dtype=torch.int32)
    q = (torch.randn(H, B, Rp, generator=g) * 0.5).to(dtype)
    out_r = torch.ones(H, B, Rp, dtype=dtype)
    ref.latent_window_attention(out_r, q, cache, pt, seq, None, None, 0.2,
                                window)
    out_d = torch.ones(H, B, Rp, dtype=dtype, device="cuda")
    ops.latent_window_attention(out_d, q.cuda(), cache.cuda(), pt.cuda(),
                                seq.cuda(), None, None, 0.2, window)
    assert float(out_d[:, lens.index(0)].abs().max()) == 0.0
    torch.testing.assert_close(out_d.cpu().float(), out_r.float(),
                               **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_elementwise_and_router(dtype):
    g = torch.Generator().manual_seed(2)
    T, H, E = 13, 3, 20
    a = torch.randn(H, T, E, generator=g).to(dtype)
    gate = torch.randn(T, H * E + 8, generator=g).to(dtype)
    o_r = torch.empty(T, H * E, dtype=dtype)
    ref.sigmoid_gate_mul(o_r, a, gate[:, 8:])
    o_d = torch.empty(T, H * E, dtype=dtype, device="cuda")
    ops.sigmoid_gate_mul(o_d, a.cuda(), gate.cuda()[:, 8:])
    torch.testing.assert_close(o_d.cpu().float(), o_r.float(), **_tol(dtype))

    for Fh in (24, 7):
        gu = torch.randn(T, 2 * Fh, generator=g).to(dtype)
        for act in ("relu", "silu"):
            o_r = torch.empty(T, Fh, dtype=dtype)
            ref.act_mul(o_r, gu[:, :Fh], gu[:, Fh:], act)
            o_d = torch.empty(T, Fh, dtype=dtype, device="cuda")
            gd = gu.cuda()
            ops.act_mul(o_d, gd[:, :Fh], gd[:, Fh:], act)
            torch.testing.assert_close(o_d.cpu().float(), o_r.float(),
                                       **_tol(dtype))

    for Ex, top in ((12, 1), (5, 2), (70, 3), (4, 4)):
        z = torch.randn(T, Ex, generator=g) * 2
        w_r = torch.empty(T, Ex)
        ref.sigmoid_topk_route(w_r, z, top)
        w_d = torch.empty(T, Ex, device="cuda")
        ops.sigmoid_topk_route(w_d, z.cuda(), top)
        torch.testing.assert_close(w_d.cpu(), w_r, rtol=1e-6, atol=1e-7)
        assert int((w_d > 0).sum()) == T * top
        Fh = 12
        gu = torch.randn(T, Ex * 2 * Fh, generator=g).to(dtype)
        o_r = torch.empty(T, Ex * Fh, dtype=dtype)
        ref.routed_scaled_silu_mul(o_r, gu, w_r)
        o_d = torch.empty(T, Ex * Fh, dtype=dtype, device="cuda")
        ops.routed_scaled_silu_mul(o_d, gu.cuda(), w_d)
        torch.testing.assert_close(o_d.cpu().float(), o_r.float(),
                                   **_tol(dtype))
