"""GPU tests of the Volalorn family's kernels: every HIP kernel against the
fp32 torch reference of the same op (scalar-gain norms, PolyNorm, rotary +
q/k norm + append, masked attention in both kernel forms)."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.gpu

from agentainer_amd import ops  # noqa: E402
from agentainer_amd.ops import reference as ref  # noqa: E402


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    assert torch.cuda.is_available(), "needs a GPU"
    assert ops.masked_available(), "masked extension must be built in-tree"
    torch.backends.cuda.matmul.allow_tf32 = False


def _tol(dtype):
    return dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(
        rtol=3e-5, atol=3e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [256, 130, 1000, 4096])
def test_scalar_postnorm_and_rmsnorm(dtype, W):
    g = torch.Generator().manual_seed(W)
    T = 23
    x = torch.randn(T, W, generator=g) * 3
    y = (torch.randn(T, W, generator=g) * 5).to(dtype)
    gain = torch.tensor([0.73])
    xr, hr = x.clone(), torch.empty(T, W, dtype=dtype)
    ref.scalar_postnorm_residual(xr, y, gain, 1e-5, hr)
    xd, hd = x.cuda(), torch.empty(T, W, dtype=dtype, device="cuda")
    ops.scalar_postnorm_residual(xd, y.cuda(), gain.cuda(), 1e-5, hd)
    torch.testing.assert_close(xd.cpu(), xr, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(hd.cpu().float(), hr.float(), **_tol(dtype))
    outr = torch.empty(T, W, dtype=dtype)
    ref.scalar_rmsnorm(outr, x, gain, 1e-5)
    outd = torch.empty(T, W, dtype=dtype, device="cuda")
    ops.scalar_rmsnorm(outd, x.cuda(), gain.cuda(), 1e-5)
    torch.testing.assert_close(outd.cpu().float(), outr.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("F_", [384, 250, 3000])
def test_poly_norm(dtype, F_):
    g = torch.Generator().manual_seed(F_)
    T = 19
    z = (torch.randn(T, F_, generator=g) * 1.7).to(dtype)
    coef = torch.tensor([0.9, -0.4, 0.3, 0.05])
    outr = torch.empty(T, F_, dtype=dtype)
    ref.poly_norm(outr, z, coef, 1e-5)
    outd = torch.empty(T, F_, dtype=dtype, device="cuda")
    ops.poly_norm(outd, z.cuda(), coef.cuda(), 1e-5)
    torch.testing.assert_close(outd.cpu().float(), outr.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("norm_first", [False, True])
@pytest.mark.parametrize("H,G,D,Dv,rot", [(4, 2, 64, 32, 32), (6, 3, 96, 40, 96),
                                          (3, 1, 20, 12, 8), (8, 8, 128, 128, 64),
                                          (5, 1, 128, 24, 128), (2, 1, 256, 64, 64),
                                          (2, 2, 64, 8, 2), (1, 1, 128, 16, 0)])
def test_rotary_norm_append(dtype, norm_first, H, G, D, Dv, rot):
    g = torch.Generator().manual_seed(D + H)
    T, PS, P = 29, 4, 12
    n = H * D + G * D + G * Dv
    # odd row stride for odd head sizes; 16-byte rows where the one-load
    # form of the kernel applies (64 / 128 / 256 coordinates per head)
    proj = torch.randn(T, n + (3 if D % 64 else 8), generator=g).to(dtype)
    pos = torch.randint(0, 3000, (T,), generator=g, dtype=torch.int32)
    slots = torch.randperm(P * PS, generator=g)[:T]
    slots[5] = -1
    scaling = ({"factor": 6.0, "original": 128, "fast": 16.0, "slow": 2.0}
               if not norm_first else None)
    freqs, amp = ops.rotary_frequencies(rot, 30000.0, scaling)
    qw = torch.rand(D, generator=g) + 0.5 if norm_first else None
    kw = torch.rand(D, generator=g) + 0.5 if norm_first else None

    def views(p):
        return (p[:, :H * D].view(T, H, D),
                p[:, H * D:H * D + G * D].view(T, G, D),
                p[:, H * D + G * D:n].view(T, G, Dv))

    pr = proj.clone()
    kc_r = torch.full((P, G, PS, D), 7.0, dtype=dtype)
    vc_r = torch.full((P, G, PS, Dv), 7.0, dtype=dtype)
    cs_r = ref.rotary_table(pos, freqs, amp)
    ref.rotary_norm_append(*views(pr), kc_r, vc_r, cs_r, slots, 1e-5, qw, kw,
                           norm_first)
    pd = proj.cuda()
    kc_d = torch.full((P, G, PS, D), 7.0, dtype=dtype, device="cuda")
    vc_d = torch.full((P, G, PS, Dv), 7.0, dtype=dtype, device="cuda")
    cs_d = ops.rotary_table(pos.cuda(), freqs.cuda(), amp)
    torch.testing.assert_close(cs_d.cpu(), cs_r, rtol=5e-4, atol=5e-4)
    ops.rotary_norm_append(*views(pd), kc_d, vc_d, cs_d, slots.cuda(), 1e-5,
                           qw.cuda() if norm_first else None,
                           kw.cuda() if norm_first else None, norm_first)
    # fp32 angles of a few thousand radians: cos/sin agree to ~1e-4
    tol = _tol(dtype) if dtype == torch.bfloat16 else dict(rtol=5e-4, atol=5e-4)
    torch.testing.assert_close(pd.cpu().float(), pr.float(), **tol)
    torch.testing.assert_close(kc_d.cpu().float(), kc_r.float(), **tol)
    torch.testing.assert_close(vc_d.cpu().float(), vc_r.float(), rtol=0, atol=0)


def _attn_case(seed, H, G, D, Dv, PS, lens, qlens, dtype):
    """Random pools + page tables for sequences of total length lens[b]
    whose last qlens[b] tokens are the queries."""
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    n_pages = sum(-(-n // PS) for n in lens) + 1
    perm = (torch.randperm(n_pages - 1, generator=g) + 1).tolist()
    max_pages = max(-(-n // PS) for n in lens)
    pt = torch.zeros(B, max_pages, dtype=torch.int32)
    for b, n in enumerate(lens):
        for i in range(-(-n // PS)):
            pt[b, i] = perm.pop()
    kc = torch.randn(n_pages, G, PS, D, generator=g).to(dtype)
    vc = torch.randn(n_pages, G, PS, Dv, generator=g).to(dtype)
    T = sum(qlens)
    q = (torch.randn(T, H, D, generator=g) * 1.5).to(dtype)
    gate = torch.randn(T, H, generator=g).to(dtype)
    bias = torch.randn(H, generator=g)
    starts = [sum(qlens[:b]) for b in range(B)]
    return (q, kc, vc, pt, torch.tensor(lens, dtype=torch.int32),
            torch.tensor(starts, dtype=torch.int32),
            torch.tensor(qlens, dtype=torch.int32), gate, bias)


MASKS = [
    # kind, size, keep_first, sigmoid, softcap, gate
    (ref.MASK_WINDOW, 40, 3, False, 0.0, False),
    (ref.MASK_WINDOW, 7, 0, False, 0.0, False),
    (ref.MASK_WINDOW, 33, 50, False, 0.0, True),   # kept prefix > one tile
    (ref.MASK_CHUNK, 48, 0, True, 8.0, True),
    (ref.MASK_CHUNK, 5, 0, True, 0.0, False),
    (ref.MASK_CHUNK, 1, 0, False, 3.0, False),
    (ref.MASK_CAUSAL, 0, 0, False, 0.0, False),
]


@pytest.mark.parametrize("simple", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,G,D,Dv,PS", [
    (4, 2, 64, 32, 16), (6, 2, 64, 48, 16), (8, 1, 32, 16, 16),
    (2, 2, 256, 256, 16), (3, 1, 20, 12, 16), (5, 5, 96, 80, 16),
    # more heads per kv head than one wave's 16 columns; page sizes that
    # are not powers of two (with and without whole four-key units)
    (40, 2, 32, 32, 16), (4, 1, 64, 64, 12), (2, 1, 32, 16, 6)])
@pytest.mark.parametrize("mask", MASKS)
def test_masked_attention_prompt_and_decode(simple, dtype, H, G, D, Dv, PS,
                                            mask):
    if simple and dtype == torch.float32:
        pytest.skip("fp32 always takes the row kernel")
    kind, size, keep, sig, cap, use_gate = mask
    lens = [1, 200, 77, 131, 64]
    qlens = [1, 150, 2, 131, 1]
    (q, kc, vc, pt, sl, qs, ql, gate, bias) = _attn_case(
        H * 100 + D, H, G, D, Dv, PS, lens, qlens, dtype)
    scale = D ** -0.5 * 2.0
    T = q.size(0)
    kw = dict(scale=scale, mask_kind=kind, mask_size=size, keep_first=keep,
              sigmoid_weights=sig, softcap=cap)
    out_r = torch.zeros(T, H, Dv, dtype=dtype)
    ref.masked_attention(out_r, q, kc, vc, pt, sl, qs, ql,
                         key_bias=bias if sig else None,
                         head_gate=gate if use_gate else None, **kw)
    prev = ops.MASKED_SIMPLE
    ops.MASKED_SIMPLE = simple
    try:
        out_d = torch.zeros(T, H, Dv, dtype=dtype, device="cuda")
        ops.masked_attention(out_d, q.cuda(), kc.cuda(), vc.cuda(), pt.cuda(),
                             sl.cuda(), qs.cuda(), ql.cuda(),
                             key_bias=bias.cuda() if sig else None,
                             head_gate=gate.cuda() if use_gate else None,
                             max_qlen=max(qlens), **kw)
        # decode form: the LAST query of every sequence, one row each, and
        # a pad row (seq_len -1) that must come back zero
        last = [int(qs[b]) + qlens[b] - 1 for b in range(len(lens))]
        qd = torch.cat([q[last], torch.ones(1, H, D, dtype=dtype)]).cuda()
        gd = torch.cat([gate[last], torch.zeros(1, H, dtype=dtype)]).cuda()
        sld = torch.cat([sl, torch.tensor([-1], dtype=torch.int32)]).cuda()
        ptd = torch.cat([pt, torch.zeros(1, pt.size(1), dtype=torch.int32)])
        out_dec = torch.full((len(lens) + 1, H, Dv), 9.0, dtype=dtype,
                             device="cuda")
        ops.masked_attention(out_dec, qd, kc.cuda(), vc.cuda(), ptd.cuda(),
                             sld, None, None,
                             key_bias=bias.cuda() if sig else None,
                             head_gate=gd if use_gate else None, **kw)
    finally:
        ops.MASKED_SIMPLE = prev
    tol = (dict(rtol=3e-2, atol=3e-2 * (4.0 if sig else 1.0))
           if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4))
    torch.testing.assert_close(out_d.cpu().float(), out_r.float(), **tol)
    torch.testing.assert_close(out_dec[:-1].cpu().float(),
                               out_r[last].float(), **tol)
    assert float(out_dec[-1].abs().max()) == 0.0


@pytest.mark.parametrize("splits", [0, 1, 3])
@pytest.mark.parametrize("mask", [
    (ref.MASK_WINDOW, 600, 40, False, 0.0, False),
    (ref.MASK_CHUNK, 512, 0, True, 6.0, True),
    (ref.MASK_CAUSAL, 0, 0, False, 0.0, True),
])
@pytest.mark.parametrize("H,G,D,Dv", [(8, 2, 64, 32), (4, 4, 128, 128),
                                      (16, 1, 32, 48)])
def test_masked_attention_long_decode_split(splits, mask, H, G, D, Dv):
    """Decode over hundreds of keys: the key range is cut into slices whose
    partial results are merged (softmax statistics, or plain sums for the
    sigmoid weights)."""
    kind, size, keep, sig, cap, use_gate = mask
    lens = [700, 513, 33, 1]
    qlens = [1, 1, 1, 1]
    (q, kc, vc, pt, sl, qs, ql, gate, bias) = _attn_case(
        H + D, H, G, D, Dv, 16, lens, qlens, torch.bfloat16)
    kw = dict(scale=D ** -0.5 * 2.0, mask_kind=kind, mask_size=size,
              keep_first=keep, sigmoid_weights=sig, softcap=cap)
    out_r = torch.zeros(4, H, Dv, dtype=torch.bfloat16)
    ref.masked_attention(out_r, q, kc, vc, pt, sl, None, None,
                         key_bias=bias if sig else None,
                         head_gate=gate if use_gate else None, **kw)
    prev = ops.MASKED_SPLITS
    ops.MASKED_SPLITS = splits
    try:
        out_d = torch.zeros(4, H, Dv, dtype=torch.bfloat16, device="cuda")
        ops.masked_attention(out_d, q.cuda(), kc.cuda(), vc.cuda(), pt.cuda(),
                             sl.cuda(), None, None,
                             key_bias=bias.cuda() if sig else None,
                             head_gate=gate.cuda() if use_gate else None, **kw)
    finally:
        ops.MASKED_SPLITS = prev
    tol = dict(rtol=3e-2, atol=3e-2 * (10.0 if sig else 1.0))
    torch.testing.assert_close(out_d.cpu().float(), out_r.float(), **tol)
