"""Each Lelitar mechanism alone: the framework's op / module against the
oracle function of the same mechanism (CPU reference ops, and marked gpu
the HIP kernels). The attention cases plant a 'beacon' key whose score
dwarfs all others, so a window edge that is one token off, a wrong page
or a dropped first token flips the output instead of hiding in a mean
over hundreds of keys."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import lelitar_oracle as O  # noqa: E402

from agentainer_amd import ops  # noqa: E402
from agentainer_amd.models import lelitar as L  # noqa: E402
from agentainer_amd.models.llama import AttnMetadata  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return 3e-2 if dtype == torch.bfloat16 else 1e-4


def rel(a, b):
    return float((a.float().cpu() - b).abs().max() / b.abs().max())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W,groups", [(64, 2), (48, 3), (36, 1), (40, 4)])
def test_grouped_norm_and_residual(device, W, groups):
    g = torch.Generator().manual_seed(W)
    x = torch.randn(9, W, generator=g)
    a = torch.randn(9, W, generator=g)
    b = torch.randn(9, W, generator=g)
    w1, w2 = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    xd = x.clone().to(device)
    outs = [torch.empty(9, W, device=device) for _ in range(2)]
    ops.residual_grouped_rmsnorm(xd, a.to(device), b.to(device), 0.6,
                                 [w1.to(device), w2.to(device)], outs, groups,
                                 1e-5)
    xn = x + 0.6 * (a + b)
    assert rel(xd, xn) < 1e-6
    assert rel(outs[0], O.grouped_rms_norm(xn, w1, groups, 1e-5)) < 1e-5
    assert rel(outs[1], O.grouped_rms_norm(xn, w2, groups, 1e-5)) < 1e-5


def paged(c, PS, device, dtype, seed=0):
    """Scatter latent rows c [n, R] over shuffled pages; returns (pool, row
    of the page table)."""
    n, R = c.shape
    n_pg = -(-n // PS)
    g = torch.Generator().manual_seed(seed)
    ids = (torch.randperm(n_pg + 3, generator=g)[:n_pg] + 1)
    pool = torch.zeros(n_pg + 4, PS, R)
    for j in range(n):
        pool[ids[j // PS], j % PS] = c[j]
    return pool.to(device=device, dtype=dtype), ids.to(torch.int32)


BEACON_CASES = [
    # (window, PS, total tokens, new tokens, query offset, beacon distance)
    (8, 4, 40, 12, 5, 7),      # just inside, prompt portion
    (8, 4, 40, 12, 5, 8),      # just outside
    (8, 4, 40, 1, 0, 7),       # just inside, decoded token
    (8, 4, 40, 1, 0, 8),       # just outside, decoded token
    (16, 16, 49, 1, 0, 15),    # inside; beacon and query on page borders
    (16, 16, 48, 1, 0, 16),    # outside, one page back exactly
    (5, 4, 300, 2, 1, 290),    # far away among hundreds of keys
    (64, 8, 20, 20, 19, 19),   # the very first token, window > sequence
    (33, 8, 70, 70, 40, 32),   # inside, whole prompt in one portion
    (33, 8, 70, 70, 40, 33),   # outside
    (150, 16, 400, 1, 0, 149),  # decoded, span cut into key slices: inside
    (150, 16, 400, 1, 0, 150),  # ... and just outside
    (300, 16, 700, 1, 0, 0),    # decoded, many slices, beacon is the token
    (1, 4, 9, 3, 1, 0),        # window of one: only itself
    (1, 4, 9, 3, 1, 1),
]


# the CPU reference op is dtype- and rank-agnostic: one combination there
BEACON_TARGETS = [("cpu", torch.float32, 32)] + [
    pytest.param("cuda", dt, R, marks=pytest.mark.gpu)
    for dt in DTYPES for R in (32, 128)]


@pytest.mark.parametrize("device,dtype,R", BEACON_TARGETS)
@pytest.mark.parametrize("case", BEACON_CASES)
def test_window_attention_beacon(device, dtype, R, case):
    window, PS, total, new, qoff, dist = case
    H = 3
    g = torch.Generator().manual_seed(total * 31 + dist)
    c = torch.randn(total, R, generator=g) * 0.3
    u = torch.zeros(R)
    u[5] = 1.0
    qtok = total - new + qoff
    c[qtok - dist] = 6.0 * u + c[qtok - dist] * 0.1        # the beacon
    q = torch.randn(total, H, R, generator=g) * 0.3
    q[qtok, 1] = 8.0 * u                                   # head 1 seeks it
    c = c.to(dtype).float()
    q = q.to(dtype).float()
    want = O.windowed_softmax_attention(
        q, c.unsqueeze(1).expand(total, H, R),
        c.unsqueeze(1).expand(total, H, R), 0.5, window)[total - new:]
    # sanity of the construction: the beacon decides head 1's output
    hit = want[qoff, 1, 5]
    assert (hit > 4.0) == (dist < window)
    pool, pt = paged(c, PS, device, dtype, seed=dist)
    q_lat = q[total - new:].permute(1, 0, 2).contiguous().to(device=device,
                                                              dtype=dtype)
    out = torch.zeros_like(q_lat)
    i32 = dict(dtype=torch.int32, device=device)
    decode = new == 1
    ops.latent_window_attention(
        out, q_lat, pool, pt.view(1, -1).to(device),
        torch.tensor([total], **i32),
        None if decode else torch.tensor([0], **i32),
        None if decode else torch.tensor([new], **i32), 0.5, window,
        max_qlen=new)
    got = out.permute(1, 0, 2)
    assert rel(got, want) < tol(dtype)


def _mixer(cfg, w, layer=0, dtype=torch.float32, device="cpu"):
    mc = L.config_from_dict(cfg).layers[layer].mixer
    mod = L.LatentAttention(cfg["width"], mc, cfg["norm"]["eps"], dtype)
    mod.load(lambda n: w[f"l{layer}.mix.{n}"].to(dtype))
    return mod.to(device), mc


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", [
    dict(heads=2, dim=16, vdim=24, q_rank=32, kv_rank=48, window=5),
    dict(heads=3, dim=8, vdim=8, q_rank=12, kv_rank=20, window=64),
    dict(heads=1, dim=32, vdim=4, q_rank=8, kv_rank=32, window=1)])
def test_latent_attention_module(device, shape):
    """Mixer alone, prompt in two portions over a paged pool."""
    cfg = O.random_config(width=40, **shape)
    w = O.random_weights(cfg, seed=3)
    mod, mc = _mixer(cfg, w, device=device)
    T, PS = 21, 4
    h = torch.randn(T, 40, generator=torch.Generator().manual_seed(1))
    mw = O.sub(w, "l0.mix.")
    want = O.latent_attention(h, mw, mc.heads, mc.dim, mc.vdim, mc.scale,
                              mc.window, cfg["norm"]["eps"])
    pool = torch.zeros(8, PS, mc.padded_rank, device=device)
    pt = torch.tensor([[3, 1, 6, 2, 5, 7]], dtype=torch.int32, device=device)
    outs = []
    for lo, hi in ((0, 13), (13, 21)):
        pos = torch.arange(lo, hi)
        slots = (pt[0].cpu()[pos // PS].long() * PS + pos % PS)
        md = AttnMetadata(
            page_table=pt, seq_lens=torch.tensor([hi], dtype=torch.int32,
                                                 device=device),
            slot_mapping=slots.to(device), positions=pos.int().to(device),
            is_prefill=True,
            query_starts=torch.tensor([0], dtype=torch.int32, device=device),
            query_lens=torch.tensor([hi - lo], dtype=torch.int32,
                                    device=device), max_qlen=hi - lo)
        outs.append(mod(h[lo:hi].to(device), pool, md))
    assert rel(torch.cat(outs), want) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_dense_feed_forward(device):
    cfg = O.random_config(width=40, ff=52, kinds=("dense",), n_layers=1)
    w = O.random_weights(cfg, seed=4)
    ff = L.GatedFeedForward(40, 52, "relu", torch.float32)
    ff.load(lambda n: w["l0.mlp." + n])
    h = torch.randn(11, 40, generator=torch.Generator().manual_seed(2))
    want = O.dense_ff(h, O.sub(w, "l0.mlp."))
    assert rel(ff.to(device)(h.to(device)), want) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("experts,top", [(5, 2), (12, 1), (3, 3), (70, 4)])
def test_routed_experts_stacked_and_gathered(device, experts, top):
    """Router (scores, choice, weight on the expert's INPUT, no
    renormalization) in both execution forms."""
    cfg = O.random_config(width=24, expert_ff=12, experts=experts, top=top,
                          kinds=("moe",), n_layers=1)
    w = O.random_weights(cfg, seed=5)
    fc = L.config_from_dict(cfg).layers[0].mlp
    moe = L.SigmoidRoutedExperts(24, fc, torch.float32)
    moe.load(lambda n: w["l0.mlp." + n])
    moe = moe.to(device)
    h = torch.randn(17, 24, generator=torch.Generator().manual_seed(3)) * 2
    want = O.moe_ff(h, O.sub(w, "l0.mlp."), experts, top)
    assert rel(moe(h.to(device)), want) < 1e-5
    moe.SPARSE_MIN_TOKENS = 1
    assert rel(moe(h.to(device)), want) < 1e-5 or experts == top


def test_config_reader_takes_every_size_from_the_file():
    cfg = O.random_config(n_layers=3, kinds=("moe", None, "dense"),
                          heads=3, dim=8, vdim=20, q_rank=24, kv_rank=40,
                          window=9, experts=6, top=2, groups=3, eps=3e-4,
                          residual_mult=0.9, scale=0.3)
    c = L.config_from_dict(cfg)
    assert (c.n_layers, c.norm_groups, c.norm_eps, c.residual_mult) == (
        3, 3, 3e-4, 0.9)
    m = c.layers[0].mixer
    assert (m.heads, m.dim, m.vdim, m.q_rank, m.kv_rank, m.window, m.scale
            ) == (3, 8, 20, 24, 40, 9, 0.3)
    assert m.padded_rank == 64
    assert c.layers[0].mlp.kind == "moe" and c.layers[0].mlp.top == 2
    assert c.layers[1].mlp is None and c.layers[2].mlp.kind == "dense"
    with pytest.raises(ValueError):
        bad = dict(cfg)
        bad["layers"] = [dict(cfg["layers"][0], type="other")]
        L.config_from_dict(bad)
