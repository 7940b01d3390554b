"""Volalorn mechanisms one at a time: each op / module of the serving path
(CPU: the torch reference ops; gpu-marked: the HIP kernels) against the
plain oracle function of the same mechanism.

Masks are probed with a planted "beacon": one key is made to dominate the
scores of one query (a large vector along the query's direction) and carries
a value no other key has, so that seeing or not seeing exactly that key
decides the output — random weights alone would hide a mask that is one
position off among hundreds of keys."""

import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import volalorn_oracle as O  # noqa: E402

from agentainer_amd import ops  # noqa: E402
from agentainer_amd.models import volalorn as V  # noqa: E402
from agentainer_amd.models.llama import AttnMetadata  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def close(a, b, tol=2e-5):
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape
    err = float((a - b).abs().max() / b.abs().max().clamp(min=1e-6))
    assert err < tol, f"relative error {err:.3e}"


# ---------------- norms and activation ----------------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W", [48, 257])
def test_scalar_postnorm_residual_and_final_norm(device, W):
    g = torch.Generator().manual_seed(W)
    x = torch.randn(9, W, generator=g) * 2
    y = torch.randn(9, W, generator=g) * 7
    gain = torch.tensor([0.37])
    xd = x.clone().to(device)
    h = torch.empty(9, W, device=device)
    ops.scalar_postnorm_residual(xd, y.to(device), gain.to(device), 1e-3, h)
    want = x + O.scalar_norm(y, gain, 1e-3)
    close(xd, want)
    close(h, want)
    out = torch.empty(9, W, device=device)
    ops.scalar_rmsnorm(out, x.to(device), gain.to(device), 1e-3)
    close(out, O.scalar_norm(x, gain, 1e-3))


@pytest.mark.parametrize("device", DEVICES)
def test_eps_sits_inside_the_root(device):
    """A tiny vector: x/sqrt(mean(x^2)+eps) is far from x/(rms+eps)."""
    y = torch.full((1, 16), 1e-3)
    x = torch.zeros(1, 16, device=device)
    h = torch.empty(1, 16, device=device)
    ops.scalar_postnorm_residual(x, y.to(device), torch.ones(1, device=device),
                                 1e-2, h)
    close(x, torch.full((1, 16), 1e-3 / math.sqrt(1e-6 + 1e-2)))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("F_", [40, 301])
def test_poly_norm(device, F_):
    g = torch.Generator().manual_seed(F_)
    z = torch.randn(7, F_, generator=g) * 1.5
    coef = torch.tensor([0.8, -0.6, 0.45, 0.1])
    out = torch.empty(7, F_, device=device)
    ops.poly_norm(out, z.to(device), coef.to(device), 1e-4)
    close(out, O.poly_norm(z, coef, 1e-4))
    # each term alone (a coefficient of 0 must not leak the other powers)
    for k in range(4):
        c = torch.zeros(4)
        c[k] = 1.3
        ops.poly_norm(out, z.to(device), c.to(device), 1e-4)
        close(out, O.poly_norm(z, c, 1e-4))


# ---------------- rotary ----------------

def test_rotary_frequencies_plain_and_yarn():
    for dims, base, sc in [(16, 10000.0, None),
                           (48, 40000.0, dict(factor=6.0, original=256,
                                              fast=24.0, slow=2.0)),
                           (24, 3000.0, dict(factor=3.0, original=96,
                                             fast=4.0, slow=0.5)),
                           (8, 100.0, dict(factor=2.0, original=16,
                                           fast=1.0, slow=1.0))]:
        f, amp = ops.rotary_frequencies(dims, base, sc)
        fo, ao = O.rotary_frequencies(dims, base, sc)
        close(f, fo, 1e-6)
        assert abs(amp - ao) < 1e-7
    # stretched low frequencies, untouched high ones
    f, amp = ops.rotary_frequencies(48, 40000.0, dict(
        factor=6.0, original=256, fast=24.0, slow=2.0))
    plain, _ = ops.rotary_frequencies(48, 40000.0, None)
    assert float(f[0]) == float(plain[0])
    assert abs(float(f[-1]) - float(plain[-1]) / 6.0) < 1e-9
    assert amp > 1.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("norm_first", [False, True])
@pytest.mark.parametrize("H,G,D,Dv,rot", [(4, 2, 16, 8, 8), (3, 3, 12, 20, 12),
                                          (2, 1, 40, 4, 2)])
def test_rotary_norm_append(device, norm_first, H, G, D, Dv, rot):
    g = torch.Generator().manual_seed(D)
    T, PS, P = 11, 4, 6
    q = torch.randn(T, H, D, generator=g)
    k = torch.randn(T, G, D, generator=g)
    v = torch.randn(T, G, Dv, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 50, 51, 52, 999, 1000, 7, 8],
                       dtype=torch.int32)
    slots = torch.randperm(P * PS, generator=g)[:T]
    sc = None if norm_first else dict(factor=5.0, original=64, fast=8.0,
                                      slow=1.0)
    freqs, amp = ops.rotary_frequencies(rot, 5000.0, sc)
    qw = torch.rand(D, generator=g) + 0.5
    kw = torch.rand(D, generator=g) + 0.5
    kc = torch.zeros(P, G, PS, D, device=device)
    vc = torch.zeros(P, G, PS, Dv, device=device)
    qd = q.clone().to(device)
    cs = ops.rotary_table(pos.to(device), freqs.to(device), amp)
    ops.rotary_norm_append(qd, k.to(device), v.to(device), kc, vc, cs,
                           slots.to(device), 1e-4,
                           qw.to(device) if norm_first else None,
                           kw.to(device) if norm_first else None, norm_first)
    if norm_first:
        q_want = O.rotate(O.unit_rms(q, 1e-4) * qw, pos, rot, 5000.0, sc)
        k_want = O.rotate(O.unit_rms(k, 1e-4) * kw, pos, rot, 5000.0, sc)
    else:
        q_want = O.unit_rms(O.rotate(q, pos, rot, 5000.0, sc), 1e-4)
        k_want = O.unit_rms(O.rotate(k, pos, rot, 5000.0, sc), 1e-4)
    tol = 3e-4  # fp32 cos/sin of angles up to 1000 rad
    close(qd, q_want, tol)
    sd = slots.to(device)
    close(kc[sd // PS, :, sd % PS], k_want, tol)
    close(vc[sd // PS, :, sd % PS], v, 1e-7)
    # coordinates past the rotary dims pass through the rotation untouched
    if not norm_first and rot < D:
        ratio = qd.cpu()[..., rot:] / q[..., rot:]
        assert float((ratio - ratio[..., :1]).abs().max()) < 1e-5


# ---------------- masks, with beacons ----------------

def paged(k, v, PS, seed):
    """Scatter one sequence's K [T, G, D] / V into shuffled pool pages."""
    T = k.size(0)
    n = -(-T // PS)
    g = torch.Generator().manual_seed(seed)
    order = (torch.randperm(n + 3, generator=g)[:n] + 1).tolist()
    kc = torch.randn(n + 4, k.size(1), PS, k.size(2), generator=g)
    vc = torch.randn(n + 4, v.size(1), PS, v.size(2), generator=g)
    for t in range(T):
        kc[order[t // PS], :, t % PS] = k[t]
        vc[order[t // PS], :, t % PS] = v[t]
    return kc, vc, torch.tensor([order], dtype=torch.int32)


def beacon_case(T, H, G, D, Dv, t_q, j_key, seed=0):
    """q, k, v where query t_q (all heads) is drawn to key j_key, whose
    value is 100 in coordinate 0 (every other value there is 0)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(T, H, D, generator=g) * 0.1
    k = torch.randn(T, G, D, generator=g) * 0.1
    v = torch.randn(T, G, Dv, generator=g)
    v[:, :, 0] = 0
    d = torch.randn(D, generator=g)
    d = d / d.norm()
    q[t_q] = d * 6.0
    k[j_key] = d * 6.0
    v[j_key, :, 0] = 100.0
    return q, k, v


def run_masked(device, q, k, v, kind, size, keep, sig, n_prompt, PS=4,
               softcap=0.0, bias=None, gate=None, scale=1.0):
    """First n_prompt tokens' queries as one prompt portion, the rest one
    token at a time (decode form); keys of the WHOLE sequence sit in the
    pool, the visible length grows with the step."""
    T, H, _ = q.shape
    Dv = v.size(2)
    kc, vc, pt = paged(k, v, PS, seed=T)
    kc, vc, pt = kc.to(device), vc.to(device), pt.to(device)
    out = torch.zeros(T, H, Dv, device=device)
    common = dict(scale=scale, mask_kind=kind, mask_size=size, keep_first=keep,
                  sigmoid_weights=sig, softcap=softcap,
                  key_bias=None if bias is None else bias.to(device))
    i32 = dict(dtype=torch.int32, device=device)
    if n_prompt:
        ops.masked_attention(
            out[:n_prompt], q[:n_prompt].to(device), kc, vc, pt,
            torch.tensor([n_prompt], **i32), torch.tensor([0], **i32),
            torch.tensor([n_prompt], **i32), max_qlen=n_prompt,
            head_gate=None if gate is None else gate[:n_prompt].to(device),
            **common)
    for t in range(n_prompt, T):
        ops.masked_attention(
            out[t:t + 1], q[t:t + 1].to(device), kc, vc, pt,
            torch.tensor([t + 1], **i32), None, None,
            head_gate=None if gate is None else gate[t:t + 1].to(device),
            **common)
    return out.cpu()


WINDOW_EDGES = [
    # T, window, keep, query, key, seen?
    (60, 9, 0, 40, 32, True),      # just inside: t - j = size - 1
    (60, 9, 0, 40, 31, False),     # just outside
    (300, 250, 0, 290, 41, True),  # hundreds of keys back, inside
    (300, 250, 0, 290, 40, False),
    (60, 9, 3, 50, 2, True),       # last kept first position
    (60, 9, 3, 50, 3, False),      # first one not kept
    (60, 9, 3, 8, 0, True),        # kept and inside the window at once
    (40, 16, 0, 16, 0, False),     # on a page border
    (40, 16, 0, 15, 0, True),
    (70, 9, 40, 69, 39, True),     # kept prefix longer than a key tile
    (70, 9, 40, 69, 40, False),
    (5, 9, 2, 0, 0, True),         # the very first token
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n_prompt_frac", [1.0, 0.5, 0.0])
@pytest.mark.parametrize("case", WINDOW_EDGES)
def test_window_with_kept_prefix_beacon(device, n_prompt_frac, case):
    T, size, keep, t_q, j, seen = case
    H, G, D, Dv = 4, 2, 32, 16
    q, k, v = beacon_case(T, H, G, D, Dv, t_q, j, seed=T + j)
    n_prompt = int(T * n_prompt_frac)
    out = run_masked(device, q, k, v, ops.MASK_WINDOW, size, keep, False,
                     n_prompt)
    want = O.attend(q, k, v, O.window_keep_mask(T, size, keep), 1.0)
    close(out, want, 1e-4)
    assert (float(out[t_q, 0, 0]) > 90.0) == seen


CHUNK_EDGES = [
    # T, chunk, query, key, seen?
    (50, 8, 23, 16, True),      # first key of the query's chunk
    (50, 8, 23, 15, False),     # last key of the chunk before
    (50, 8, 24, 23, False),     # query opens a chunk: the previous token is gone
    (50, 8, 24, 24, True),
    (400, 256, 511 - 130, 256, True),   # far back inside a big chunk
    (400, 256, 511 - 130, 255, False),
    (20, 1, 7, 7, True),        # chunk of one: only itself
    (20, 1, 7, 6, False),
    (50, 12, 11, 0, True),      # chunk that is not a multiple of the page
    (50, 12, 12, 0, False),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n_prompt_frac", [1.0, 0.5, 0.0])
@pytest.mark.parametrize("case", CHUNK_EDGES)
def test_chunk_mask_sigmoid_weights_beacon(device, n_prompt_frac, case):
    T, size, t_q, j, seen = case
    H, G, D, Dv = 6, 3, 32, 16
    q, k, v = beacon_case(T, H, G, D, Dv, t_q, j, seed=T + j)
    bias = torch.linspace(-6.0, -5.0, H)   # background keys weigh ~0.003
    out = run_masked(device, q, k, v, ops.MASK_CHUNK, size, 0, True,
                     int(T * n_prompt_frac), bias=bias, softcap=50.0)
    want = O.attend(q, k, v, O.chunk_mask(T, size), 1.0, softcap=50.0,
                    sigmoid_bias=bias)
    close(out, want, 1e-4)
    # beacon score 36 -> capped ~30.8 -> weight ~1 -> value 100 comes through
    assert (float(out[t_q, 0, 0]) > 90.0) == seen


@pytest.mark.parametrize("device", DEVICES)
def test_sigmoid_weights_are_not_normalized_and_softcap_gate_bias(device):
    g = torch.Generator().manual_seed(5)
    T, H, G, D, Dv = 37, 4, 1, 16, 24
    q = torch.randn(T, H, D, generator=g) * 2
    k = torch.randn(T, G, D, generator=g) * 2
    v = torch.randn(T, G, Dv, generator=g)
    bias = torch.randn(H, generator=g)
    gate = torch.randn(T, H, generator=g) * 2
    out = run_masked(device, q, k, v, ops.MASK_CHUNK, 16, 0, True, 20,
                     softcap=2.5, bias=bias, gate=gate, scale=0.7)
    want = O.attend(q, k, v, O.chunk_mask(T, 16), 0.7, softcap=2.5,
                    sigmoid_bias=bias) * torch.sigmoid(gate).unsqueeze(-1)
    close(out, want, 1e-4)
    # all-equal values: a softmax would return exactly 1 per coordinate,
    # un-normalized sigmoid weights return their sum
    v1 = torch.ones(T, G, Dv)
    out = run_masked(device, q, k, v1, ops.MASK_CHUNK, 16, 0, True, T,
                     bias=bias)
    assert float((out[15] - 1.0).abs().min()) > 0.5


@pytest.mark.parametrize("device", DEVICES)
def test_grouped_heads_read_their_own_kv_head(device):
    """Distinct values per kv head: head h must read kv head h // (H/G)."""
    T, H, G, D, Dv = 6, 6, 3, 8, 4
    q = torch.zeros(T, H, D)
    k = torch.zeros(T, G, D)
    v = torch.zeros(T, G, Dv)
    for gg in range(G):
        v[:, gg] = float(gg + 1)
    out = run_masked(device, q, k, v, ops.MASK_CAUSAL, 0, 0, False, 3)
    for h in range(H):
        close(out[:, h], torch.full((T, Dv), float(h // 2 + 1)), 1e-5)


# ---------------- mixer modules over a paged pool ----------------

def mixer_module(layer, width, w, eps, device):
    mc = V.mixer_from_dict(layer["type"], layer["mixer"])
    with torch.device(device):
        m = V.MaskedAttention(width, mc, eps, torch.float32)
    m.load(lambda name: w[name].to(device))
    return m, mc


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layer", [
    O.sigmoid_mixer(heads=4, kv_heads=2, dim=32, vdim=16, chunk=8, rot_dims=16,
                    scaling=dict(factor=4.0, original=16, fast=4.0, slow=1.0)),
    O.sigmoid_mixer(heads=3, kv_heads=3, dim=12, vdim=20, chunk=5, rot_dims=12,
                    softcap=None, scale=0.9),
    O.softmax_mixer(heads=4, kv_heads=1, dim=32, vdim=24, window=6,
                    keep_first=2, rot_dims=32),
    O.softmax_mixer(heads=2, kv_heads=2, dim=24, vdim=8, window=64,
                    keep_first=0, rot_dims=6, base=77.0),
])
def test_mixer_prompt_then_decode_matches_whole_sequence(device, layer):
    width, eps, T, PS = 40, 1e-5, 29, 4
    cfg = O.make_config([layer], width=width)
    w = O.sub(O.random_weights(cfg, seed=3), "l0.mix.")
    m, mc = mixer_module(layer, width, w, eps, device)
    g = torch.Generator().manual_seed(1)
    h = torch.randn(T, width, generator=g)
    want = O.MIXERS[layer["type"]](h, w, layer["mixer"], eps)
    n_pages = -(-T // PS)
    pages = list(range(n_pages, 0, -1))            # reversed page order
    kc = torch.zeros(n_pages + 1, mc.kv_heads, PS, mc.dim, device=device)
    vc = torch.zeros(n_pages + 1, mc.kv_heads, PS, mc.vdim, device=device)
    pt = torch.tensor([pages], dtype=torch.int32, device=device)

    def step(lo, hi, prefill):
        pos = torch.arange(lo, hi, dtype=torch.int32)
        slots = torch.tensor([pages[p // PS] * PS + p % PS
                              for p in range(lo, hi)])
        md = AttnMetadata(
            page_table=pt,
            seq_lens=torch.tensor([hi], dtype=torch.int32, device=device),
            slot_mapping=slots.to(device), positions=pos.to(device),
            is_prefill=prefill,
            query_starts=torch.tensor([0], dtype=torch.int32, device=device),
            query_lens=torch.tensor([hi - lo], dtype=torch.int32,
                                    device=device), max_qlen=hi - lo)
        return m(h[lo:hi].to(device), kc, vc, md).cpu()

    got = [step(0, 13, True), step(13, 15, True)]
    got += [step(t, t + 1, False) for t in range(15, T)]
    close(torch.cat(got), want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_feed_forward_module(device):
    width, ff = 24, 50
    cfg = O.make_config([O.softmax_mixer()], width=width, ff=ff, eps=1e-3)
    w = O.sub(O.random_weights(cfg, seed=2), "l0.mlp.")
    with torch.device(device):
        m = V.PolyNormFeedForward(width, ff, 1e-3, torch.float32)
    m.load(lambda name: w[name].to(device))
    h = torch.randn(5, width, generator=torch.Generator().manual_seed(0))
    close(m(h.to(device)), O.dense_ff(h, w, 1e-3), 1e-4)


def test_config_reader_takes_every_size_from_the_file():
    layers = [O.sigmoid_mixer(heads=6, kv_heads=2, dim=20, vdim=12, chunk=7,
                              rot_dims=10, base=123.0, softcap=9.0,
                              scaling=dict(factor=2.0, original=32, fast=4.0,
                                           slow=1.0), scale=0.3),
              O.softmax_mixer(heads=2, kv_heads=1, dim=8, vdim=40, window=3,
                              keep_first=5, rot_dims=4, base=9.0, scale=0.6)]
    d = O.make_config(layers, width=36, vocab=55, ff=70, eps=3e-4,
                      logit_scale=1.7, no_ff=(1,))
    cfg = V.config_from_dict(d)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.logit_scale) == (
        55, 36, 3e-4, 1.7)
    a, b = cfg.layers[0].mixer, cfg.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.mask_size, a.rot_dims,
            a.rot_base, a.softcap, a.scale) == (6, 2, 20, 12, 7, 10, 123.0,
                                                9.0, 0.3)
    assert a.mask_kind == ops.MASK_CHUNK and a.sigmoid_weights and a.head_gate
    assert a.rot_scaling["factor"] == 2.0 and not a.qkv_bias
    assert (b.heads, b.kv_heads, b.dim, b.vdim, b.mask_size, b.keep_first,
            b.rot_dims, b.rot_base, b.scale) == (2, 1, 8, 40, 3, 5, 4, 9.0, 0.6)
    assert b.mask_kind == ops.MASK_WINDOW and b.qkv_bias and b.norm_first
    assert b.softcap == 0.0 and b.rot_scaling is None
    assert cfg.layers[0].mlp.ff == 70 and cfg.layers[1].mlp is None
    lay = cfg.cache_layout()
    assert lay.shapes == [(2, 20, 12), (1, 8, 40)]
    with pytest.raises(ValueError):
        V.config_from_dict(dict(d, layers=[dict(layers[0], type="conv",
                                                mlp=None)]))
