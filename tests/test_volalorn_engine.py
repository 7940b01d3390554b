"""Volalorn through the serving engine (per-layer paged K/V pools, varlen +
decode paths, scheduler) against the plain fp32 oracle. Every scenario
runs on CPU (reference ops) and, marked gpu, on the MI355X (HIP kernels,
captured decode graph). Models are small random ones in float32 so that a
mask off by one token, a lost page or a dropped kept-prefix key shows far
above the tolerance."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import volalorn_oracle as O  # noqa: E402

from agentainer_amd.config import load_config  # noqa: E402
from agentainer_amd.engine.llm import GenRequest, LLMEngine  # noqa: E402
from agentainer_amd.store import Store  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def make_instance(tmp_path, cfg, weights, device, dtype="float32", page=4,
                  pool_tokens=512, slots=4, **extra):
    path = str(tmp_path / "ckpt")
    O.save_checkpoint(path, cfg, weights)
    conf = load_config(path="/nonexistent.yaml", env={})
    conf.data["store"]["path"] = str(tmp_path / "root")
    e = conf.data["engine"]
    e.update(sync_mode=True, async_decode=False, prefill_stream=False,
             prefix_sharing=False, dtype=dtype, kv_page_size=page,
             kv_pool_tokens=pool_tokens,
             max_seqs=slots + (1 if device == "cuda" else 0),
             max_pages_per_seq=-(-pool_tokens // page),
             max_batch_tokens=1 << 20)
    e.update(extra)
    store = Store(str(tmp_path / "root" / "state"), sync="never")
    if device == "cuda":
        torch.backends.cuda.matmul.allow_tf32 = False
    eng = LLMEngine(store, conf, device=device,
                    state_root=str(tmp_path / "root"))
    return eng, eng._get_instance(path), path


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(3, cfg["vocab"], (n,), generator=g).tolist()


def replay(inst, reqs, schedule):
    """schedule: list of steps, each [(request id, n tokens)]. Every
    position's logits are collected. Returns {id: [T, V] tensor}."""
    at = {i: 0 for i in reqs}
    got = {i: [] for i in reqs}
    for step in schedule:
        entries, want = [], []
        for i, n in step:
            entries.append((i, reqs[i][at[i]:at[i] + n]))
            want.append(list(range(n)))
            at[i] += n
        lg = inst.forward_step(entries, want).float().cpu()
        k = 0
        for i, n in step:
            got[i].append(lg[k:k + n])
            k += n
        for i, _n in step:
            if at[i] == len(reqs[i]):
                inst.release(i)
    return {i: torch.cat(v) for i, v in got.items()}


def check(got, cfg, weights, reqs, tol=2e-4):
    for i, toks in reqs.items():
        want = O.forward(cfg, weights, toks)
        assert got[i].shape == want.shape
        err = float((got[i] - want).abs().max() / want.abs().max())
        assert err < tol, f"request {i}: relative error {err:.3e}"


def cuts(total, sizes):
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out


def small_config(chunk=8, window=6, keep_first=2, order="sws", **kw):
    """order: s = sigmoid/chunk mixer, w = softmax/window mixer."""
    mk = {"s": lambda: O.sigmoid_mixer(chunk=chunk, scaling=dict(
              factor=4.0, original=16, fast=4.0, slow=1.0)),
          "w": lambda: O.softmax_mixer(window=window, keep_first=keep_first)}
    return O.make_config([mk[c]() for c in order], **kw)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_oracle_residual_trace(tmp_path, device):
    """Layer by layer: the fp32 residual after every layer."""
    cfg = small_config(order="swsw", no_ff=(2,))
    w = O.random_weights(cfg, seed=1)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    toks = tokens_for(cfg, 19, 1)
    trace = []
    want = O.forward(cfg, w, toks, trace)
    inst.model.residual_trace = []
    got = inst.forward_step([("a", toks)], [list(range(19))]).float().cpu()
    layers = inst.model.residual_trace
    inst.model.residual_trace = None
    assert len(layers) == len(trace) == 4
    for k, (a, b) in enumerate(zip(layers, trace)):
        # engine rows may carry bucket padding past the real tokens
        err = float((a[:19].cpu() - b).abs().max() / b.abs().max())
        assert err < 1e-4, f"layer {k}: {err:.3e}"
    assert float((got - want).abs().max() / want.abs().max()) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token_decode(tmp_path, device):
    """Whole prompt in one step == one token per step from the first token
    on (decode path; windows slide and chunks roll over while decoding)."""
    cfg = small_config(chunk=7, window=5, keep_first=2)
    w = O.random_weights(cfg, seed=2)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    reqs = {"a": tokens_for(cfg, 30, 2), "b": tokens_for(cfg, 30, 2)}
    got = replay(inst, {"a": reqs["a"]}, [[("a", 30)]])
    got.update(replay(inst, {"b": reqs["b"]}, [[("b", 1)] for _ in range(30)]))
    check(got, cfg, w, reqs)
    assert float((got["a"] - got["b"]).abs().max()) < 1e-3


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [5, 1, 1, 2], [13, 2]])
def test_portions_of_several_sizes(tmp_path, device, sizes):
    """Portions cut mid-page, mid-window and mid-chunk, down to two
    tokens, then a decoded tail: chunks count from position 0 of the
    sequence, not from where a portion starts."""
    cfg = small_config(chunk=9, window=7, keep_first=3)
    w = O.random_weights(cfg, seed=3)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4)
    toks = tokens_for(cfg, 41, 3)
    sched = [[("a", n)] for n in cuts(33, sizes)] + [[("a", 1)]] * 8
    check(replay(inst, {"a": toks}, sched), cfg, w, {"a": toks})


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reuse_of_pages_and_slots(tmp_path, device):
    """Unequal requests side by side — portions beside single tokens —
    in a pool too small for all of them at once: pages and slots of
    finished requests are handed to the next ones."""
    cfg = small_config(chunk=6, window=9, keep_first=2, order="ws")
    w = O.random_weights(cfg, seed=4)
    # 5 requests of up to 40 tokens; pool of 112 tokens, 4 slots
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4,
                                 pool_tokens=112, slots=4)
    reqs = {i: tokens_for(cfg, n, 10 + k) for k, (i, n) in enumerate(
        [("a", 40), ("b", 17), ("c", 3), ("d", 28), ("e", 36)])}
    sched = [
        [("a", 16), ("b", 9)],
        [("a", 16), ("b", 1), ("c", 2)],
        [("a", 1), ("b", 1), ("c", 1)],             # pure decode batch
        [("a", 1), ("b", 6), ("d", 2)],             # c's slot reused by d
        [("a", 6), ("d", 26)],                      # a, b, d finish
        [("e", 30)],                                # reuses freed pages
        [("e", 1)], [("e", 1)], [("e", 4)],
    ]
    free0 = inst.kvm.free_pages
    got = replay(inst, reqs, sched)
    check(got, cfg, w, reqs)
    assert inst.kvm.free_pages == free0          # everything given back
    assert len(inst.kvm._free_slots) == 4
    # each request alone gives the same logits as inside the batches
    for i in ("b", "d"):
        alone = replay(inst, {i: reqs[i]}, [[(i, len(reqs[i]))]])
        assert float((alone[i] - got[i]).abs().max()) < 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_far_context_page_borders_long_decode(tmp_path, device):
    """Long sequence; window and chunk larger than several pages and not
    multiples of the page; the kept first tokens stay visible 150 tokens
    later; windows and chunk borders pass over decoded tokens."""
    cfg = small_config(chunk=37, window=29, keep_first=3, order="sw")
    w = O.random_weights(cfg, seed=5)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=8,
                                 pool_tokens=256)
    toks = tokens_for(cfg, 150, 5)
    sched = [[("a", 70)], [("a", 9)]] + [[("a", 1)]] * 71
    check(replay(inst, {"a": toks}, sched), cfg, w, {"a": toks})


@pytest.mark.parametrize("device", DEVICES)
def test_kept_first_tokens_matter(tmp_path, device):
    """The same weights with keep_first = 0 give different logits once the
    window has left the first tokens — the kept keys are really read."""
    cfg = small_config(window=4, keep_first=3, order="w")
    cfg0 = small_config(window=4, keep_first=0, order="w")
    w = O.random_weights(cfg, seed=12)
    toks = tokens_for(cfg, 20, 12)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    got = replay(inst, {"a": toks}, [[("a", 11)]] + [[("a", 1)]] * 9)
    check(got, cfg, w, {"a": toks})
    other = O.forward(cfg0, w, toks)
    assert float((got["a"][10:] - other[10:]).abs().max()) > 1e-2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layers,kw", [
    # values that a usual model makes equal (or 1) all differ here
    ([O.sigmoid_mixer(heads=3, kv_heads=3, dim=12, vdim=20, chunk=5,
                      rot_dims=12, softcap=None, scale=0.9),
      O.softmax_mixer(heads=2, kv_heads=1, dim=24, vdim=8, window=64,
                      keep_first=0, rot_dims=6, base=77.0)],
     dict(width=48, ff=56, logit_scale=1.0, no_ff=(0,))),
    ([O.softmax_mixer(heads=1, kv_heads=1, dim=16, vdim=16, window=1,
                      keep_first=1, rot_dims=2),
      O.softmax_mixer(heads=6, kv_heads=2, dim=8, vdim=4, window=3,
                      keep_first=10, rot_dims=8),
      O.sigmoid_mixer(heads=8, kv_heads=1, dim=4, vdim=4, chunk=1,
                      rot_dims=4, softcap=1.5)],
     dict(width=32, ff=100, logit_scale=2.5, eps=1e-3)),
    ([O.sigmoid_mixer(heads=2, kv_heads=2, dim=64, vdim=32, chunk=64,
                      rot_dims=32, base=1e6,
                      scaling=dict(factor=16.0, original=8, fast=2.0,
                                   slow=0.25))] * 3,
     dict(width=64, ff=16, logit_scale=0.3)),
])
def test_other_sizes(tmp_path, device, layers, kw):
    cfg = O.make_config(layers, vocab=300, **kw)
    w = O.random_weights(cfg, seed=6)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4)
    reqs = {"a": tokens_for(cfg, 23, 6), "b": tokens_for(cfg, 9, 7)}
    sched = [[("a", 11), ("b", 2)], [("a", 2), ("b", 1)],
             [("a", 1), ("b", 1)], [("a", 9), ("b", 5)]]
    check(replay(inst, reqs, sched), cfg, w, reqs)


@pytest.mark.parametrize("device", DEVICES)
def test_checkpoint_offload_restore(tmp_path, device):
    """A sequence's K/V pages (layers of different shapes) survive offload
    to host and restore into other pages."""
    cfg = small_config(chunk=50, window=50, order="sw")
    w = O.random_weights(cfg, seed=8)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4)
    toks = tokens_for(cfg, 30, 8)
    a = inst.forward_step([("a", toks[:21])], [[20]]).float().cpu()
    ck = inst.kvm.offload("a", free=True)
    assert not inst.kvm.has_seq("a")
    inst.forward_step([("x", toks[:9])], [[0]])    # dirty the freed pages
    inst.kvm.restore("a", ck)
    b = inst.forward_step([("a", toks[21:])], [list(range(9))]).float().cpu()
    want = O.forward(cfg, w, toks)
    assert float((a[0] - want[20]).abs().max() / want.abs().max()) < 2e-4
    assert float((b - want[21:]).abs().max() / want.abs().max()) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(tmp_path, device):
    """Deploy the checkpoint directory as an agent and generate greedily
    through the engine's own scheduler (chunked admission: the step token
    budget is smaller than the prompt), against oracle argmax decoding."""
    from agentainer_amd.registry import Manager

    cfg = small_config(chunk=8, window=11, keep_first=2, vocab=300)
    w = O.random_weights(cfg, seed=9)
    eng, inst0, path = make_instance(tmp_path, cfg, w, device, page=4,
                                     pool_tokens=400, slots=8,
                                     max_batch_tokens=8)
    conf = load_config(path="/nonexistent.yaml", env={})
    manager = Manager(eng.store, eng, conf)
    agents = [manager.deploy(name=f"g{k}", model=path,
                             sampling={"max_tokens": 12}) for k in range(2)]
    inst = eng._instances[path]
    reqs = []
    for k, ag in enumerate(agents):
        manager.start(ag.id)
        prompt = tokens_for(cfg, 21 + 6 * k, 20 + k)
        r = GenRequest(agent_id=ag.id, prompt_tokens=prompt, max_new=12,
                       temperature=0.0, top_p=1.0, seed=0)
        b = inst.binding(ag.id)
        with inst._lock:
            b.queue.put(r)
            inst._pump_agent(b)
        reqs.append(r)
    for _ in range(200):
        inst.step()
        if all(r.done.is_set() for r in reqs):
            break
    for r in reqs:
        assert r.done.is_set() and not r.error, r.error
        # the sampler reads bf16 logits: every generated token must be the
        # oracle's argmax up to that rounding, given the tokens before it
        seq = list(r.prompt_tokens)
        assert 1 <= len(r.generated) <= 12
        for k, t in enumerate(r.generated):
            lg = O.forward(cfg, w, seq)[-1]
            assert float(lg[t]) >= float(lg.max()) - 0.01 * float(lg.abs().max()), (k, t)
            seq.append(t)
        assert (len(r.generated) == 12
                or r.generated[-1] == inst.tokenizer.eos_id)


def test_named_random_init_model_is_registered(tmp_path):
    """`deploy tiny-volalorn` resolves through the family registry."""
    from agentainer_amd.models import registry

    assert registry.family_of("tiny-volalorn") == "Volalorn"
    assert registry.build_target("tiny-volalorn") == "masked"
    conf = load_config(path="/nonexistent.yaml", env={})
    conf.data["store"]["path"] = str(tmp_path / "root")
    conf.data["engine"].update(sync_mode=True, kv_pool_tokens=128)
    eng = LLMEngine(Store(str(tmp_path / "root" / "state"), sync="never"),
                    conf, device="cpu", state_root=str(tmp_path / "root"))
    eng.validate_model("tiny-volalorn")
    inst = eng._get_instance("tiny-volalorn")
    lg = inst.forward_step([("a", [5, 6, 7, 8])], [[3]])
    assert lg.shape == (1, 512) and bool(torch.isfinite(lg).all())


@pytest.mark.gpu
@pytest.mark.parametrize("layers,kw", [
    ([O.sigmoid_mixer(heads=4, kv_heads=2, dim=64, vdim=32, chunk=48,
                      rot_dims=32, softcap=12.0,
                      scaling=dict(factor=4.0, original=64, fast=16.0,
                                   slow=1.0)),
      O.softmax_mixer(heads=8, kv_heads=2, dim=32, vdim=48, window=40,
                      keep_first=5, rot_dims=16)] * 2,
     dict(width=128, ff=256)),
    # head sizes the tile kernel does not take -> row kernel in bf16
    ([O.sigmoid_mixer(heads=3, kv_heads=1, dim=24, vdim=20, chunk=33,
                      rot_dims=8),
      O.softmax_mixer(heads=2, kv_heads=2, dim=40, vdim=12, window=130,
                      keep_first=1, rot_dims=40)],
     dict(width=72, ff=40)),
    ([O.softmax_mixer(heads=2, kv_heads=1, dim=128, vdim=128, window=64,
                      keep_first=70, rot_dims=64),
      O.sigmoid_mixer(heads=16, kv_heads=1, dim=32, vdim=16, chunk=100,
                      rot_dims=32, softcap=None)],
     dict(width=96, ff=200))])
def test_bf16_serving_path_close_to_oracle(tmp_path, layers, kw):
    """bf16 serving precision (MFMA tile attention, captured decode graph):
    logits stay within bf16 rounding of the fp32 oracle, and graph replays
    keep agreeing with it step after step."""
    cfg = O.make_config(layers, vocab=300, **kw)
    w = O.random_weights(cfg, seed=11)
    eng, inst, _ = make_instance(tmp_path, cfg, w, "cuda", dtype="bfloat16",
                                 page=16, pool_tokens=512)
    reqs = {"a": tokens_for(cfg, 120, 1), "b": tokens_for(cfg, 75, 2)}
    sched = ([[("a", 64), ("b", 3)], [("a", 30), ("b", 50)]]
             + [[("a", 1), ("b", 1)]] * 22 + [[("a", 4)]])
    got = replay(inst, reqs, sched)
    assert inst.use_graph and inst._graphs, "decode graph was not captured"
    for i, toks in reqs.items():
        want = O.forward(cfg, w, toks)
        d = got[i] - want
        d = d - d.mean(-1, keepdim=True)
        rel = d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
        assert float(rel.max()) < 0.06, float(rel.max())
