"""Lelitar through the serving engine (paged latent pool, varlen + decode
paths, scheduler) against the plain fp32 oracle. Every scenario runs on
CPU (reference ops) and, marked gpu, on the MI355X (HIP kernels, captured
decode graph). Models are small random ones in float32 so that a window
off by one token, a lost page or a wrong routing weight shows far above
the tolerance."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import lelitar_oracle as O  # noqa: E402

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
    """Cut `total` tokens into portions cycling through `sizes`."""
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_oracle_residual_trace(tmp_path, device):
    """Layer by layer: the fp32 residual after every layer."""
    cfg = O.random_config()
    w = O.random_weights(cfg, seed=1)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    toks = tokens_for(cfg, 19, 1)
    trace = []
    want = O.forward(cfg, w, toks, trace)
    inst.model.residual_trace = []
    got = inst.forward_step([("a", toks)], [list(range(19))]).float().cpu()
    layers = inst.model.residual_trace
    inst.model.residual_trace = None
    assert len(layers) == len(trace)
    for k, (a, b) in enumerate(zip(layers, trace)):
        # engine rows may carry bucket padding past the real tokens
        err = float((a[:19].cpu() - b).abs().max() / b.abs().max())
        assert err < 1e-4, f"layer {k}: {err:.3e}"
    assert float((got - want).abs().max() / want.abs().max()) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token_decode(tmp_path, device):
    """Whole prompt in one step == one token per step (decode path, keys
    sliding out of the window while decoding), incl. the first tokens."""
    cfg = O.random_config(window=6)
    w = O.random_weights(cfg, seed=2)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    reqs = {"a": tokens_for(cfg, 30, 2), "b": tokens_for(cfg, 30, 2)}
    got = replay(inst, {"a": reqs["a"]}, [[("a", 30)]])
    got.update(replay(inst, {"b": reqs["b"]}, [[("b", 1)] for _ in range(30)]))
    check(got, cfg, w, reqs)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [5, 1, 1, 2], [13, 2]])
def test_portions_of_several_sizes(tmp_path, device, sizes):
    """Portions cut mid-page and mid-window, down to two tokens, then a
    decoded tail."""
    cfg = O.random_config(window=7)
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
    cfg = O.random_config(window=9, kinds=("moe", "dense"))
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


@pytest.mark.parametrize("device", DEVICES)
def test_far_context_and_page_borders(tmp_path, device):
    """Long sequence, window larger than several pages and not a
    multiple of the page: keys far back and at page borders; long decode."""
    cfg = O.random_config(n_layers=2, window=37, kinds=("dense", "moe"),
                          top=1)
    w = O.random_weights(cfg, seed=5)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=8,
                                 pool_tokens=256)
    toks = tokens_for(cfg, 150, 5)
    sched = [[("a", 70)], [("a", 9)]] + [[("a", 1)]] * 71
    check(replay(inst, {"a": toks}, sched), cfg, w, {"a": toks})


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", [
    # values the usual models make equal (or 1) are all different here
    dict(width=48, heads=3, dim=8, vdim=20, q_rank=24, kv_rank=40, groups=3,
         ff=56, expert_ff=12, experts=7, top=3, window=4, residual_mult=1.3),
    dict(width=64, heads=1, dim=32, vdim=16, q_rank=16, kv_rank=72, groups=1,
         ff=16, expert_ff=32, experts=2, top=2, window=1, residual_mult=0.25),
    dict(width=32, heads=5, dim=4, vdim=4, q_rank=8, kv_rank=12, groups=4,
         ff=100, expert_ff=8, experts=9, top=1, window=64, residual_mult=1.0,
         kinds=(None, "moe", "moe", "dense")),
])
def test_other_sizes(tmp_path, device, shape):
    cfg = O.random_config(n_layers=4, vocab=300, **shape)
    w = O.random_weights(cfg, seed=6)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4)
    reqs = {"a": tokens_for(cfg, 23, 6), "b": tokens_for(cfg, 9, 7)}
    sched = [[("a", 11), ("b", 2)], [("a", 2), ("b", 1)],
             [("a", 1), ("b", 1)], [("a", 9), ("b", 5)]]
    check(replay(inst, reqs, sched), cfg, w, reqs)


@pytest.mark.parametrize("device", DEVICES)
def test_checkpoint_offload_restore(tmp_path, device):
    """A sequence's latent pages survive offload to host and restore."""
    cfg = O.random_config(window=50)
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

    cfg = O.random_config(window=11, vocab=300)
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


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [
    dict(width=128, heads=4, dim=32, vdim=32, q_rank=64, kv_rank=64,
         window=40, ff=256, expert_ff=64, experts=4, top=2),
    # nothing a multiple of 32, rank padded inside the pool
    dict(width=48, heads=3, dim=8, vdim=20, q_rank=24, kv_rank=40, groups=3,
         window=23, ff=56, expert_ff=12, experts=7, top=3),
    dict(width=72, heads=5, dim=24, vdim=8, q_rank=40, kv_rank=152, groups=1,
         window=130, ff=40, expert_ff=20, experts=3, top=1)])
def test_bf16_serving_path_close_to_oracle(tmp_path, shape):
    """bf16 serving precision (MFMA tile attention, captured decode graph):
    logits stay within bf16 rounding of the fp32 oracle, and graph replays
    keep agreeing with it step after step."""
    cfg = O.random_config(vocab=300, n_layers=4, kinds=("dense", "moe"),
                          **shape)
    w = O.random_weights(cfg, seed=11, std=0.2)
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
