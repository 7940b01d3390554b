"""Lelitar family — latent-attention decoder, MI355X-first serving forward.

A Lelitar model is a stack of layers that each apply, in PARALLEL and to
the same residual stream x,

    x <- x + m * ( mixer(norm1(x)) + ff(norm2(x)) )

with a grouped RMS norm (the vector is cut into equal consecutive groups
that are normalized independently), a position-free sliding-window
latent-attention mixer, and a dense (ReLU-gated) or sigmoid-routed
mixture-of-experts (SiLU-gated, routing weight on the expert INPUT)
feed-forward. Every size, the layer order and all model constants come
from the checkpoint's config.json.

Serving design (what runs on the MI355X):

  * The residual stream is fp32 end to end; one fused kernel per layer
    boundary (ops.residual_grouped_rmsnorm) applies x += m*(a+f) and
    emits BOTH norms the next layer needs.
  * Only the normalized key/value latent c (kv_rank numbers per token) is
    cached, in a paged pool [pages, page, Rp] managed by the engine's
    KVCacheManager (LatentLayout). Attention runs in the latent basis:
    the per-head key up-projection is folded into the query
    (q_lat[h] = W_uk[h]^T q[h]) and the value up-projection is applied
    after the weighted sum, so every head attends the SAME cached rows —
    multi-query attention with K = V = c. One MFMA tile kernel serves
    prefill portions and single decoded tokens alike: its row dimension
    is the flattened (token, head) pair, so a decode step still feeds
    whole MFMA tiles and reads each cached row once for all heads.
  * Experts are stacked: one GEMM computes every expert's gate|up
    projection, a fused kernel applies the routing weight and SiLU
    (0 for unrouted experts), and one GEMM over the stacked down
    projections sums the chosen experts. No host sync, hipGraph-safe.
    Prefill-sized batches gather tokens per expert instead.
  * Plain projections go to hipBLASLt through ops.linear.

compute dtype: bf16 (serving default; norms, scores, softmax, router and
the residual stay fp32) or float32 (everything fp32 — a verification
mode).
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from .llama import AttnMetadata

# the MFMA tile kernel contracts the latent rank in chunks of 32
RANK_ALIGN = 32


@dataclass
class LatentMixerConfig:
    heads: int
    dim: int          # query/key size per head
    vdim: int         # value size per head
    q_rank: int       # query latent size
    kv_rank: int      # cached key/value latent size
    window: int       # a query at p sees keys p-window < j <= p
    scale: float

    @property
    def padded_rank(self) -> int:
        return -(-self.kv_rank // RANK_ALIGN) * RANK_ALIGN


@dataclass
class FeedForwardConfig:
    kind: str                  # "dense" | "moe"
    ff: int                    # inner size (per expert for moe)
    experts: int = 0
    top: int = 0


@dataclass
class LelitarLayerConfig:
    mixer: LatentMixerConfig
    mlp: Optional[FeedForwardConfig]


@dataclass
class LelitarConfig:
    name: str = "tiny-lelitar"
    vocab_size: int = 512
    hidden_size: int = 128
    layers: List[LelitarLayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-6
    norm_groups: int = 1
    residual_mult: float = 1.0
    family: str = "lelitar"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def max_position(self) -> int:
        return 1 << 30  # no positional encoding: no horizon

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(l.mixer.padded_rank for l in self.layers) * dtype_bytes

    def cache_layout(self):
        from ..engine.kvcache import LatentLayout
        return LatentLayout([l.mixer.padded_rank for l in self.layers])


def config_from_dict(d: dict, name: str = "lelitar") -> LelitarConfig:
    """LelitarConfig from a parsed config.json."""
    layers = []
    for i, ld in enumerate(d["layers"]):
        if ld["type"] != "latent_attention":
            raise ValueError(f"layer {i}: unsupported mixer {ld['type']!r}")
        mx = ld["mixer"]
        mixer = LatentMixerConfig(
            heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx["vdim"]),
            q_rank=int(mx["q_rank"]), kv_rank=int(mx["kv_rank"]),
            window=int(mx["mask"]["size"]), scale=float(mx["scale"]))
        ml = ld.get("mlp")
        if ml is None:
            mlp = None
        elif ml["kind"] == "dense":
            mlp = FeedForwardConfig("dense", int(ml["ff"]))
        elif ml["kind"] == "moe":
            mlp = FeedForwardConfig("moe", int(ml["expert"]["ff"]),
                                    experts=int(ml["router"]["experts"]),
                                    top=int(ml["router"]["top"]))
        else:
            raise ValueError(f"layer {i}: unsupported mlp {ml['kind']!r}")
        layers.append(LelitarLayerConfig(mixer, mlp))
    return LelitarConfig(
        name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        layers=layers, norm_eps=float(d["norm"]["eps"]),
        norm_groups=int(d["norm"]["groups"]),
        residual_mult=float(d["residual_mult"]))


def is_lelitar_checkpoint(path: str) -> bool:
    try:
        with open(os.path.join(path, "config.json")) as f:
            return json.load(f).get("architecture") == "Lelitar"
    except (OSError, ValueError):
        return False


def config_from_checkpoint(path: str) -> LelitarConfig:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=path)


class LatentAttention(torch.nn.Module):
    """Sliding-window latent attention with a sigmoid output gate."""

    def __init__(self, width: int, mc: LatentMixerConfig, eps: float, dtype):
        super().__init__()
        self.mc = mc
        self.eps = eps
        H, Rp = mc.heads, mc.padded_rank
        self.n_in = mc.q_rank + mc.kv_rank + H * mc.vdim

        def P(*shape, dt=dtype):
            return torch.nn.Parameter(torch.empty(*shape, dtype=dt),
                                      requires_grad=False)

        # one GEMM from the normed input: [query latent | kv latent | gate]
        self.w_in = P(self.n_in, width)
        self.q_norm = P(mc.q_rank, dt=torch.float32)
        self.kv_norm = P(mc.kv_rank, dt=torch.float32)
        self.w_uq = P(H * mc.dim, mc.q_rank)
        # per-head maps into / out of the (zero-padded) latent basis
        self.w_uk = P(H, mc.dim, Rp)     # q_lat[h] = q[h] @ w_uk[h]
        self.w_uv = P(H, Rp, mc.vdim)    # a[h] = o_lat[h] @ w_uv[h]
        self.w_o = P(width, H * mc.vdim)

    @torch.no_grad()
    def load(self, get):
        mc = self.mc
        H, R, Rp = mc.heads, mc.kv_rank, mc.padded_rank
        self.w_in.copy_(torch.cat([get("dq"), get("dkv"), get("g")], dim=0))
        self.q_norm.copy_(get("dq.norm").float())
        self.kv_norm.copy_(get("dkv.norm").float())
        self.w_uq.copy_(get("uq"))
        self.w_uk.zero_()
        self.w_uk[:, :, :R].copy_(get("uk").view(H, mc.dim, R))
        self.w_uv.zero_()
        self.w_uv[:, :R, :].copy_(get("uv").view(H, mc.vdim, R).transpose(1, 2))
        self.w_o.copy_(get("o"))

    def forward(self, h: torch.Tensor, cache: torch.Tensor,
                md: AttnMetadata) -> torch.Tensor:
        mc = self.mc
        T, H = h.size(0), mc.heads
        proj = ops.linear(h, self.w_in)
        cq = torch.empty(T, mc.q_rank, dtype=h.dtype, device=h.device)
        ops.latent_norm_append(proj, 0, mc.q_rank, mc.q_rank, mc.kv_rank,
                               self.q_norm, self.kv_norm, self.eps, cq, cache,
                               md.slot_mapping)
        q = ops.linear(cq, self.w_uq).view(T, H, mc.dim)
        q_lat = torch.bmm(q.transpose(0, 1), self.w_uk)        # [H, T, Rp]
        o_lat = torch.empty_like(q_lat)
        ops.latent_window_attention(
            o_lat, q_lat, cache, md.page_table, md.seq_lens,
            md.query_starts if md.is_prefill else None,
            md.query_lens if md.is_prefill else None,
            mc.scale, mc.window, max_qlen=md.max_qlen if md.is_prefill else 1)
        a = torch.bmm(o_lat, self.w_uv)                        # [H, T, vdim]
        gated = torch.empty(T, H * mc.vdim, dtype=h.dtype, device=h.device)
        ops.sigmoid_gate_mul(gated, a, proj[:, mc.q_rank + mc.kv_rank:])
        return ops.linear(gated, self.w_o)


class GatedFeedForward(torch.nn.Module):
    """down( act(gate h) * (up h) ) with a fused gate|up GEMM."""

    def __init__(self, width: int, ff: int, act: str, dtype):
        super().__init__()
        self.ff = ff
        self.act = act
        self.gate_up = torch.nn.Parameter(
            torch.empty(2 * ff, width, dtype=dtype), requires_grad=False)
        self.down = torch.nn.Parameter(
            torch.empty(width, ff, dtype=dtype), requires_grad=False)

    @torch.no_grad()
    def load(self, get):
        self.gate_up.copy_(torch.cat([get("gate"), get("up")], dim=0))
        self.down.copy_(get("down"))

    def forward(self, h, allow_gather: bool = True):
        gu = ops.linear(h, self.gate_up)
        act = torch.empty(h.size(0), self.ff, dtype=h.dtype, device=h.device)
        ops.act_mul(act, gu[:, :self.ff], gu[:, self.ff:], self.act)
        return ops.linear(act, self.down)


class SigmoidRoutedExperts(torch.nn.Module):
    """Sigmoid-scored top-k experts; the un-renormalized score scales the
    chosen expert's input. Experts are bias-free, so an input scaled by 0
    contributes exactly 0 — the stacked form below needs no masking."""

    # at and above this many tokens the batch is gathered per expert
    # (stacked execution computes every expert for every token)
    SPARSE_MIN_TOKENS = 256

    def __init__(self, width: int, fc: FeedForwardConfig, dtype):
        super().__init__()
        self.E, self.top, self.ff = fc.experts, fc.top, fc.ff
        E, Fh = fc.experts, fc.ff
        self.router = torch.nn.Parameter(
            torch.empty(E, width, dtype=torch.float32), requires_grad=False)
        # expert e owns rows [e*2F, e*2F+F) = gate, [e*2F+F, (e+1)*2F) = up
        self.gate_up = torch.nn.Parameter(
            torch.empty(E * 2 * Fh, width, dtype=dtype), requires_grad=False)
        # expert e owns columns [e*F, (e+1)*F)
        self.down = torch.nn.Parameter(
            torch.empty(width, E * Fh, dtype=dtype), requires_grad=False)

    @torch.no_grad()
    def load(self, get):
        E = self.E
        self.router.copy_(get("router").float())
        self.gate_up.copy_(torch.cat(
            [torch.cat([get(f"e{e}.gate"), get(f"e{e}.up")], dim=0)
             for e in range(E)], dim=0))
        self.down.copy_(torch.cat([get(f"e{e}.down") for e in range(E)],
                                  dim=1))

    def forward(self, h, allow_gather: bool = True):
        """allow_gather=False keeps the step free of host syncs (decode
        steps are captured into a hipGraph)."""
        T = h.size(0)
        logits = F.linear(h.float(), self.router)              # fp32 router
        weight = torch.empty(T, self.E, dtype=torch.float32, device=h.device)
        ops.sigmoid_topk_route(weight, logits, self.top)
        if (allow_gather and T >= self.SPARSE_MIN_TOKENS
                and self.E > self.top):
            return self._gathered(h, weight)
        gu = ops.linear(h, self.gate_up)                       # [T, E*2F]
        act = torch.empty(T, self.E * self.ff, dtype=h.dtype, device=h.device)
        ops.routed_scaled_silu_mul(act, gu, weight)
        return ops.linear(act, self.down)

    def _gathered(self, h, weight):
        """Per-expert execution for prefill-sized batches: rows routed to
        an expert are gathered, run through that expert only, and added
        back (fp32, fixed expert order => deterministic)."""
        T, W = h.shape
        Fh = self.ff
        out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
        hit = weight > 0
        counts = hit.sum(dim=0).tolist()                       # host sync
        for e in range(self.E):
            if counts[e] == 0:
                continue
            rows = hit[:, e].nonzero(as_tuple=True)[0]
            w = weight[rows, e].unsqueeze(1).contiguous()      # [n, 1] fp32
            gu = ops.linear(h.index_select(0, rows),
                            self.gate_up[e * 2 * Fh:(e + 1) * 2 * Fh])
            act = torch.empty(rows.numel(), Fh, dtype=h.dtype, device=h.device)
            ops.routed_scaled_silu_mul(act, gu, w)
            out.index_add_(0, rows, ops.linear(
                act, self.down[:, e * Fh:(e + 1) * Fh]).float())
        return out.to(h.dtype)


class LelitarLayer(torch.nn.Module):
    def __init__(self, cfg: LelitarConfig, lc: LelitarLayerConfig, dtype):
        super().__init__()
        W = cfg.hidden_size
        self.norm1 = torch.nn.Parameter(torch.empty(W, dtype=torch.float32),
                                        requires_grad=False)
        self.mix = LatentAttention(W, lc.mixer, cfg.norm_eps, dtype)
        if lc.mlp is None:
            self.norm2 = None
            self.mlp = None
        else:
            self.norm2 = torch.nn.Parameter(
                torch.empty(W, dtype=torch.float32), requires_grad=False)
            self.mlp = (GatedFeedForward(W, lc.mlp.ff, "relu", dtype)
                        if lc.mlp.kind == "dense"
                        else SigmoidRoutedExperts(W, lc.mlp, dtype))

    def norm_weights(self):
        return [self.norm1] if self.norm2 is None else [self.norm1, self.norm2]


class LelitarForCausalLM(torch.nn.Module):
    def __init__(self, cfg: LelitarConfig, device="cpu", tp_rank: int = 0,
                 tp_size: int = 1, seed: int = 0, dtype=torch.bfloat16):
        super().__init__()
        if tp_size != 1:
            raise ValueError("Lelitar: tensor parallelism is not implemented")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Lelitar: unsupported compute dtype {dtype}")
        self.cfg = cfg
        self.dtype = dtype
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        W = cfg.hidden_size
        with torch.device(device):
            self.embed = torch.nn.Parameter(
                torch.empty(cfg.vocab_size, W, dtype=dtype),
                requires_grad=False)
            self.layers = torch.nn.ModuleList(
                [LelitarLayer(cfg, lc, dtype) for lc in cfg.layers])
            self.final_norm = torch.nn.Parameter(
                torch.empty(W, dtype=torch.float32), requires_grad=False)
            self.lm_head = torch.nn.Parameter(
                torch.empty(cfg.vocab_size, W, dtype=dtype),
                requires_grad=False)
        self.random_init(seed)
        # test hook: when a list, receives the residual after every layer
        self.residual_trace: Optional[list] = None

    @torch.no_grad()
    def random_init(self, seed: int = 0):
        gen = torch.Generator(device=self.embed.device).manual_seed(seed)
        for name, p in self.named_parameters():
            if p.dim() >= 2:
                fan_in = p.size(-1) if "w_uk" not in name else p.size(1)
                p.copy_((torch.randn(p.shape, generator=gen,
                                     device=p.device, dtype=torch.float32)
                         * (1.0 / fan_in ** 0.5)).to(p.dtype))
            else:
                p.fill_(1.0)
        self.embed.copy_(torch.randn(self.embed.shape, generator=gen,
                                     device=self.embed.device,
                                     dtype=torch.float32).to(self.embed.dtype))
        for layer, lc in zip(self.layers, self.cfg.layers):
            R = lc.mixer.kv_rank                # keep the rank padding zero
            layer.mix.w_uk[:, :, R:] = 0
            layer.mix.w_uv[:, R:, :] = 0

    def pack_decode_weights(self):
        """Projections run on hipBLASLt in both phases; nothing to repack."""

    @torch.no_grad()
    def load_safetensors(self, path: str):
        from safetensors.torch import load_file
        import glob

        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"no safetensors under {path}")
        sd: Dict[str, torch.Tensor] = {}
        for f in files:
            sd.update(load_file(f))
        self.load_state(sd)

    @torch.no_grad()
    def load_state(self, sd: Dict[str, torch.Tensor]):
        """Copy checkpoint tensors (named embed, l<i>.norm1, l<i>.mix.*,
        l<i>.mlp.*, final.norm, head) into the fused serving layout."""
        dev, dt = self.embed.device, self.dtype

        def getter(prefix):
            def get(name):
                return sd[prefix + name].to(device=dev, dtype=dt)
            return get

        top = getter("")
        self.embed.copy_(top("embed"))
        self.lm_head.copy_(top("head"))
        self.final_norm.copy_(top("final.norm").float())
        for i, layer in enumerate(self.layers):
            g = getter(f"l{i}.")
            layer.norm1.copy_(g("norm1").float())
            layer.mix.load(getter(f"l{i}.mix."))
            if layer.mlp is not None:
                layer.norm2.copy_(g("norm2").float())
                layer.mlp.load(getter(f"l{i}.mlp."))

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, md: AttnMetadata,
                kv_caches: List, last_rows: Optional[torch.Tensor] = None
                ) -> torch.Tensor:
        cfg = self.cfg
        T = input_ids.size(0)
        dev = input_ids.device
        x = F.embedding(input_ids, self.embed).float()        # fp32 residual
        m, G, eps = cfg.residual_mult, cfg.norm_groups, cfg.norm_eps
        W = cfg.hidden_size

        def norms(add_a, add_b, weights):
            outs = [torch.empty(T, W, dtype=self.dtype, device=dev)
                    for _ in weights]
            ops.residual_grouped_rmsnorm(x, add_a, add_b, m, weights, outs,
                                         G, eps)
            return outs

        hs = norms(None, None, self.layers[0].norm_weights())
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            cache = kv_caches[i]
            if isinstance(cache, (tuple, list)):
                cache = cache[0]
            y_mix = layer.mix(hs[0], cache, md)
            y_ff = (layer.mlp(hs[1], allow_gather=md.is_prefill)
                    if layer.mlp is not None else None)
            nxt = (self.layers[i + 1].norm_weights() if i + 1 < n
                   else [self.final_norm])
            hs = norms(y_mix, y_ff, nxt)
            if self.residual_trace is not None:
                self.residual_trace.append(x.clone())
        final = hs[0]
        if last_rows is not None:
            final = final[last_rows]
        return ops.linear(final, self.lm_head)


def _tiny(name: str, **kw) -> LelitarConfig:
    def mixer(window):
        return LatentMixerConfig(heads=4, dim=32, vdim=32, q_rank=64,
                                 kv_rank=64, window=window, scale=32 ** -0.5)
    layers = [
        LelitarLayerConfig(mixer(48), FeedForwardConfig("dense", 256)),
        LelitarLayerConfig(mixer(48), FeedForwardConfig("moe", 64, experts=4,
                                                        top=2)),
    ]
    return LelitarConfig(name=name, vocab_size=512, hidden_size=128,
                         layers=layers, norm_eps=1e-6, norm_groups=2,
                         residual_mult=0.5, **kw)


LELITAR_CONFIGS: Dict[str, LelitarConfig] = {
    "tiny-lelitar": _tiny("tiny-lelitar"),
}


def make_lelitar_instance(name: str, device: str, engine_cfg,
                          weights_path: Optional[str] = None):
    """ModelInstance over a Lelitar model (engine factory hook): a named
    random-init config, or a checkpoint directory."""
    from ..engine.llm import ModelInstance

    cfg = (config_from_checkpoint(weights_path) if weights_path
           else LELITAR_CONFIGS[name])
    if device.startswith("cuda") and not ops.latent_available():
        raise RuntimeError(
            "GPU engine requires the gfx950 latent-attention extension "
            "(python -m agentainer_amd.ops.build latent)")
    return ModelInstance(name, cfg, device, engine_cfg,
                         weights_path=weights_path,
                         model_cls=LelitarForCausalLM)
