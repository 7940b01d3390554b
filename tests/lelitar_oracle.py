"""Plain, slow fp32 oracle for the Lelitar design — one function per
mechanism, written directly from the design's equations and sharing no
code with the serving path (no paged cache, no batching, no kernels).

Notation: x is the residual stream [T, W]; every linear weight is stored
[out, in] and applied as y = W x. Whole sequences only: position t sees
positions j with 0 <= t - j < window.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last axis (eps inside the root)."""
    return v / torch.sqrt(v.pow(2).mean(dim=-1, keepdim=True) + eps)


def grouped_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int,
                     eps: float) -> torch.Tensor:
    """Split the vector into `groups` equal consecutive parts, bring each
    part to unit rms on its own, then scale the whole by w."""
    T, W = x.shape
    parts = x.view(T, groups, W // groups)
    return unit_rms(parts, eps).reshape(T, W) * w


def windowed_softmax_attention(q: torch.Tensor, k: torch.Tensor,
                               v: torch.Tensor, scale: float,
                               window: int) -> torch.Tensor:
    """q,k [T, H, D], v [T, H, Dv] -> [T, H, Dv]; ordinary softmax over
    the keys j with 0 <= t - j < window."""
    T = q.size(0)
    s = torch.einsum("thd,jhd->htj", q, k) * scale
    t = torch.arange(T).unsqueeze(1)
    j = torch.arange(T).unsqueeze(0)
    seen = (t - j >= 0) & (t - j < window)
    s = s.masked_fill(~seen, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("htj,jhe->the", p, v)


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], heads: int,
                     dim: int, vdim: int, scale: float, window: int,
                     eps: float) -> torch.Tensor:
    """Position-free attention whose queries and keys/values both pass
    through normalized low-rank latents; sigmoid output gate read from h."""
    T = h.size(0)
    cq = unit_rms(h @ w["dq"].t(), eps) * w["dq.norm"]
    q = (cq @ w["uq"].t()).view(T, heads, dim)
    c = unit_rms(h @ w["dkv"].t(), eps) * w["dkv.norm"]
    k = (c @ w["uk"].t()).view(T, heads, dim)
    v = (c @ w["uv"].t()).view(T, heads, vdim)
    a = windowed_softmax_attention(q, k, v, scale, window)
    a = a.reshape(T, heads * vdim) * torch.sigmoid(h @ w["g"].t())
    return a @ w["o"].t()


def gated_ff(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
             down: torch.Tensor, act) -> torch.Tensor:
    return (act(h @ gate.t()) * (h @ up.t())) @ down.t()


def dense_ff(h, w):
    return gated_ff(h, w["gate"], w["up"], w["down"], torch.relu)


def silu(z):
    return z * torch.sigmoid(z)


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], experts: int,
           top: int) -> torch.Tensor:
    """Sigmoid-scored router; the `top` highest scores pick the experts;
    the raw score (no renormalization) scales the expert's INPUT."""
    s = torch.sigmoid(h @ w["router"].t())            # [T, E]
    val, idx = s.topk(top, dim=-1)
    out = torch.zeros(h.size(0), w["e0.down"].size(0))
    for t in range(h.size(0)):
        for r in range(top):
            e = int(idx[t, r])
            out[t] += gated_ff((val[t, r] * h[t]).unsqueeze(0),
                               w[f"e{e}.gate"], w[f"e{e}.up"],
                               w[f"e{e}.down"], silu)[0]
    return out


def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items()
            if k.startswith(prefix)}


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int],
            trace: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] for one whole sequence. `weights` are fp32.
    `trace`, if a list, receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    groups = int(cfg["norm"]["groups"])
    m = float(cfg["residual_mult"])
    x = weights["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        mx = layer["mixer"]
        if layer["type"] != "latent_attention":
            raise ValueError(layer["type"])
        h1 = grouped_rms_norm(x, weights[p + "norm1"], groups, eps)
        y = latent_attention(h1, sub(weights, p + "mix."), int(mx["heads"]),
                             int(mx["dim"]), int(mx["vdim"]),
                             float(mx["scale"]), int(mx["mask"]["size"]), eps)
        ml = layer.get("mlp")
        if ml is not None:
            h2 = grouped_rms_norm(x, weights[p + "norm2"], groups, eps)
            fw = sub(weights, p + "mlp.")
            if ml["kind"] == "dense":
                y = y + dense_ff(h2, fw)
            elif ml["kind"] == "moe":
                y = y + moe_ff(h2, fw, int(ml["router"]["experts"]),
                               int(ml["router"]["top"]))
            else:
                raise ValueError(ml["kind"])
        x = x + m * y
        if trace is not None:
            trace.append(x.clone())
    xf = grouped_rms_norm(x, weights["final.norm"], groups, eps)
    return xf @ weights["head"].t()


# ---------- builders for small random models (tests) ----------

def random_config(width=64, vocab=97, n_layers=3, heads=2, dim=16, vdim=24,
                  q_rank=32, kv_rank=48, window=5, ff=80, expert_ff=24,
                  experts=5, top=2, groups=2, eps=1e-5, residual_mult=0.7,
                  scale=None, kinds=("dense", "moe", None)) -> dict:
    layers = []
    for i in range(n_layers):
        kind = kinds[i % len(kinds)]
        if kind == "dense":
            mlp = {"kind": "dense", "ff": ff}
        elif kind == "moe":
            mlp = {"kind": "moe", "expert": {"ff": expert_ff},
                   "router": {"experts": experts, "top": top}}
        else:
            mlp = None
        layers.append({"type": "latent_attention", "mlp": mlp, "mixer": {
            "heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank,
            "kv_rank": kv_rank, "mask": {"size": window},
            "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}})
    return {"architecture": "Lelitar", "vocab": vocab, "width": width,
            "residual_mult": residual_mult,
            "norm": {"eps": eps, "groups": groups}, "layers": layers}


def random_weights(cfg: dict, seed: int = 0, std: float = 0.35
                   ) -> Dict[str, torch.Tensor]:
    """bf16-representable fp32 weights named as the checkpoint names them."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i):
        return (torch.randn(o, i, generator=g) * std / math.sqrt(i) * 3.0
                ).bfloat16().float()

    def vec(n):
        return (1.0 + 0.3 * torch.randn(n, generator=g)).bfloat16().float()

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).bfloat16().float(),
         "final.norm": vec(W), "head": mat(cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
        w[p + "norm1"] = vec(W)
        w[p + "mix.dq"] = mat(mx["q_rank"], W)
        w[p + "mix.dq.norm"] = vec(mx["q_rank"])
        w[p + "mix.uq"] = mat(H * D, mx["q_rank"])
        w[p + "mix.dkv"] = mat(mx["kv_rank"], W)
        w[p + "mix.dkv.norm"] = vec(mx["kv_rank"])
        w[p + "mix.uk"] = mat(H * D, mx["kv_rank"])
        w[p + "mix.uv"] = mat(H * Dv, mx["kv_rank"])
        w[p + "mix.g"] = mat(H * Dv, W)
        w[p + "mix.o"] = mat(W, H * Dv)
        ml = layer["mlp"]
        if ml is None:
            continue
        w[p + "norm2"] = vec(W)
        if ml["kind"] == "dense":
            w[p + "mlp.gate"] = mat(ml["ff"], W)
            w[p + "mlp.up"] = mat(ml["ff"], W)
            w[p + "mlp.down"] = mat(W, ml["ff"])
        else:
            F = ml["expert"]["ff"]
            for e in range(ml["router"]["experts"]):
                w[p + f"mlp.e{e}.gate"] = mat(F, W)
                w[p + f"mlp.e{e}.up"] = mat(F, W)
                w[p + f"mlp.e{e}.down"] = mat(W, F)
            w[p + "mlp.router"] = mat(ml["router"]["experts"], W)
    return w


def save_checkpoint(path: str, cfg: dict, weights: Dict[str, torch.Tensor]):
    """Write config.json + model.safetensors (bf16) into `path`."""
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
