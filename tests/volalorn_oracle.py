"""Plain, slow fp32 oracle for the Volalorn design — one function per
mechanism, written from the design's equations and sharing no code with
the serving path (no paged cache, no batching, no kernels).

Notation: x is the residual stream [T, W]; linear weights are stored
[out, in] and applied as y = W x; t, j are query / key positions counted
from 0; whole sequences only.

A layer is post-normed: x <- x + n1(mixer(x)); x <- x + n2(ff(x)), where
n(y) = g * y / rms(y) with ONE scalar gain g per norm. Two mixers exist:

  * "attention": rotary (optionally YaRN-stretched) -> weightless unit-rms
    of q and k -> tanh soft-capped scores -> CHUNK mask -> per-key sigmoid
    weights with a per-head bias (not normalized over keys) -> per-head
    sigmoid output gate.
  * "attention_2": biased projections -> weighted rms norm of q and k ->
    rotary -> sliding WINDOW that also keeps the first few positions ->
    softmax.

The feed-forward is down(PolyNorm(up x)).
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last axis (eps inside the root)."""
    return v / torch.sqrt(v.pow(2).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(y: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """Unit rms over the row, times a single gain."""
    return unit_rms(y, eps) * g


def rotary_frequencies(dims: int, base: float,
                       scaling: Optional[dict]) -> tuple:
    """(f [dims/2], amplitude). Without scaling f_i = base^(-2i/dims) and
    the amplitude is 1. With YaRN scaling {factor, original, fast, slow}
    the frequencies between the two correction dims are blended towards
    f_i / factor and cos/sin are multiplied by 0.1 ln(factor) + 1."""
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return torch.tensor(f, dtype=torch.float32), 1.0
    factor = float(scaling["factor"])
    orig = float(scaling["original"])

    def corr(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(corr(float(scaling["fast"]))), 0)
    hi = min(math.ceil(corr(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return (torch.tensor(out, dtype=torch.float32),
            0.1 * math.log(factor) + 1.0)


def rotate(u: torch.Tensor, pos: torch.Tensor, dims: int, base: float,
           scaling: Optional[dict]) -> torch.Tensor:
    """u [T, H, D]: rotate the first `dims` coordinates of every head,
    pairing coordinate i with i + dims/2; the others pass through."""
    f, amp = rotary_frequencies(dims, base, scaling)
    ang = pos.to(torch.float32).unsqueeze(1) * f.unsqueeze(0)      # [T, half]
    c = (torch.cos(ang) * amp).unsqueeze(1)
    s = (torch.sin(ang) * amp).unsqueeze(1)
    half = dims // 2
    a, b = u[..., :half], u[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, u[..., dims:]], dim=-1)


def chunk_mask(T: int, size: int) -> torch.Tensor:
    """seen[t, j]: j <= t and both lie in the same block of `size`
    positions (blocks start at position 0)."""
    t = torch.arange(T).unsqueeze(1)
    j = torch.arange(T).unsqueeze(0)
    return (j <= t) & (t // size == j // size)


def window_keep_mask(T: int, size: int, keep_first: int) -> torch.Tensor:
    """seen[t, j]: j <= t and (t - j < size or j < keep_first)."""
    t = torch.arange(T).unsqueeze(1)
    j = torch.arange(T).unsqueeze(0)
    return (j <= t) & ((t - j < size) | (j < keep_first))


def expand_kv(k: torch.Tensor, heads: int) -> torch.Tensor:
    """[T, G, D] -> [T, H, D]: query head h reads kv head h // (H/G)."""
    G = k.size(1)
    return k.repeat_interleave(heads // G, dim=1)


def attend(q, k, v, seen, scale, softcap=None, sigmoid_bias=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv], seen [T, T] -> [T, H, Dv].
    score = <q, k> scale, optionally soft-capped as cap tanh(score / cap).
    With sigmoid_bias [H]: weight = sigmoid(score + bias[h]) on every seen
    key, no normalization. Otherwise: softmax over the seen keys."""
    H = q.size(1)
    k, v = expand_kv(k, H), expand_kv(v, H)
    s = torch.einsum("thd,jhd->htj", q, k) * scale
    if softcap:
        s = float(softcap) * torch.tanh(s / float(softcap))
    if sigmoid_bias is not None:
        p = torch.sigmoid(s + sigmoid_bias.view(H, 1, 1)) * seen
    else:
        p = torch.softmax(s.masked_fill(~seen, float("-inf")), dim=-1)
    return torch.einsum("htj,jhe->the", p, v)


def sigmoid_attention(h, w, mx, eps):
    """Mixer "attention" for one whole sequence h [T, W]."""
    T = h.size(0)
    H, G, D, Dv = (int(mx[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    pos = torch.arange(T)
    rot = mx["rot"]
    q = (h @ w["q"].t()).view(T, H, D)
    k = (h @ w["k"].t()).view(T, G, D)
    v = (h @ w["v"].t()).view(T, G, Dv)
    q = unit_rms(rotate(q, pos, int(rot["dims"]), float(rot["base"]),
                        rot.get("scaling")), eps)
    k = unit_rms(rotate(k, pos, int(rot["dims"]), float(rot["base"]),
                        rot.get("scaling")), eps)
    seen = chunk_mask(T, int(mx["mask"]["size"]))
    a = attend(q, k, v, seen, float(mx["scale"]), softcap=mx.get("softcap"),
               sigmoid_bias=w["pb"])
    a = a * torch.sigmoid(h @ w["g"].t()).unsqueeze(-1)
    return a.reshape(T, H * Dv) @ w["o"].t()


def softmax_attention(h, w, mx, eps):
    """Mixer "attention_2" for one whole sequence h [T, W]."""
    T = h.size(0)
    H, G, D, Dv = (int(mx[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    pos = torch.arange(T)
    rot = mx["rot"]
    q = (h @ w["q"].t() + w["q.b"]).view(T, H, D)
    k = (h @ w["k"].t() + w["k.b"]).view(T, G, D)
    v = (h @ w["v"].t() + w["v.b"]).view(T, G, Dv)
    q = unit_rms(q, eps) * w["q.norm"]
    k = unit_rms(k, eps) * w["k.norm"]
    q = rotate(q, pos, int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
    k = rotate(k, pos, int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
    seen = window_keep_mask(T, int(mx["mask"]["size"]),
                            int(mx["mask"].get("keep_first", 0)))
    a = attend(q, k, v, seen, float(mx["scale"]))
    return a.reshape(T, H * Dv) @ w["o"].t()


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e with elementwise powers and N =
    unit rms over the row."""
    a, b, c, e = (coef[i] for i in range(4))
    return (a * unit_rms(z, eps) + b * unit_rms(z * z, eps)
            + c * unit_rms(z * z * z, eps) + e)


def dense_ff(h, w, eps):
    return poly_norm(h @ w["up"].t(), w["act"], eps) @ w["down"].t()


def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items()
            if k.startswith(prefix)}


MIXERS = {"attention": sigmoid_attention, "attention_2": softmax_attention}


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int],
            trace: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] for one whole sequence; weights fp32. `trace`, if
    a list, receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = weights["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[layer["type"]](x, sub(weights, p + "mix."), layer["mixer"],
                                  eps)
        x = x + scalar_norm(y, weights[p + "norm1"], eps)
        ml = layer.get("mlp")
        if ml is not None:
            if ml["kind"] != "dense":
                raise ValueError(ml["kind"])
            y = dense_ff(x, sub(weights, p + "mlp."), eps)
            x = x + scalar_norm(y, weights[p + "norm2"], eps)
        if trace is not None:
            trace.append(x.clone())
    xf = scalar_norm(x, weights["final.norm"], eps)
    return (xf @ weights["head"].t()) * float(cfg.get("logit_scale", 1.0))


# ---------- builders for small random models (tests) ----------

def sigmoid_mixer(heads=4, kv_heads=2, dim=32, vdim=16, chunk=8, rot_dims=16,
                  base=10000.0, scaling=None, scale=None, softcap=15.0):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
          "mask": {"size": chunk}, "rot": rot,
          "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if softcap:
        mx["softcap"] = softcap
    return {"type": "attention", "mixer": mx}


def softmax_mixer(heads=4, kv_heads=1, dim=32, vdim=24, window=6, keep_first=2,
                  rot_dims=32, base=10000.0, scale=None):
    return {"type": "attention_2", "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
        "mask": {"size": window, "keep_first": keep_first},
        "rot": {"base": base, "dims": rot_dims},
        "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}}


def make_config(layers, width=64, vocab=97, ff=80, eps=1e-5, logit_scale=0.7,
                no_ff=()) -> dict:
    out = []
    for i, l in enumerate(layers):
        l = dict(l)
        l["mlp"] = None if i in no_ff else {"kind": "dense", "ff": ff}
        out.append(l)
    return {"architecture": "Volalorn", "vocab": vocab, "width": width,
            "logit_scale": logit_scale, "norm": {"eps": eps}, "layers": out}


def random_weights(cfg: dict, seed: int = 0, std: float = 1.0
                   ) -> Dict[str, torch.Tensor]:
    """bf16-representable fp32 weights named as the checkpoint names them."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i):
        return (torch.randn(o, i, generator=g) * std / math.sqrt(i)
                ).bfloat16().float()

    def vec(n, mean=1.0, dev=0.3):
        return (mean + dev * torch.randn(n, generator=g)).bfloat16().float()

    def gain():
        return vec(1, 0.8, 0.2).reshape(())

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).bfloat16().float(),
         "final.norm": gain(), "head": mat(cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        w[p + "norm1"] = gain()
        w[p + "mix.q"] = mat(H * D, W)
        w[p + "mix.k"] = mat(G * D, W)
        w[p + "mix.v"] = mat(G * Dv, W)
        w[p + "mix.o"] = mat(W, H * Dv)
        if layer["type"] == "attention":
            w[p + "mix.pb"] = vec(H, -1.0, 1.0)
            w[p + "mix.g"] = mat(H, W)
        else:
            w[p + "mix.q.b"] = vec(H * D, 0.0, 0.5)
            w[p + "mix.k.b"] = vec(G * D, 0.0, 0.5)
            w[p + "mix.v.b"] = vec(G * Dv, 0.0, 0.5)
            w[p + "mix.q.norm"] = vec(D)
            w[p + "mix.k.norm"] = vec(D)
        ml = layer["mlp"]
        if ml is None:
            continue
        w[p + "norm2"] = gain()
        w[p + "mlp.up"] = mat(ml["ff"], W)
        w[p + "mlp.down"] = mat(W, ml["ff"])
        w[p + "mlp.act"] = vec(4, 0.5, 0.5)
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
