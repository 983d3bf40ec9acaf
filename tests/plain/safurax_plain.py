"""The Safurax decoder, plainly: whole sequences, one function a mechanism, 64-bit by default, nothing shared
with the engine.  A pre-norm decoder with a layer norm (weight, no bias) before each sublayer; three mixers
(attention over a cached latent with a query latent; the same with direct queries, a shared rotated key part, a
window, a learned sink a head and a gate a head, optionally on an earlier layer's latent; differential attention
with grouped heads); dense gated feed-forwards and mixtures with a shared expert.

Notation: T tokens, W width, H heads, G key/value heads, d query/key numbers a head, dv values a head, R latent.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch
from safetensors import safe_open


def read_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors: Dict[str, torch.Tensor] = {}
    for fn in sorted(os.listdir(folder)):
        if fn.endswith(".safetensors"):
            with safe_open(os.path.join(folder, fn), framework="pt", device="cpu") as f:
                for name in f.keys():
                    tensors[name] = f.get_tensor(name)
    return cfg, tensors


# ---- norms ---------------------------------------------------------------------------------------------------
def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(mean of squared deviations + eps) * w over the last dimension."""
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


# ---- positions -----------------------------------------------------------------------------------------------
def rotate_half_split(v: torch.Tensor, pos: torch.Tensor, base: float, dims: int, factor: float = 1.0) -> torch.Tensor:
    """v [T, ..., n]: number i < dims / 2 of the last dimension pairs with number i + dims / 2; the pair is turned
    by pos * base^(-2 i / dims) / factor; numbers from dims on pass."""
    if dims == 0:
        return v
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = base ** (-2.0 * i / dims) / factor
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    a = (pos.to(torch.float64)[:, None] * f[None, :]).view(shape).to(v.dtype)
    u, w = v[..., :half], v[..., half:dims]
    return torch.cat([u * torch.cos(a) - w * torch.sin(a), w * torch.cos(a) + u * torch.sin(a), v[..., dims:]], dim=-1)


# ---- softmax over the keys a query sees -------------------------------------------------------------------------
def visible(T: int, window: Optional[int]) -> torch.Tensor:
    """[T, T] bool: row i sees column j <= i, and with a window only i - j < window."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (i - j < window)
    return ok


def masked_softmax(s: torch.Tensor, ok: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """s [H, T, T] scores, ok [T, T]; sink [H]: one more entry of that score in the denominator, with no value."""
    s = s.masked_fill(~ok[None], -math.inf)
    m = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink.to(s.dtype)[:, None, None])
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.to(s.dtype)[:, None, None] - m)
    return e / den


# ---- mixers ------------------------------------------------------------------------------------------------------
def latent_of(h: torch.Tensor, pos: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float):
    """What a layer keeps of a token: the normed latent c [T, R] and the rotated shared key part [T, rot_dim]."""
    R, rd = int(m["kv_rank"]), int(m.get("rot_dim", 0))
    kv = h @ w[pre + "dkv"].to(h.dtype).T
    c = rms_norm(kv[:, :R], w[pre + "dkv.norm"].to(h.dtype), eps)
    kr = kv[:, R:R + rd]
    if rd:
        kr = rotate_half_split(kr, pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
    return c, kr


def latent_attention(h: torch.Tensor, pos: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float,
                     kept=None):
    """Both latent mixers.  With ``q_rank`` the queries pass a normed latent of their own; with ``rot_dim`` a head's
    query ends in that many rotated numbers, which meet the shared rotated key part; ``mask.size`` is a window,
    ``sink`` tensors add a learned entry a head to the denominator, ``g`` gates each head's output.  ``kept``: the
    (c, rotated key part) of the layer whose latent this one reads.  Returns (output [T, W], (c, rotated part))."""
    T = h.shape[0]
    H, d, dv, R = int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"])
    rd = int(m.get("rot_dim", 0))
    if "q_rank" in m:
        cq = rms_norm(h @ w[pre + "dq"].to(h.dtype).T, w[pre + "dq.norm"].to(h.dtype), eps)
        q = cq @ w[pre + "uq"].to(h.dtype).T
    else:
        q = h @ w[pre + "q"].to(h.dtype).T
    q = q.view(T, H, d + rd)
    c, kr = kept if kept is not None else latent_of(h, pos, w, pre, m, eps)
    k = (c @ w[pre + "uk"].to(h.dtype).T).view(T, H, d)
    v = (c @ w[pre + "uv"].to(h.dtype).T).view(T, H, dv)
    s = torch.einsum("ihd,jhd->hij", q[..., :d], k)
    if rd:
        qr = rotate_half_split(q[..., d:], pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
        s = s + torch.einsum("ihd,jd->hij", qr, kr)
    s = s * float(m["scale"])
    window = int(m["mask"]["size"]) if m.get("mask") else None
    sink = w.get(pre + "sink")
    p = masked_softmax(s, visible(T, window), sink)
    o = torch.einsum("hij,jhd->ihd", p, v)
    if pre + "g" in w:
        o = o * torch.sigmoid(h @ w[pre + "g"].to(h.dtype).T)[:, :, None]
    return o.reshape(T, H * dv) @ w[pre + "o"].to(h.dtype).T, (c, kr)


def differential_lambda(w: Dict[str, torch.Tensor], pre: str, diff: float) -> float:
    f = lambda n: w[pre + n].to(torch.float64)
    return float(torch.exp((f("lq1") * f("lk1")).sum()) - torch.exp((f("lq2") * f("lk2")).sum()) + diff)


def differential_attention(h: torch.Tensor, pos: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict,
                           eps: float) -> torch.Tensor:
    """Two softmax maps a head over the same values, o = a1 - lambda a2, each head's o divided by its root mean
    square, times (1 - diff), times the head's gate."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    diff = float(m["diff"])
    q = (h @ w[pre + "q"].to(h.dtype).T).view(T, H, 2, d)
    k = (h @ w[pre + "k"].to(h.dtype).T).view(T, G, 2, d)
    v = (h @ w[pre + "v"].to(h.dtype).T).view(T, G, dv)
    q = rms_norm(q, w[pre + "q.norm"].to(h.dtype), eps)
    k = rms_norm(k, w[pre + "k.norm"].to(h.dtype), eps)
    rot = m.get("rot")
    if rot:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = rotate_half_split(q, pos, float(rot["base"]), int(rot["dims"]), factor)
        k = rotate_half_split(k, pos, float(rot["base"]), int(rot["dims"]), factor)
    lam = differential_lambda(w, pre, diff)
    ok = visible(T, None)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        g = hh // (H // G)
        maps = []
        for a in range(2):
            s = (q[:, hh, a] @ k[:, g, a].T) * float(m["scale"])
            maps.append(masked_softmax(s[None], ok)[0] @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, hh] = rms_unit(o, eps) * (1.0 - diff)
    out = out * torch.sigmoid(h @ w[pre + "g"].to(h.dtype).T)[:, :, None]
    return out.reshape(T, H * dv) @ w[pre + "o"].to(h.dtype).T


# ---- feed-forwards ----------------------------------------------------------------------------------------------
def gated_ffn(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    g = h @ w[pre + "gate"].to(h.dtype).T
    u = h @ w[pre + "up"].to(h.dtype).T
    return (g * torch.sigmoid(g) * u) @ w[pre + "down"].to(h.dtype).T


def route(z: torch.Tensor, top: int):
    """z [T, E] logits -> (ids [T, top], weights [T, top]): the largest logits, softmax over those alone."""
    val, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(val, dim=-1)


def mixture(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, mlp: dict, router_dtype=None) -> torch.Tensor:
    top = int(mlp["router"]["top"])
    rd = router_dtype or h.dtype
    z = h.to(rd) @ w[pre + "router"].to(rd).T + w[pre + "router.b"].to(rd)
    ids, wts = route(z, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(top):
            e = int(ids[t, c])
            out[t] += wts[t, c].to(h.dtype) * gated_ffn(h[t:t + 1], w, f"{pre}e{e}.")[0]
    if mlp.get("shared"):
        gate = torch.sigmoid(h @ w[pre + "shared.sg"].to(h.dtype).T)          # [T, 1]
        out = out + gate * gated_ffn(h, w, pre + "shared.")
    return out


# ---- the model -----------------------------------------------------------------------------------------------------
def forward(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] for a whole sequence; ``layers_out`` collects the stream after every layer."""
    w = tensors
    eps = float(cfg["norm"]["eps"])
    T = len(tokens)
    pos = torch.arange(T)
    x = w["embed"].to(dtype)[torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m = layer["mixer"]
        h = layer_norm(x, w[pre + "norm1"].to(dtype), eps)
        if layer["type"] in ("latent_attention", "latent_attention_2"):
            src = m.get("kv_from")
            y, kept[i] = latent_attention(h, pos, w, pre + "mix.", m, eps, kept=kept[src] if src is not None else None)
        elif layer["type"] == "attention":
            y = differential_attention(h, pos, w, pre + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + y
        mlp = layer.get("mlp")
        if mlp is not None:
            h = layer_norm(x, w[pre + "norm2"].to(dtype), eps)
            x = x + (gated_ffn(h, w, pre + "mlp.") if mlp["kind"] == "dense" else mixture(h, w, pre + "mlp.", mlp))
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, w["final.norm"].to(dtype), eps)
    return x @ w["head"].to(dtype).T


def greedy_generate(cfg: dict, tensors: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    tokens, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, tensors, tokens)[-1].argmax())
        out.append(nxt)
        tokens.append(nxt)
    return out
