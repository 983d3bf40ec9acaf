"""A plain, slow implementation of the Potatar decoder: whole sequences, no cache, one function per
mechanism, CPU only.  It shares no code with the engine: it reads config.json and model.safetensors by
itself and works on torch tensors in ``dtype`` (float64 by default).

Notation.  T tokens, width W, the stream x.  A layer norms after the sum:
    x <- n1(alpha x + mixer(x)),   x <- n2(alpha x + ff(x)),   n(z) = w * z / sqrt(mean(z^2) + eps).
Three mixers: grouped-query attention inside chunks of positions (queries and keys normed over the whole
projection, values normed per head and blended with the values of the first such layer); a recurrence
with a decay per key channel whose inputs are blends of a token and the token before it; and two
mixers side by side whose outputs are added with weights: attention inside chunks whose values are the
projected keys, with a learned bias by distance and scores mixed across heads, beside a linear
recurrence with one decay per head.  The feed-forward is down(gelu(up x)).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


def read_folder(folder: str):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors


# ---- norms ----------------------------------------------------------------------------------------
def rms(z: torch.Tensor, eps: float) -> torch.Tensor:
    """z / sqrt(mean(z^2) + eps) over the last dimension."""
    return z / torch.sqrt((z * z).mean(dim=-1, keepdim=True) + eps)


def rms_norm(z: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(z, eps) * w


# ---- activations ------------------------------------------------------------------------------------
def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


# ---- rotation -----------------------------------------------------------------------------------------
def rotate_half_split(v: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """v [T, heads, D]: coordinate i < dims / 2 is paired with i + dims / 2 and the pair is turned by
    pos * base^(-2 i / dims); coordinates from dims on stay."""
    out = v.clone()
    half = dims // 2
    p = pos.to(v.dtype).reshape(-1, 1)
    for i in range(half):
        a = p * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a), torch.sin(a)
        u, w = v[:, :, i], v[:, :, i + half]
        out[:, :, i] = u * c - w * s
        out[:, :, i + half] = w * c + u * s
    return out


# ---- which keys a query sees ----------------------------------------------------------------------------
def sees(i: int, j: int, size: int) -> bool:
    """Chunks of ``size`` positions counted from the sequence's start: a query sees the keys of its own chunk
    up to itself."""
    return j <= i and i // size == j // size


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the bias table for a distance n >= 0: the first half of the rows one distance each, the second
    half logarithmic steps up to ``far``, the last row everything beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def softmax_rows(s: torch.Tensor) -> torch.Tensor:
    e = torch.exp(s - s.max(dim=-1, keepdim=True).values)
    return e / e.sum(dim=-1, keepdim=True)


# ---- attention inside chunks ---------------------------------------------------------------------------
def chunk_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, pos: torch.Tensor, scale: float, size: int,
                    bias: Optional[torch.Tensor] = None, far: float = 0.0,
                    talk: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv].  Query head h reads key/value head h // (H / G).
    ``bias`` [rows, H] is added to the scaled scores by distance; ``talk`` [H, H] then mixes the heads' scores."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    for i in range(T):
        pi = int(pos[i])
        js = [j for j in range(T) if sees(pi, int(pos[j]), size)]
        s = torch.stack([(k[js, h // (H // G)] @ q[i, h]) * scale for h in range(H)])      # [H, n]
        if bias is not None:
            rows = torch.tensor([distance_bucket(pi - int(pos[j]), bias.shape[0], far) for j in js])
            s = s + bias[rows].t().to(q.dtype)
        if talk is not None:
            s = talk.to(q.dtype) @ s
        p = softmax_rows(s)
        for h in range(H):
            out[i, h] = p[h] @ v[js, h // (H // G)]
    return out


def attention_mixer(h: torch.Tensor, pos: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float,
                    shared: dict) -> torch.Tensor:
    """The mixer 'attention'.  ``shared`` carries the first blending layer's values to the later ones."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    f = lambda name: w[pre + name].to(h.dtype)
    q = h @ f("q").t() + f("q.b")
    k = h @ f("k").t() + f("k.b")
    v = h @ f("v").t() + f("v.b")
    q = rms_norm(q, f("q.norm"), eps).view(T, H, D)       # over the whole projection
    k = rms_norm(k, f("k.norm"), eps).view(T, G, D)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q = rotate_half_split(q, pos, rot["base"], rot["dims"])
        k = rotate_half_split(k, pos, rot["base"], rot["dims"])
    v = rms(v.view(T, G, Dv), eps)
    if m.get("v_mix"):
        if "v_first" not in shared:
            shared["v_first"] = v
        else:
            lam = f("vmix")
            v = (1.0 - lam) * v + lam * shared["v_first"]
    o = chunk_attention(q, k, v, pos, m["scale"], m["mask"]["size"])
    return o.reshape(T, H * Dv) @ f("o").t() + f("o.b")


def biased_attention_mixer(h: torch.Tensor, pos: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict,
                           eps: float) -> torch.Tensor:
    """The left half of the mixer 'parallel': the values are the projected keys, before their norm."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    f = lambda name: w[pre + name].to(h.dtype)
    q = (h @ f("q").t() + f("q.b")).view(T, H, D)
    k = (h @ f("k").t() + f("k.b")).view(T, G, D)
    v = k
    q = rms_norm(q, f("q.norm"), eps)                     # per head, one weight for all heads
    k = rms_norm(k, f("k.norm"), eps)
    o = chunk_attention(q, k, v, pos, m["scale"], m["mask"]["size"], bias=f("rel"), far=float(m["bias_max"]),
                        talk=f("talk"))
    return o.reshape(T, H * D) @ f("o").t() + f("o.b")


# ---- recurrences ---------------------------------------------------------------------------------------
def decayed_sum_state(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """S_t = decay * S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t, per head.  q, k [T, H, D], v [T, H, Dv], decay [H]."""
    T, H, D = q.shape
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    S = torch.zeros((H, D, v.shape[2]), dtype=q.dtype)
    for t in range(T):
        S = decay.view(H, 1, 1) * S + k[t].unsqueeze(2) * v[t].unsqueeze(1)
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def linear_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    """The right half of the mixer 'parallel'."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    f = lambda name: w[pre + name].to(h.dtype)
    q = silu(h @ f("q").t()).view(T, H, D)
    k = silu(h @ f("k").t()).view(T, H, D)
    v = silu(h @ f("v").t()).view(T, H, Dv)
    o = decayed_sum_state(q, k, v, torch.tensor(m["decay"], dtype=h.dtype))
    o = rms_norm(o.reshape(T, H * Dv), f("norm"), eps) * sigmoid(h @ f("g").t())
    return o @ f("o").t()


def bonus_state(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, wdec: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    """o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t, then S_t = diag(w_t) S_(t-1) + k_t v_t^T.  All [T, H, D], u [H, D]."""
    T, H, D = r.shape
    out = torch.zeros_like(v)
    S = torch.zeros((H, D, v.shape[2]), dtype=r.dtype)
    for t in range(T):
        kv = k[t].unsqueeze(2) * v[t].unsqueeze(1)
        out[t] = torch.einsum("hdv,hd->hv", S + u.unsqueeze(2) * kv, r[t])
        S = wdec[t].unsqueeze(2) * S + kv
    return out


def shifted_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    """The mixer 'wkv'."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    f = lambda name: w[pre + name].to(h.dtype)
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    blend = lambda s: h + (before - h) * f("mu." + s)
    r = (blend("r") @ f("r").t()).view(T, H, D)
    k = (blend("k") @ f("k").t()).view(T, H, D)
    v = (blend("v") @ f("v").t()).view(T, H, D)
    gate = silu(blend("g") @ f("g").t())
    wdec = torch.exp(-torch.exp(torch.tanh(blend("w") @ f("w1").t()) @ f("w2").t() + f("w0"))).view(T, H, D)
    o = bonus_state(r, k, v, wdec, f("u"))
    o = rms(o, eps).reshape(T, H * D) * f("norm") * gate
    return o @ f("o").t()


# ---- feed-forward ---------------------------------------------------------------------------------------
def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    return gelu_erf(h @ w[pre + "up"].to(h.dtype).t()) @ w[pre + "down"].to(h.dtype).t()


# ---- the model -------------------------------------------------------------------------------------------
def mixer(h, pos, w, pre, layer, eps, shared):
    kind, m = layer["type"], layer["mixer"]
    if kind == "attention":
        return attention_mixer(h, pos, w, pre, m, eps, shared)
    if kind == "wkv":
        return shifted_mixer(h, w, pre, m, eps)
    if kind == "parallel":
        left = biased_attention_mixer(h, pos, w, pre + "left.", m["left"], eps)
        right = linear_mixer(h, w, pre + "right.", m["right"], eps)
        return m["left_scale"] * left + m["right_scale"] * right
    raise ValueError(kind)


def forward(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its start.  ``layers_out``: the stream after every layer."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = tensors["embed"].to(dtype)[torch.tensor(tokens)]
    pos = torch.arange(len(tokens))
    shared: dict = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = rms_norm(alpha * x + mixer(x, pos, tensors, p + "mix.", layer, eps, shared), tensors[p + "norm1"].to(dtype), eps)
        if layer["mlp"] is not None:
            x = rms_norm(alpha * x + dense_ff(x, tensors, p + "mlp."), tensors[p + "norm2"].to(dtype), eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_norm(x, tensors["final.norm"].to(dtype), eps)
    logits = x @ tensors["head"].to(dtype).t()
    cap = cfg["logit_softcap"]
    return cap * torch.tanh(logits / cap)
