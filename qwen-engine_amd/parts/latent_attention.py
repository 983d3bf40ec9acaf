"""Attention over one cached latent per token.

Per token the cache holds c = norm(W_dkv x)[:R] (R = kv_rank) and one rotated key part of Dr numbers that
all heads share; a head's key is [Uk_h c | rotated part], its value Uv_h c.  The engine never expands keys
or values: with q'_h = Uk_h^T q_h the score of head h against token j is q'_h . c_j + q_rot_h . k_rot_j, one
dot product against the cached row, and the head's output is Uv_h (sum_j p_j c_j).  So the attention
kernel sees one key/value head of R + Dr numbers whose first R are also the value, read by all query heads,
and the two maps are products per head before and after it (``ops.gemm_heads``).

Queries come straight from the input (``q``), or through a normed latent of their own (``dq``, ``dq.norm``,
``uq``).  With ``output_gate`` the heads' outputs are multiplied by sigmoid(W_g x) before ``o``, a number per output
or (``gate_per_head``) per head.  A window, a learned sink per head (``sink``) and the pairing of the rotation
(neighbouring or half-split, by the kind of the position part) are parameters of the kernels.  A layer without a
latent of its own (``own_latent`` False) reads the cache of the schedule entry it is bound to.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.plan import KVNeed
from ..kernels import ops
from .base import CacheBinding, Runtime, TensorInfo
from .registry import build_part, register_part


class LatentAttention:
    graph_safe = True

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.h, self.dn, self.dr, self.dv = int(spec.num_heads), int(spec.head_dim), int(spec.rot_dim), int(spec.v_head_dim)
        self.r = int(spec.kv_rank)
        self.q_rank = int(spec.q_rank) if spec.q_rank else 0
        self.gated = bool(spec.output_gate)
        self.gate_per_head = bool(getattr(spec, "gate_per_head", False))
        self.window = int(spec.window) if getattr(spec, "window", None) else 0
        self.has_sink = bool(getattr(spec, "sink", False))
        self.own_latent = bool(getattr(spec, "own_latent", True))
        self.scale = float(spec.scale)
        self.eps = float(spec.norm_eps)
        self.position = build_part(spec.position, hidden_size) if spec.position is not None else None
        self.half_split = spec.position is not None and spec.position.kind == "rope_half_angles"
        self.sink = None
        self.w_q = self.w_dq = self.w_uq = self.q_norm = self.w_dkv = self.kv_norm = None
        self.w_uk_t = self.w_uv = self.w_g = self.w_o = None
        self._no_turn: Optional[torch.Tensor] = None

    # ---- what it needs --------------------------------------------------------------------------
    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        h, dq, dv, r = spec.num_heads, spec.head_dim + spec.rot_dim, spec.v_head_dim, spec.kv_rank
        t = {
            "uk": TensorInfo((h * spec.head_dim, r)),
            "uv": TensorInfo((h * dv, r)),
            "o": TensorInfo((hidden, h * dv)),
        }
        if getattr(spec, "own_latent", True):
            t["dkv"] = TensorInfo((r + spec.rot_dim, hidden))
            t["dkv.norm"] = TensorInfo((r,), "ones", "vector")
        if getattr(spec, "sink", False):
            t["sink"] = TensorInfo((h,), "zeros", "vector")
        if spec.q_rank:
            t["dq"] = TensorInfo((spec.q_rank, hidden))
            t["dq.norm"] = TensorInfo((spec.q_rank,), "ones", "vector")
            t["uq"] = TensorInfo((h * dq, spec.q_rank))
        else:
            t["q"] = TensorInfo((h * dq, hidden))
        if spec.output_gate:
            t["g"] = TensorInfo((h if getattr(spec, "gate_per_head", False) else h * dv, hidden))
        return t

    @staticmethod
    def cache_need(spec) -> Optional[KVNeed]:
        """One row of R + Dr numbers a token; with a window the cache keeps the window's keys, or ``keep_window``
        where later layers that read this cache look further back."""
        window = getattr(spec, "window", None)
        if window is not None and getattr(spec, "keep_window", None) is not None:
            window = max(int(window), int(spec.keep_window))
        return KVNeed(num_kv_heads=1, head_dim=spec.kv_rank + spec.rot_dim, window=window, planes=1)

    @staticmethod
    def state_need(spec, hidden: int):
        return None

    # ---- weights -----------------------------------------------------------------------------------
    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        if self.q_rank:
            self.w_dq = rt.place_matrix(tensors["dq"])
            self.q_norm = rt.place_vector(tensors["dq.norm"])
            self.w_uq = rt.place_matrix(tensors["uq"])
        else:
            self.w_q = rt.place_matrix(tensors["q"])
        if self.own_latent:
            self.w_dkv = rt.place_matrix(tensors["dkv"])
            self.kv_norm = rt.place_vector(tensors["dkv.norm"])
        if self.has_sink:
            self.sink = rt.place_vector(tensors["sink"])
        # the key map per head, transposed: q' = Uk_h^T q is then a product against [R, dn] rows
        uk = tensors["uk"].view(self.h, self.dn, self.r)
        self.w_uk_t = rt.place_matrix(uk.transpose(1, 2).contiguous()) if self.dn > 0 else None
        self.w_uv = rt.place_matrix(tensors["uv"].view(self.h, self.dv, self.r))
        if self.gated:
            self.w_g = rt.place_matrix(tensors["g"])
        self.w_o = rt.place_matrix(tensors["o"])
        if self.position is not None:
            self.position.load({}, rt)
        self._no_turn = torch.zeros(0, dtype=torch.float32, device=rt.device)

    # ---- one step ------------------------------------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        """x [T, H] in the activation type.  Returns the mixer's output [T, H], or float32 partial
        products [S, T, H] of it."""
        if binding.kv is None:
            raise RuntimeError("latent attention was given no cache")
        T, dt = x.shape[0], ctx.rt.dtype
        g, cache = binding.group, binding.kv
        inv_freq = self.position.inv_freq() if self.position is not None else self._no_turn
        # queries
        if self.q_rank:
            cq = ops.rmsnorm(ops.gemm(x, self.w_dq, out_dtype=torch.float32), self.q_norm, self.eps, dt)
            q = ops.gemm(cq, self.w_uq)
        else:
            q = ops.gemm(x, self.w_q)
        q = q.view(T, self.h, self.dn + self.dr)
        # the token's cache row (normed latent | rotated shared key part) and the rotated parts of the packed
        # queries [Uk^T q | rotated q], in one launch
        qp = torch.empty((T, self.h, self.r + self.dr), dtype=dt, device=x.device)
        if binding.write and not self.own_latent:
            raise RuntimeError("latent attention: a layer without a latent of its own has nothing to write into a cache")
        if binding.write:
            kv = ops.gemm(x, self.w_dkv, out_dtype=torch.float32)
            ops.latent_kv_store(kv, self.kv_norm, self.eps, ctx.positions, inv_freq, ctx.slots[g], cache, q, qp, self.dn,
                                half_split=self.half_split)
        else:
            ops.latent_q_rotate(q, ctx.positions, inv_freq, qp, self.dn, half_split=self.half_split)
        if self.dn > 0:
            ops.gemm_heads(q, self.w_uk_t, qp)
        else:
            qp[:, :, :self.r].zero_()
        o_lat = ops.latent_attention(qp, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g], self.r, self.scale,
                                     window=self.window, sink=self.sink)
        gate = ops.gemm(x, self.w_g) if self.gated else None
        o = torch.empty((T, self.h, self.dv), dtype=dt, device=x.device)
        ops.gemm_heads(o_lat, self.w_uv, o, gate)
        o = o.view(T, self.h * self.dv)
        splits = ops.gemm_branch_splits(o, self.w_o)
        if splits:
            return ops.gemm(o, self.w_o, epilogue=ops.EPI_PARTIAL, splits=splits)
        return ops.gemm(o, self.w_o)


register_part("latent_attention", LatentAttention)
