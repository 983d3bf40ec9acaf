"""Differential attention over the paged cache.

Every head has two softmax maps over the same values; its output is a1 - lambda a2, divided by its root mean square
and scaled.  The engine runs the two maps as two query heads against two key heads, so that the attention kernels of
``PagedAttention`` serve them as they are: with H heads in G groups, map m of head h = g (H / G) + j becomes query head
g (2 H / G) + m (H / G) + j and reads key/value head 2 g + m, which is what those kernels' grouping of query heads gives;
the value head of a group is projected once per map (the rows of its matrix stand twice in the stacked projection), so
that each map's key head finds its values beside it in the cache.  The rows of the q projection are put into that
order when the weights are loaded.  One product gives q | k | v | gate; one kernel norms every map of q and k, rotates
it and writes q and the cache; the attention kernels run over 2 H and 2 G heads; one kernel joins the maps, norms,
scales and gates; then the output projection.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.plan import KVNeed
from ..kernels import ops
from .attention import PagedAttention, common_head_dim
from .base import CacheBinding, Runtime, TensorInfo
from .registry import build_part, register_part


def differential_lambda(lq1: torch.Tensor, lk1: torch.Tensor, lq2: torch.Tensor, lk2: torch.Tensor, diff: float) -> float:
    """exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number for the layer, formed in 64-bit once."""
    d = lambda a, b: (a.to(torch.float64) * b.to(torch.float64)).sum()
    return float(torch.exp(d(lq1, lk1)) - torch.exp(d(lq2, lk2)) + diff)


class DiffAttention(PagedAttention):
    takes_stream = False
    graph_safe = True        # every launch's grid follows the rows alone

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.h, self.g = int(spec.num_heads), int(spec.num_kv_heads)
        if self.h % self.g:
            raise ValueError(f"{self.h} query heads are no multiple of {self.g} key/value heads")
        # what the attention kernels see: two heads per head
        self.hq, self.hkv = 2 * self.h, 2 * self.g
        self.dk, self.dv = int(spec.head_dim), int(spec.v_head_dim)
        self.d = common_head_dim(self.dk, self.dv)
        self.scale = float(spec.scale)
        self.diff = float(spec.diff)
        self.eps = float(spec.norm_eps)
        self.window = 0
        self.gated = bool(spec.output_gate)
        self.position = build_part(spec.position, hidden_size) if spec.position is not None else None
        self.w_qkvg = self.w_o = self.q_norm = self.k_norm = None
        self.lam = 0.0

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        nq, nk, nv, no, ng = spec.names
        h, g, d, dv = spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.v_head_dim
        t = {nq: TensorInfo((h * 2 * d, hidden)), nk: TensorInfo((g * 2 * d, hidden)), nv: TensorInfo((g * dv, hidden)),
             no: TensorInfo((hidden, h * dv))}
        if spec.qk_norm_eps is not None:
            t[nq + spec.norm_suffix] = TensorInfo((d,), "ones", "vector")
            t[nk + spec.norm_suffix] = TensorInfo((d,), "ones", "vector")
        for name in spec.lambda_names:
            t[name] = TensorInfo((d,), "normal", "vector")
        if spec.output_gate:
            t[ng] = TensorInfo((h, hidden))
        return t

    @staticmethod
    def cache_need(spec) -> Optional[KVNeed]:
        return KVNeed(num_kv_heads=2 * spec.num_kv_heads, head_dim=common_head_dim(spec.head_dim, spec.v_head_dim), window=None)

    @staticmethod
    def state_need(spec, hidden: int):
        return None

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        s = self.spec
        nq, nk, nv, no, ng = s.names
        h, g, d, dv, per = self.h, self.g, self.dk, self.dv, self.h // self.g
        # q rows [head][map][d] -> [group][map][head of the group][d]
        wq = tensors[nq].view(g, per, 2, d, self.hidden).permute(0, 2, 1, 3, 4).reshape(h * 2 * d, self.hidden)
        wv = tensors[nv].view(g, 1, dv, self.hidden).expand(g, 2, dv, self.hidden).reshape(g * 2 * dv, self.hidden)
        mats = [wq, tensors[nk], wv] + ([tensors[ng]] if self.gated else [])
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_qkvg = rt.place_matrix(torch.cat(mats, dim=0))
        if s.qk_norm_eps is not None:
            self.q_norm = rt.place_vector(tensors[nq + s.norm_suffix])
            self.k_norm = rt.place_vector(tensors[nk + s.norm_suffix])
        self.lam = differential_lambda(*(tensors[n] for n in s.lambda_names), self.diff)
        self.w_o = rt.place_matrix(tensors[no])
        if self.position is not None:
            self.position.load({}, rt)

    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        """x [T, H] in the activation type.  Returns the mixer's output [T, H], or float32 partial products of it."""
        if binding.kv is None:
            raise RuntimeError("attention was given no cache")
        s = self.spec
        T, g, cache = x.shape[0], binding.group, binding.kv
        rows = ops.gemm(x, self.w_qkvg)                    # q | k | v (once per map) | gate
        q = ops.qkv_norm_store(rows, self.hq, self.hkv, self.dk, self.dv, cache, ctx.slots[g] if binding.write else None,
                               qk_norm=ops.QK_NORM_HEAD if s.qk_norm_eps is not None else ops.QK_NORM_NONE,
                               q_weight=self.q_norm, k_weight=self.k_norm, qk_eps=float(s.qk_norm_eps or 0.0),
                               positions=ctx.positions,
                               inv_freq=self.position.inv_freq() if self.position is not None else None)
        ex = self._extras(ctx)
        a = ops.attention(q, cache, ctx.positions, ctx.tok_seq, ctx.block_tables[g], self.scale, 0,
                          dec_tokens=ex["dec_tokens"], max_dec_position=ex["max_dec_position"],
                          other_tokens=ex["other_tokens"],
                          other_tiles=self._other_tiles(ctx) if ex["other_tokens"] is not None else None,
                          max_other_keys=ex.get("max_other_keys", 0), other_keys_row=ex.get("other_keys_row"),
                          shared_keys=ctx.shared_keys)
        gate = rows[:, rows.shape[1] - self.h:] if self.gated else None
        o = ops.diff_heads(a, self.h, self.g, self.dv, self.lam, self.eps, 1.0 - self.diff, gate=gate)
        return self._project_out(o.view(T, self.h * self.dv))


register_part("diff_attention", DiffAttention)
