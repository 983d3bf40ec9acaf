"""Mixers that carry a matrix per head from token to token instead of keys and values, and the mixer that runs
two mixers side by side.  A request's state lives in its state slot, in 32-bit, and is cleared when the request
starts; a portion cut anywhere continues where the last one ended."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.plan import StateNeed
from ..kernels import ops
from .base import CacheBinding, Runtime, TensorInfo, join_name, named_tensors
from .registry import build_part, part_class, register_part


def _single_rows(ctx, T: int) -> bool:
    """True if every request of the step brings exactly one token."""
    return len(ctx.seqs) == T and all(s.q_len == 1 for s in ctx.seqs)


# From this many rows of one request in a step, the recurrences take the step's rows chunk by chunk (the chunks in
# parallel) instead of row by row.
CHUNKED_FROM_ROWS = 64


def _chunks(ctx, head_dim: int):
    """The step's rows cut into chunks for the chunked recurrence, if a request brings many rows: built and sent to the
    device once per step and chunk length, shared by the layers.  None: row by row."""
    if max((s.q_len for s in ctx.seqs), default=0) < CHUNKED_FROM_ROWS:
        return None
    C = ops.recurrence_chunk_len(head_dim)
    key = ("recurrence.chunks", C)
    if key not in ctx.memo:
        ch, po = ops.recurrence_chunks([(s.q_start, s.q_len) for s in ctx.seqs], C)
        ctx.memo[key] = (ch.to(ctx.rt.device), po.to(ctx.rt.device))
    return ctx.memo[key]


class ShiftedDecayMixer:
    """``ShiftedDecaySpec``: five blends of each token with the token before it, projections r, k, v, a silu gate
    and a decay per key channel through a low rank, the recurrence with a bonus for the token itself, a norm per
    head, the gate, the output projection.  State: the request's last input row, then the heads' matrices."""
    graph_safe = True
    BLENDS = ("r", "k", "v", "g", "w")

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.h, self.d, self.rank = int(spec.num_heads), int(spec.head_dim), int(spec.decay_rank)
        self.eps = float(spec.norm_eps)
        self.mu = self.w_r = self.w_k = self.w_v = self.w_g = self.w_1 = self.w_2 = self.w_o = None
        self.w0 = self.u = self.norm = None

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        n = spec.num_heads * spec.head_dim
        t = {f"mu.{s}": TensorInfo((hidden,), "normal", "vector") for s in ShiftedDecayMixer.BLENDS}
        for name in ("r", "k", "v", "g"):
            t[name] = TensorInfo((n, hidden))
        t["w1"] = TensorInfo((int(spec.decay_rank), hidden))
        t["w2"] = TensorInfo((n, int(spec.decay_rank)))
        t["w0"] = TensorInfo((n,), "zeros", "vector")
        t["u"] = TensorInfo((spec.num_heads, spec.head_dim), "normal", "vector")
        t["norm"] = TensorInfo((n,), "ones", "vector")
        t["o"] = TensorInfo((hidden, n))
        return t

    @staticmethod
    def cache_need(spec):
        return None

    @staticmethod
    def state_need(spec, hidden: int) -> Optional[StateNeed]:
        return StateNeed(shape=(hidden + spec.num_heads * spec.head_dim * spec.head_dim,), dtype="float32")

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.mu = rt.place_vector(torch.stack([tensors[f"mu.{s}"].float() for s in self.BLENDS]))
        self.w_r, self.w_k, self.w_v, self.w_g = (rt.place_matrix(tensors[n]) for n in ("r", "k", "v", "g"))
        self.w_1, self.w_2, self.w_o = (rt.place_matrix(tensors[n]) for n in ("w1", "w2", "o"))
        self.w0 = rt.place_vector(tensors["w0"])
        self.u = rt.place_vector(tensors["u"].reshape(-1))
        self.norm = rt.place_vector(tensors["norm"])

    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        if binding.state is None:
            raise RuntimeError("the recurrence was given no state")
        T, W, st = x.shape[0], self.hidden, binding.state
        m = ops.token_shift(x, self.mu, st, ctx.tok_seq, single_rows=_single_rows(ctx, T))
        r, k, v, gate = (ops.gemm(m[i], w) for i, w in enumerate((self.w_r, self.w_k, self.w_v, self.w_g)))
        low = ops.unary(ops.gemm(m[4], self.w_1, out_dtype=torch.float32), ops.UNARY_TANH, out_dtype=ctx.rt.dtype)
        decay_x = ops.gemm(low, self.w_2, out_dtype=torch.float32)      # (exponentials of the decay: in the recurrence, 32-bit)
        o = ops.linear_recurrence(r, k, v, st[:, W:], ctx.tok_seq, self.h, decay_x=decay_x, decay_bias=self.w0,
                                  bonus=self.u, chunks=_chunks(ctx, self.d))
        y = ops.gated_norm(o.view(T, self.h * self.d), self.norm, self.eps, self.h, ctx.rt.dtype, gate=gate,
                           gate_act=ops.GATE_SILU)
        return ops.gemm(y, self.w_o, out_dtype=torch.float32)


class DecayedLinearMixer:
    """``DecayedLinearSpec``: one product for q | k | v | gate, the recurrence with one decay per head (silu on q, k
    and v as they are read), all heads normed together, the sigmoid gate, the output projection."""
    graph_safe = True

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.h, self.d, self.dv = int(spec.num_heads), int(spec.head_dim), int(spec.v_head_dim)
        if len(spec.decay) != self.h:
            raise ValueError(f"{len(spec.decay)} decays for {self.h} heads")
        self.eps = float(spec.norm_eps)
        self.w_in = self.w_o = self.norm = self.decay = None

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        nk, nv = spec.num_heads * spec.head_dim, spec.num_heads * spec.v_head_dim
        return {"q": TensorInfo((nk, hidden)), "k": TensorInfo((nk, hidden)), "v": TensorInfo((nv, hidden)),
                "g": TensorInfo((nv, hidden)), "o": TensorInfo((hidden, nv)), "norm": TensorInfo((nv,), "ones", "vector")}

    @staticmethod
    def cache_need(spec):
        return None

    @staticmethod
    def state_need(spec, hidden: int) -> Optional[StateNeed]:
        return StateNeed(shape=(spec.num_heads * spec.head_dim * spec.v_head_dim,), dtype="float32")

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        mats = [tensors[n] for n in ("q", "k", "v", "g")]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_in = rt.place_matrix(torch.cat(mats, dim=0))
        self.w_o = rt.place_matrix(tensors["o"])
        self.norm = rt.place_vector(tensors["norm"])
        self.decay = torch.tensor(list(self.spec.decay), dtype=torch.float64).to(torch.float32).to(rt.device)

    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        if binding.state is None:
            raise RuntimeError("the recurrence was given no state")
        T = x.shape[0]
        nk, nv = self.h * self.d, self.h * self.dv
        y = ops.gemm(x, self.w_in)
        o = ops.linear_recurrence(y[:, :nk], y[:, nk:2 * nk], y[:, 2 * nk:2 * nk + nv], binding.state, ctx.tok_seq,
                                  self.h, decay=self.decay, silu=True, chunks=_chunks(ctx, self.d))
        z = ops.gated_norm(o.view(T, nv), self.norm, self.eps, 1, ctx.rt.dtype, gate=y[:, 2 * nk + nv:],
                           gate_act=ops.GATE_SIGMOID)
        return ops.gemm(z, self.w_o, out_dtype=torch.float32)


class SideBySideMixer:
    """``SideBySideMixerSpec``: two mixers read the same rows; their outputs are added with weights, in 32-bit.  The
    two share the block's one cache binding: the keys and values of the one that has any, the state of the one that
    has any."""

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.left = build_part(spec.left, hidden_size)
        self.right = build_part(spec.right, hidden_size)
        self.left_scale, self.right_scale = float(spec.left_scale), float(spec.right_scale)

    @property
    def graph_safe(self):
        return getattr(self.left, "graph_safe", False) is True and getattr(self.right, "graph_safe", False) is True

    @staticmethod
    def _subs(spec):
        return list(zip(spec.names, (spec.left, spec.right)))

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        out: Dict[str, TensorInfo] = {}
        for name, sub in SideBySideMixer._subs(spec):
            for rel, info in part_class(sub.kind).expected_tensors(sub, hidden).items():
                out[join_name(name, rel)] = info
        return out

    @staticmethod
    def _one(spec, hidden, what: str):
        found = []
        for _, sub in SideBySideMixer._subs(spec):
            cls = part_class(sub.kind)
            if hasattr(cls, what):
                need = getattr(cls, what)(sub) if what == "cache_need" else getattr(cls, what)(sub, hidden)
                if need is not None:
                    found.append(need)
        if len(found) > 1:
            raise ValueError(f"two mixers side by side both ask for a {what.split('_')[0]}: one binding holds one")
        return found[0] if found else None

    @staticmethod
    def cache_need(spec):
        return SideBySideMixer._one(spec, 0, "cache_need")

    @staticmethod
    def state_need(spec, hidden: int):
        return SideBySideMixer._one(spec, hidden, "state_need")

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        for (name, sub), part in zip(self._subs(self.spec), (self.left, self.right)):
            names = type(part).expected_tensors(sub, self.hidden)
            part.load(named_tensors(tensors, name, names), rt)

    def forward(self, x: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        a = self.left.forward(x, ctx, binding)
        b = self.right.forward(x, ctx, binding)
        return ops.scaled_sum(a, self.left_scale, b, self.right_scale)


register_part("shifted_decay", ShiftedDecayMixer)
register_part("decayed_linear", DecayedLinearMixer)
register_part("side_by_side", SideBySideMixer)
