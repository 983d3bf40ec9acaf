"""A pre-norm residual block: x += mixer(norm(x)); x += ffn(norm(x))
(src/models/qwen3/model.py:278-298).  The residual stream is kept in 32-bit and each
residual sum is fused into the norm that follows it, so the block hands its last
branch output on as ``pending`` instead of adding it itself."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import CacheBinding, Runtime, Stream, StreamInput, TensorInfo, join_name, named_tensors, sub_tensors
from ..kernels import ops
from .registry import build_part, part_class, register_part

def _names(spec):
    """Checkpoint names of the four parts inside the layer's prefix (LayerSpec.part_names)."""
    return spec.part_names


class PreNormBlock:
    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.mixer_norm = build_part(spec.mixer_norm, hidden_size)
        self.mixer = build_part(spec.mixer, hidden_size)
        # (a layer without a feed-forward is its mixer alone; its second norm then has nothing to stand before)
        self.ffn = build_part(spec.ffn, hidden_size) if spec.ffn is not None else None
        self.ffn_norm = build_part(spec.ffn_norm, hidden_size) if self.ffn is not None else None

    @property
    def graph_safe(self) -> bool:
        """False if any part of the block says that its forward cannot be recorded into a graph."""
        return all(getattr(p, "graph_safe", True) for p in self.parts())

    @property
    def graph_safe_with_state(self) -> bool:
        """A part with per-request state is recorded into graphs only if it says itself that it can be."""
        return getattr(self.mixer, "graph_safe", False) is True

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None)

    @staticmethod
    def _named(spec):
        """(checkpoint name, part spec) of the block's parts."""
        out = [(_names(spec)[0], spec.mixer_norm), (_names(spec)[1], spec.mixer)]
        if spec.ffn is not None:
            out += [(_names(spec)[2], spec.ffn_norm), (_names(spec)[3], spec.ffn)]
        return out

    @staticmethod
    def cache_needs(spec, hidden: int):
        """What the block's parts keep per request, one (keys and values, fixed-size state) per cache
        user, in the order in which forward gets their bindings: this block has one, its mixer."""
        cls = part_class(spec.mixer.kind)
        kv = cls.cache_need(spec.mixer) if hasattr(cls, "cache_need") else None
        state = cls.state_need(spec.mixer, hidden) if hasattr(cls, "state_need") else None
        return [(kv, state)]

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        out: Dict[str, TensorInfo] = {}
        for name, sub in PreNormBlock._named(spec):
            for rel, info in part_class(sub.kind).expected_tensors(sub, hidden).items():
                out[join_name(name, rel)] = info
        return out

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        for (name, sub), part in zip(self._named(self.spec), self.parts()):
            names = type(part).expected_tensors(sub, self.hidden)
            if "" in names:        # (a part that is one tensor, which carries the part's own name)
                part.load(named_tensors(tensors, name, names), rt)
            else:
                part.load(sub_tensors(tensors, name + "."), rt)

    def forward(self, h, pending: Optional[torch.Tensor], ctx, bindings) -> torch.Tensor:
        """h: the 32-bit residual stream, a tensor (updated in place) or a Stream (whose buffers may
        change places).  pending: branch output not yet added to the stream, or None.  bindings: one
        CacheBinding per cache user of the block (cache_needs), here the mixer's.  Returns the
        feed-forward output, to be added by whoever norms next.  A branch output is [T, H] in the
        activation type, or float32 [S, T, H]: partial products that the norm adds in the order of S."""
        stream = h if isinstance(h, Stream) else Stream(h)
        x = self._input(self.mixer_norm, self.mixer, stream, pending, ctx)
        a = self.mixer.forward(x, ctx, bindings[0])
        if self.ffn is None:
            return a
        x = self._input(self.ffn_norm, self.ffn, stream, a, ctx)
        return self.ffn.forward(x, ctx)

    @staticmethod
    def _input(norm, part, stream: Stream, delta, ctx):
        """The part's input: the normed rows, or, with few rows (the model then gave the stream a second
        buffer) and where both the norm and the part can do it, the stream, what is to be added, and
        the norm, for the part's first product."""
        if (getattr(part, "takes_stream", False) and hasattr(norm, "fusable_weight") and
                stream.spare is not None):
            fw = norm.fusable_weight()
            si = StreamInput(stream, delta, norm, fw[0], fw[1], ctx.rt) if fw is not None else None
            if si is not None and si.fusable():
                return si
        return norm.forward(stream.h, ctx.rt, delta=delta)


class PostNormBlock:
    """x <- mixer_norm(alpha x + mixer(conv(x))); x <- ffn_norm(alpha x + ffn(x)).  The stream x stays
    32-bit and normed; each norm forms the sum, norms it in place and hands the next part a copy in the
    activation type.  The convolution in front of the mixer keeps a request's last inputs in the block's
    state slot; the mixer keeps its cache: one cache user with both."""

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.alpha = float(spec.alpha)
        self.mixer_norm = build_part(spec.mixer_norm, hidden_size)
        self.mixer = build_part(spec.mixer, hidden_size)
        self.ffn = build_part(spec.ffn, hidden_size) if spec.ffn is not None else None
        # without a feed-forward the second norm is there only if the folder holds its tensor
        self.ffn_norm = build_part(spec.ffn_norm or spec.mixer_norm, hidden_size)
        self.has_ffn_norm = spec.ffn is not None
        self.conv = build_part(spec.conv, hidden_size) if spec.conv is not None else None

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.conv) if p is not None)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", True) for p in self.parts())

    @property
    def graph_safe_with_state(self) -> bool:
        return all(getattr(p, "graph_safe", False) is True for p in (self.mixer, self.conv) if p is not None)

    # the stream's copy in the activation type that the block's last norm made, for the block after it
    _COPY = "postnorm_block.copy"

    @staticmethod
    def _named(spec):
        """(checkpoint name, part spec, optional) of the block's parts."""
        n_norm1, n_mix, n_norm2, n_ffn, n_conv = spec.names
        out = [(n_norm1, spec.mixer_norm, False), (n_mix, spec.mixer, False)]
        if spec.ffn is not None:
            out += [(n_norm2, spec.ffn_norm or spec.mixer_norm, False), (n_ffn, spec.ffn, False)]
        else:
            out += [(n_norm2, spec.ffn_norm or spec.mixer_norm, True)]
        if spec.conv is not None:
            out.append((n_conv, spec.conv, False))
        return out

    @staticmethod
    def cache_needs(spec, hidden: int):
        cls = part_class(spec.mixer.kind)
        kv = cls.cache_need(spec.mixer) if hasattr(cls, "cache_need") else None
        state = part_class(spec.conv.kind).state_need(spec.conv, hidden) if spec.conv is not None else None
        mixer_state = cls.state_need(spec.mixer, hidden) if hasattr(cls, "state_need") else None
        if mixer_state is not None and state is not None:
            raise ValueError("a post-norm block's state slot belongs to its convolution: the mixer cannot ask for one too")
        return [(kv, state if state is not None else mixer_state)]

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        out: Dict[str, TensorInfo] = {}
        for name, sub, optional in PostNormBlock._named(spec):
            for rel, info in part_class(sub.kind).expected_tensors(sub, hidden).items():
                out[join_name(name, rel)] = info._replace(optional=True) if optional else info
        return out

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        n_norm1, n_mix, n_norm2, n_ffn, n_conv = self.spec.names
        for name, part in ((n_norm1, self.mixer_norm), (n_mix, self.mixer), (n_norm2, self.ffn_norm),
                           (n_ffn, self.ffn), (n_conv, self.conv)):
            if part is None:
                continue
            names = type(part).expected_tensors(self._spec_of(part), self.hidden)
            held = named_tensors(tensors, name, names)
            if part is self.ffn_norm and self.ffn is None:
                self.has_ffn_norm = len(held) == len(names)
                if not self.has_ffn_norm:
                    continue
            part.load(held, rt)

    def _spec_of(self, part):
        s = self.spec
        return {id(self.mixer_norm): s.mixer_norm, id(self.mixer): s.mixer, id(self.ffn_norm): s.ffn_norm or s.mixer_norm,
                id(self.ffn): s.ffn, id(self.conv): s.conv}[id(part)]

    def forward(self, h, pending: Optional[torch.Tensor], ctx, bindings):
        """h: the 32-bit stream (a tensor, or a Stream).  pending: a branch output that a block of another
        kind before this one left to be added.  Returns None: nothing is left to add."""
        x = h.h if isinstance(h, Stream) else h
        rt = ctx.rt
        if pending is not None:
            ops.residual_add(x, pending)
        binding = bindings[0]
        kept = ctx.memo.pop(self._COPY, None) if pending is None else None
        if self.conv is not None:
            xin = self.conv.forward(x, ctx, binding.state)
        elif rt.dtype == torch.float32:
            xin = x
        elif kept is not None and kept[0] is x:
            xin = kept[1]              # (the norm of the block before left its copy: nothing is converted again)
        else:
            xin = x.to(rt.dtype)
        y = self.mixer.forward(xin, ctx, binding)
        xa = self.mixer_norm.after_sum(x, y, self.alpha, rt)
        if self.ffn is not None:
            y = self.ffn.forward(x if xa is None else xa, ctx)
            xa = self.ffn_norm.after_sum(x, y, self.alpha, rt)
        elif self.has_ffn_norm:
            xa = self.ffn_norm.after_sum(x, None, self.alpha, rt)
        if xa is not None:
            ctx.memo[self._COPY] = (x, xa)
        return None


class ParallelBlock:
    """n = norm(x); x <- x + (mixer(n) + ffn(n)): one norm, whose output both branches read, and one residual
    sum in 32-bit.  The norm also adds what the block before left to be added (fused, as in PreNormBlock); the
    mixer's output is added to the stream here, the feed-forward's is handed on for the next norm to add."""

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.norm = build_part(spec.norm, hidden_size)
        self.mixer = build_part(spec.mixer, hidden_size)
        self.ffn = build_part(spec.ffn, hidden_size) if spec.ffn is not None else None

    def parts(self):
        return tuple(p for p in (self.norm, self.mixer, self.ffn) if p is not None)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", True) for p in self.parts())

    @property
    def graph_safe_with_state(self) -> bool:
        return getattr(self.mixer, "graph_safe", False) is True

    @staticmethod
    def _named(spec):
        n_norm, n_mix, n_ffn = spec.names
        out = [(n_norm, spec.norm), (n_mix, spec.mixer)]
        if spec.ffn is not None:
            out.append((n_ffn, spec.ffn))
        return out

    @staticmethod
    def cache_needs(spec, hidden: int):
        cls = part_class(spec.mixer.kind)
        kv = cls.cache_need(spec.mixer) if hasattr(cls, "cache_need") else None
        state = cls.state_need(spec.mixer, hidden) if hasattr(cls, "state_need") else None
        return [(kv, state)]

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        out: Dict[str, TensorInfo] = {}
        for name, sub in ParallelBlock._named(spec):
            for rel, info in part_class(sub.kind).expected_tensors(sub, hidden).items():
                out[join_name(name, rel)] = info
        return out

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        for (name, sub), part in zip(self._named(self.spec), self.parts()):
            names = type(part).expected_tensors(sub, self.hidden)
            part.load(named_tensors(tensors, name, names), rt)

    def forward(self, h, pending: Optional[torch.Tensor], ctx, bindings):
        stream = h if isinstance(h, Stream) else Stream(h)
        n = self.norm.forward(stream.h, ctx.rt, delta=pending)
        T = n.shape[0]
        if self.ffn is not None and stream.spare is not None and hasattr(self.mixer, "output_parts") and \
                hasattr(self.ffn, "output_parts"):
            # few rows: both branches leave 32-bit parts, side by side in one tensor, which the next norm adds in order
            sa, sf = self.mixer.output_parts(T, ctx.rt.dtype), self.ffn.output_parts(T)
            if sa > 0 and sf > 0:
                parts = torch.empty((sa + sf, T, self.hidden), dtype=torch.float32, device=n.device)
                self.mixer.forward(n, ctx, bindings[0], parts_out=parts[:sa])
                self.ffn.forward(n, ctx, parts_out=parts[sa:])
                return parts
        if self.ffn is not None and hasattr(self.mixer, "output_parts"):
            # (the mixer's last product adds into the stream itself where it can: the feed-forward reads n, not the stream)
            a = self.mixer.forward(n, ctx, bindings[0], add_to=stream.h)
        else:
            a = self.mixer.forward(n, ctx, bindings[0])
        if self.ffn is None:
            return a
        y = self.ffn.forward(n, ctx)
        if a is None:
            return y
        ops.residual_add(stream.h, a)
        return y


register_part("prenorm_block", PreNormBlock)
register_part("parallel_block", ParallelBlock)
register_part("postnorm_block", PostNormBlock)
