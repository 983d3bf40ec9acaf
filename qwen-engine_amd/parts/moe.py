"""Feed-forwards of a post-norm decoder: a dense one with a polynomial activation normed per power, and
a routed mixture of small gated experts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Runtime, TensorInfo
from .registry import register_part


class PolyNormMLP:
    """down(a N(z) + b N(z^2) + c N(z^3) + e), z = up x, N(v) = v / sqrt(mean(v^2) + eps) per token.  The
    up product leaves z in 32-bit; the activation is formed in 32-bit and rounded once."""
    graph_safe = True

    def __init__(self, spec, hidden_size: int):
        self.hidden = int(hidden_size)
        self.inter = int(spec.intermediate_size)
        self.eps = float(spec.eps)
        self.w_up = self.w_down = self.coef = None

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        i = spec.intermediate_size
        return {"up": TensorInfo((i, hidden)), "down": TensorInfo((hidden, i)), "act": TensorInfo((4,), "ones", "vector")}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.w_up = rt.place_matrix(tensors["up"])
        self.w_down = rt.place_matrix(tensors["down"])
        self.coef = rt.place_vector(tensors["act"])

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        z = ops.gemm(x, self.w_up, out_dtype=torch.float32)
        a = ops.polynorm(z, self.coef, self.eps, ctx.rt.dtype)
        splits = ops.gemm_branch_splits(a, self.w_down)
        if splits:
            return ops.gemm(a, self.w_down, epilogue=ops.EPI_PARTIAL, splits=splits)
        return ops.gemm(a, self.w_down)


class GroupedMoE:
    """Router logits in 32-bit, softmax over all experts, the best groups of neighbouring experts, the
    largest scores among them (``ops.moe_route``); then the chosen experts' two products over the
    (token, choice) pairs grouped by expert on the device (``ops.moe_experts``).  The output is float32
    [top, T, H]: a token's weighted expert outputs in the order of its choices, which the norm that
    follows adds to the stream (or, with many rows, float32 [1, T, H]: already added up in that order)."""
    graph_safe = True

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.e, self.top, self.inter = int(spec.num_experts), int(spec.top), int(spec.intermediate_size)
        self.w_router = self.w_gate_up = self.w_down = None
        # gate and up rows in alternating blocks of 32 (what the tiled product's epilogue wants side by side)
        # where the experts' width allows; else gate rows, then up rows
        self.interleaved = self.inter % 32 == 0

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        f = spec.intermediate_size
        t = {"router": TensorInfo((spec.num_experts, hidden))}
        for e in range(spec.num_experts):
            t[f"e{e}.gate"] = TensorInfo((f, hidden))
            t[f"e{e}.up"] = TensorInfo((f, hidden))
            t[f"e{e}.down"] = TensorInfo((hidden, f))
        return t

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.w_router = rt.place_matrix(tensors["router"])
        first = tensors["e0.gate"]
        dt = torch.float32 if rt.dtype == torch.float32 or first.dtype == torch.float32 else torch.bfloat16
        self.w_gate_up = torch.empty((self.e, 2 * self.inter, self.hidden), dtype=dt, device=rt.device)
        self.w_down = torch.empty((self.e, self.hidden, self.inter), dtype=dt, device=rt.device)
        for e in range(self.e):           # an expert at a time: the host never holds more
            g, u = tensors[f"e{e}.gate"], tensors[f"e{e}.up"]
            self.w_gate_up[e].copy_(ops.interleave_gate_up(g, u) if self.interleaved else torch.cat([g, u], dim=0))
            self.w_down[e].copy_(tensors[f"e{e}.down"])

    def active_weight_bytes(self, tokens: int) -> int:
        """Bytes of expert weights that a step of ``tokens`` tokens reads at most."""
        per = (self.w_gate_up[0].numel() + self.w_down[0].numel()) * self.w_down.element_size()
        return min(self.e, tokens * self.top) * per + self.w_router.numel() * self.w_router.element_size()

    def output_parts(self, rows: int) -> int:
        """How many 32-bit parts forward leaves for ``rows`` rows where it can write them into a tensor it is given
        (``parts_out``); 0 where it cannot (many pairs: the sum is formed here)."""
        return self.top if rows * self.top < 1024 else 0

    def forward(self, x: torch.Tensor, ctx, parts_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        s = self.spec
        logits = ops.gemm(x, self.w_router, out_dtype=torch.float32)
        ids, weights = ops.moe_route(logits, s.num_groups, s.keep_groups, s.top)
        return ops.moe_experts(x, ids, weights, self.w_gate_up, self.w_down, s.limit, s.slope, interleaved=self.interleaved)


class BiasedMoE:
    """A mixture of squared-relu experts with identity experts (``BiasedMoESpec``): router logits in 32-bit, softmax
    over experts and identity experts together, the choice by score + correction, weights from the scores alone,
    renormalised and scaled (``ops.moe_route_biased``, or inside the one launch that a step of few tokens
    needs for routing, sort and identity rows); then the chosen experts' two products over the (token,
    choice) pairs grouped by expert on the device, a pair that chose an identity expert contributing its token's
    row itself (``ops.moe_experts``).  The output is float32 [top, T, H] or [1, T, H], as GroupedMoE's."""
    graph_safe = True
    rows_in_activation_type = False

    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.e, self.ident, self.top, self.inter = (int(spec.num_experts), int(spec.num_identity), int(spec.top),
                                                    int(spec.intermediate_size))
        self.w_router = self.correction = self.w_up = self.w_down = None

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        f, outs = spec.intermediate_size, spec.num_experts + spec.num_identity
        t = {"router": TensorInfo((outs, hidden)), "correction": TensorInfo((outs,), "zeros", "vector")}
        for e in range(spec.num_experts):
            t[f"e{e}.up"] = TensorInfo((f, hidden))
            t[f"e{e}.down"] = TensorInfo((hidden, f))
        return t

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.w_router = rt.place_matrix(tensors["router"])
        self.correction = rt.place_vector(tensors["correction"])
        first = tensors["e0.up"]
        dt = torch.float32 if rt.dtype == torch.float32 or first.dtype == torch.float32 else torch.bfloat16
        self.w_up = torch.empty((self.e, self.inter, self.hidden), dtype=dt, device=rt.device)
        self.w_down = torch.empty((self.e, self.hidden, self.inter), dtype=dt, device=rt.device)
        for e in range(self.e):           # an expert at a time: the host never holds more
            self.w_up[e].copy_(tensors[f"e{e}.up"])
            self.w_down[e].copy_(tensors[f"e{e}.down"])

    def active_weight_bytes(self, tokens: int) -> int:
        """Bytes of expert weights that a step of ``tokens`` tokens reads at most."""
        per = (self.w_up[0].numel() + self.w_down[0].numel()) * self.w_down.element_size()
        return min(self.e, tokens * self.top) * per + self.w_router.numel() * self.w_router.element_size()

    def output_parts(self, rows: int) -> int:
        """How many 32-bit parts forward leaves for ``rows`` rows where it can write them into a tensor it is given
        (``parts_out``); 0 where it cannot (many pairs: the sum is formed here)."""
        return self.top if rows * self.top < 1024 else 0

    def forward(self, x: torch.Tensor, ctx, parts_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        s = self.spec
        # Many rows against the router's few: the product the other way round, logits^T = W_router x^T, is a product of
        # few rows against a large matrix, which fills the chip where the router's few outputs give a handful of tiles;
        # the logits are 32-bit sums of the same products either way.
        transposed = x.shape[0] > 64 and self.w_router.shape[0] <= 64
        logits = ops.gemm(self.w_router, x, out_dtype=torch.float32) if transposed else \
            ops.gemm(x, self.w_router, out_dtype=torch.float32)
        # (rows_in_activation_type: the experts' output rows of a long portion in bfloat16 instead of 32-bit before
        # they are weighed and added in 32-bit: 7 % less time for the down product and 18 % for the sum at 8192
        # pairs of width 2048, for one more rounding of every expert's output; off)
        rows = ctx.rt.dtype if self.rows_in_activation_type else torch.float32
        return ops.moe_experts(x, None, None, self.w_up, self.w_down, act="relu_sq", identity=self.ident, rows_dtype=rows,
                               biased_route=(logits, self.correction, s.top, s.route_scale, transposed), parts_out=parts_out)


class TopSoftmaxMoE:
    """A mixture of plain gated experts (``TopSoftmaxMoESpec``): router logits in 32-bit, a bias added to them, the
    largest ``top`` chosen and weighed by the softmax over those alone (``ops.moe_route_biased`` without a correction,
    or inside the one launch that a step of few tokens needs for routing and sort); then the chosen experts' two
    products over the (token, choice) pairs grouped by expert on the device (``ops.moe_experts``).  A shared expert is
    a dense gated feed-forward of its own that every token uses; its output is one more 32-bit part, or is added to
    the sum, weighed by sigmoid of one number a token (``ops.moe_row_gate``).  The router's rows and the shared
    expert's gate row are one matrix, so one product gives the logits of both.
    The output is float32 [top (+ 1), T, H] or [1, T, H], as GroupedMoE's."""
    graph_safe = True

    def __init__(self, spec, hidden_size: int):
        from .mlp import SwiGLU
        from ..config.spec import SwiGLUSpec
        self.spec = spec
        self.hidden = int(hidden_size)
        self.e, self.top, self.inter = int(spec.num_experts), int(spec.top), int(spec.intermediate_size)
        self.interleaved = self.inter % 32 == 0
        self.shared = None
        if spec.shared_intermediate_size:
            self.shared = SwiGLU(SwiGLUSpec(intermediate_size=int(spec.shared_intermediate_size), names=("gate", "up", "down")),
                                 hidden_size)
        self.shared_gate = bool(spec.shared_gate) and self.shared is not None
        self.w_router = self.router_bias = self.w_gate_up = self.w_down = None

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        f = spec.intermediate_size
        t = {"router": TensorInfo((spec.num_experts, hidden))}
        if spec.router_bias:
            t["router.b"] = TensorInfo((spec.num_experts,), "zeros", "vector")
        for e in range(spec.num_experts):
            t[f"e{e}.gate"] = TensorInfo((f, hidden))
            t[f"e{e}.up"] = TensorInfo((f, hidden))
            t[f"e{e}.down"] = TensorInfo((hidden, f))
        if spec.shared_intermediate_size:
            s = int(spec.shared_intermediate_size)
            t["shared.gate"] = TensorInfo((s, hidden))
            t["shared.up"] = TensorInfo((s, hidden))
            t["shared.down"] = TensorInfo((hidden, s))
            if spec.shared_gate:
                t["shared.sg"] = TensorInfo((1, hidden))
        return t

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        router = tensors["router"]
        if self.shared_gate:              # (the gate's row behind the router's: one product for both)
            sg = tensors["shared.sg"]
            if sg.dtype != router.dtype:
                router, sg = router.float(), sg.float()
            router = torch.cat([router, sg.view(1, self.hidden)], dim=0)
        self.w_router = rt.place_matrix(router)
        if self.spec.router_bias:
            self.router_bias = rt.place_vector(tensors["router.b"])
        first = tensors["e0.gate"]
        dt = torch.float32 if rt.dtype == torch.float32 or first.dtype == torch.float32 else torch.bfloat16
        self.w_gate_up = torch.empty((self.e, 2 * self.inter, self.hidden), dtype=dt, device=rt.device)
        self.w_down = torch.empty((self.e, self.hidden, self.inter), dtype=dt, device=rt.device)
        for e in range(self.e):           # an expert at a time: the host never holds more
            g, u = tensors[f"e{e}.gate"], tensors[f"e{e}.up"]
            self.w_gate_up[e].copy_(ops.interleave_gate_up(g, u) if self.interleaved else torch.cat([g, u], dim=0))
            self.w_down[e].copy_(tensors[f"e{e}.down"])
        if self.shared is not None:
            self.shared.load({n: tensors["shared." + n] for n in ("gate", "up", "down")}, rt)

    def active_weight_bytes(self, tokens: int) -> int:
        """Bytes of expert weights that a step of ``tokens`` tokens reads at most."""
        per = (self.w_gate_up[0].numel() + self.w_down[0].numel()) * self.w_down.element_size()
        total = min(self.e, tokens * self.top) * per + self.w_router.numel() * self.w_router.element_size()
        if self.shared is not None:
            total += (self.shared.w_gu.numel() + self.shared.w_down.numel()) * self.shared.w_down.element_size()
        return total

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        T = x.shape[0]
        outputs = self.w_router.shape[0]
        # (many rows against the router's few: the product the other way round fills the chip, see BiasedMoE)
        transposed = T > 64 and outputs <= 64
        logits = ops.gemm(self.w_router, x, out_dtype=torch.float32) if transposed else \
            ops.gemm(x, self.w_router, out_dtype=torch.float32)
        route = (logits, None, self.top, 1.0, transposed, self.router_bias, self.e)
        if self.shared is None:
            return ops.moe_experts(x, None, None, self.w_gate_up, self.w_down, interleaved=self.interleaved, biased_route=route)
        few = T * self.top < 1024          # (the paths of ops.moe_experts that leave a part per choice)
        parts = torch.empty((self.top + 1, T, self.hidden), dtype=torch.float32, device=x.device) if few else None
        out = ops.moe_experts(x, None, None, self.w_gate_up, self.w_down, interleaved=self.interleaved, biased_route=route,
                              parts_out=parts[:self.top] if few else None)
        a = self.shared.activation(x)
        if not self.shared_gate:
            if few:
                ops.gemm(a, self.shared.w_down, out_dtype=torch.float32, out=parts[self.top])
                return parts
            ops.residual_add(out[0], ops.gemm(a, self.shared.w_down, out_dtype=torch.float32))
            return out
        gate = logits[self.e] if transposed else logits[:, self.e]
        if few:
            y = ops.gemm(a, self.shared.w_down, out_dtype=torch.float32, out=parts[self.top])
            ops.moe_row_gate(y, y, gate, accumulate=False)
            return parts
        ops.moe_row_gate(out[0], ops.gemm(a, self.shared.w_down), gate, accumulate=True)
        return out


register_part("polynorm_mlp", PolyNormMLP)
register_part("top_softmax_moe", TopSoftmaxMoE)
register_part("biased_moe", BiasedMoE)
register_part("grouped_moe", GroupedMoE)
