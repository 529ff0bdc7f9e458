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


register_part("polynorm_mlp", PolyNormMLP)
register_part("biased_moe", BiasedMoE)
register_part("grouped_moe", GroupedMoE)
