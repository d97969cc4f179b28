"""A feed-forward of many small gated feed-forwards (experts) of which each token uses a few.

The router's logits are a product with 32-bit sums, the scores (softmax over all experts), the
choice (the best experts, optionally only of the best groups of neighbouring experts) and the
weights (chosen scores over their sum) are 32-bit.  The step's (token, choice) pairs are sorted by
expert on the device, all experts' first two products and their activation run as one launch over
the sorted rows, the down products as a second, and the weighted sum of a token's experts is
32-bit, in the order of the choices.  Nothing is read back to the host, so a step can be recorded.

Other ways to score: ``sigmoid`` of every logit by itself, a learned correction that counts for the choice only,
groups scored by the sum of their two best.  A shared expert (a gated feed-forward of a size of its own that
every token uses) is added at the end, times ``sigmoid(W_sg h)``, one number per token.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import RoutedExpertsSpec
from ..errors import ConfigError
from .base import BuildContext, FeedForward, ParamSpec
from .registry import register_feed_forward
from .residual import stream


class RoutedExperts(FeedForward):
    adds_only = True
    prompt_graph_safe = True
    kernel_families = ("moe",)

    def __init__(self, spec: RoutedExpertsSpec, ctx: BuildContext):
        if spec.activation != "silu":
            raise ConfigError(f"the experts' activation {spec.activation!r} is not supported; known: silu")
        if not 1 <= spec.top <= min(spec.n_experts, 64):
            raise ConfigError(f"a token uses {spec.top} of {spec.n_experts} experts; at least 1 and at most 64")
        if spec.n_experts > 512:
            raise ConfigError(f"{spec.n_experts} experts exceed the 512 the routing kernel takes")
        if spec.groups is not None:
            count, keep = spec.groups
            if count <= 0 or spec.n_experts % count != 0 or not 1 <= keep <= count or spec.top > keep * (spec.n_experts // count):
                raise ConfigError(f"{spec.n_experts} experts in {count} groups of which {keep} are kept do not allow "
                                  f"{spec.top} choices")
        self.weighting = getattr(spec, "weighting", "softmax_all")
        if self.weighting not in ("softmax_all", "softmax_chosen", "sigmoid"):
            raise ConfigError(f"unknown weighting of the chosen experts {self.weighting!r}; known: softmax_all, softmax_chosen, sigmoid")
        self.correction = bool(getattr(spec, "correction", False))
        self.group_score = getattr(spec, "group_score", "max")
        if self.group_score not in ("max", "top2_sum"):
            raise ConfigError(f"unknown score of a group of experts {self.group_score!r}; known: max, top2_sum")
        self.shared = getattr(spec, "shared_intermediate", None)
        self.shared_gate = bool(getattr(spec, "shared_gate", False))
        if self.shared is None and self.shared_gate:
            raise ConfigError("a gate on the shared expert needs a shared expert")
        if self.weighting == "softmax_chosen" and spec.groups is not None:
            raise ConfigError("the softmax over the chosen logits alone goes without groups of experts")
        self.router_bias = bool(getattr(spec, "router_bias", False))
        self.spec = spec
        self.dtype = ctx.dtype
        self.w_router: Optional[torch.Tensor] = None
        self.b_router: Optional[torch.Tensor] = None
        self.c_router: Optional[torch.Tensor] = None
        self.w_shared_gate_up: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        specs = {"router.weight": ParamSpec((s.n_experts, s.hidden))}
        if self.router_bias:
            specs["router.bias"] = ParamSpec((s.n_experts,), role="gain", init="normal")
        for e in range(s.n_experts):
            specs[f"experts.{e}.gate_proj.weight"] = ParamSpec((s.intermediate, s.hidden))
            specs[f"experts.{e}.up_proj.weight"] = ParamSpec((s.intermediate, s.hidden))
            specs[f"experts.{e}.down_proj.weight"] = ParamSpec((s.hidden, s.intermediate))
        if self.correction:
            specs["correction"] = ParamSpec((s.n_experts,), role="gain", init="normal")
        if self.shared is not None:
            specs["shared.gate_proj.weight"] = ParamSpec((self.shared, s.hidden))
            specs["shared.up_proj.weight"] = ParamSpec((self.shared, s.hidden))
            specs["shared.down_proj.weight"] = ParamSpec((s.hidden, self.shared))
            if self.shared_gate:
                specs["shared.gate.weight"] = ParamSpec((1, s.hidden))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.spec.n_experts
        self.w_router = tensors["router.weight"]
        if self.router_bias:
            self.b_router = tensors["router.bias"]
        # one tensor per kind, expert after expert: a launch reaches every expert's matrix by a stride
        self.w_gate = torch.stack([tensors[f"experts.{e}.gate_proj.weight"] for e in range(n)]).contiguous()
        self.w_up = torch.stack([tensors[f"experts.{e}.up_proj.weight"] for e in range(n)]).contiguous()
        self.w_down = torch.stack([tensors[f"experts.{e}.down_proj.weight"] for e in range(n)]).contiguous()
        if self.correction:
            self.c_router = tensors["correction"]
        if self.shared is not None:
            # rows in (gate_j, up_j) pairs, as the dense gated feed-forward keeps them
            gate, up = tensors["shared.gate_proj.weight"], tensors["shared.up_proj.weight"]
            self.w_shared_gate_up = torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1]).contiguous()
            self.w_shared_down = tensors["shared.down_proj.weight"]
            if self.shared_gate:
                # the gate's logit rides in the router's product, as one more row
                self.w_router = torch.cat([self.w_router, tensors["shared.gate.weight"]], dim=0).contiguous()

    def matrix_elements(self) -> int:
        """What a token is multiplied with: the router and the experts it uses."""
        s = self.spec
        shared = 0 if self.shared is None else 3 * s.hidden * self.shared + (s.hidden if self.shared_gate else 0)
        return s.n_experts * s.hidden + s.top * 3 * s.hidden * s.intermediate + shared

    def activation_bytes(self, n_tokens: int) -> int:
        s = self.spec
        size = 2 if self.dtype == torch.bfloat16 else 4
        shared = 0 if self.shared is None else self.shared * (size + 8) + s.hidden * 4
        return n_tokens * ((s.n_experts + 1) * 8 + s.top * (s.intermediate * size + s.hidden * 4 + 16) + shared)

    def forward(self, step, xn, x_accum) -> None:
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        gate_logit = None
        if self.shared_gate:
            # router and shared gate in one product; the choice kernel reads rows of n_experts numbers
            both = ws.get("moe.logits_gate", (n, s.n_experts + 1), torch.float32)
            ops.gemm(xn, self.w_router, both, workspace=ws.scratch())
            logits, gate_logit = both[:, :s.n_experts], both[:, s.n_experts:]
        else:
            logits = ws.get("moe.logits", (n, s.n_experts), torch.float32)
            ops.gemm(xn, self.w_router, logits, workspace=ws.scratch())
        chosen = ws.get("moe.chosen", (n, s.top), torch.int32)
        weight = ws.get("moe.weight", (n, s.top), torch.float32)
        # The softmax over the chosen logits alone is the softmax over all of them divided by the chosen ones' sum
        # (the largest logit is among the chosen, so no term underflows that the other form keeps): the same kernel
        # with nothing under the sum.
        ops.moe_route(logits, s.top, s.groups, 0.0 if self.weighting == "softmax_chosen" else s.sum_eps, chosen, weight,
                      bias=self.b_router, sigmoid=self.weighting == "sigmoid", correction=self.c_router,
                      group_top2=self.group_score == "top2_sum")
        pairs = n * s.top
        plan = ops.moe_plan(chosen, s.n_experts, ws.get("moe.plan", (ops.moe_plan_words(pairs, s.n_experts),), torch.int32))
        h = ws.get("moe.h", (pairs, s.intermediate), self.dtype)
        ops.moe_gemm(xn, self.w_gate, h, plan, s.top, gather=True, w2=self.w_up)
        y = ws.get("moe.y", (pairs, s.hidden), torch.float32)
        ops.moe_gemm(h, self.w_down, y, plan, s.top, gather=False)
        accumulate = not stream(step).overwrite
        if accumulate:
            ws.flush_pending()        # the stream must be whole before this kernel adds to it
        ops.moe_combine(y, plan, weight, x_accum, accumulate=accumulate)
        if self.shared is not None:
            hs = ws.get("moe.shared_h", (n, self.shared), self.dtype)
            if self.dtype == torch.bfloat16 and s.hidden % 8 == 0:
                ops.gemm(xn, self.w_shared_gate_up, hs, workspace=ws.scratch(), epilogue="swiglu")
            else:
                gate_up = ws.get("moe.shared_gate_up", (n, 2 * self.shared), torch.float32)
                ops.gemm(xn, self.w_shared_gate_up, gate_up, workspace=ws.scratch())
                ops.swiglu(gate_up, hs, interleaved=True, activation="silu")
            if gate_logit is None:
                ops.gemm(hs, self.w_shared_down, x_accum, accumulate=True, workspace=ws.scratch())
            else:
                ys = ws.get("moe.shared_y", (n, s.hidden), torch.float32)
                ops.gemm(hs, self.w_shared_down, ys, workspace=ws.scratch())
                ops.row_gate_add(x_accum, ys, gate_logit)


register_feed_forward("routed_experts", RoutedExperts)
