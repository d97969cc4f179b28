"""A sublayer whose input depends on the token's id: ``W_proj (act(W_gate x) * e)`` with ``e`` the
layer's columns of the token's row of a table that the model holds once for all layers
(``step.tables[name]``).  The gate's product has 32-bit sums, the activation is 32-bit; the gated
row is rounded to the compute type for the second product."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import TokenSideSpec
from ..errors import ConfigError
from .base import BuildContext, FeedForward, ParamSpec
from .registry import register_feed_forward
from .residual import stream


class TokenSide(FeedForward):
    adds_only = True
    prompt_graph_safe = True

    def __init__(self, spec: TokenSideSpec, ctx: BuildContext):
        if spec.activation not in ops.SIDE_ACTIVATIONS:
            raise ConfigError(f"unknown activation {spec.activation!r}; known: {sorted(ops.SIDE_ACTIVATIONS)}")
        if spec.dim <= 0 or spec.column0 < 0:
            raise ConfigError("a token-side input needs a positive width and a first column")
        self.spec = spec
        self.dtype = ctx.dtype
        self.w_gate: Optional[torch.Tensor] = None
        self.w_proj: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        return {"gate_proj.weight": ParamSpec((s.dim, s.hidden)), "out_proj.weight": ParamSpec((s.hidden, s.dim))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_gate, self.w_proj = tensors["gate_proj.weight"], tensors["out_proj.weight"]

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * self.spec.dim * (4 + size)

    def forward(self, step, xn, x_accum) -> None:
        s = self.spec
        table = getattr(step, "tables", {}).get(s.table)
        if table is None:
            raise ConfigError(f"the model holds no table {s.table!r} for a token-side input")
        if table.shape[1] < s.column0 + s.dim:
            raise ConfigError(f"table {s.table!r} has {table.shape[1]} columns, the layer reads up to {s.column0 + s.dim}")
        ws = step.workspace
        g = ws.get("side.gate", (step.n_tokens, s.dim), torch.float32)
        ops.gemm(xn, self.w_gate, g, workspace=ws.scratch())
        ge = ws.get("side.gated", (step.n_tokens, s.dim), self.dtype)
        ops.token_side_gate(g, table, step.token_ids, s.column0, ge, s.activation)
        stream(step).add_product(ge, self.w_proj, x_accum)


register_feed_forward("token_side", TokenSide)
