"""Layer norm with a weight and a bias: ``y = (x - mean) / sqrt(var + eps) * gain + bias``, ``var`` the
mean of the squared deviations from the mean, all statistics 32-bit; reads the 32-bit residual
stream and writes the activation type."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import LayerNormSpec
from .base import BuildContext, Norm, ParamSpec
from .registry import register_norm


class LayerNorm(Norm):
    prompt_graph_safe = True
    centred = True            # the mean is taken off and a bias added: not of the root-mean-square kind

    def __init__(self, spec: LayerNormSpec, ctx: BuildContext):
        self.size = spec.size
        self.eps = float(spec.eps)
        self.gain: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), role="gain", init="gain"),
                "bias": ParamSpec((self.size,), role="gain", init="offset")}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gain, self.bias = tensors["weight"], tensors["bias"]

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        ops.layernorm(x, self.gain, self.bias, self.eps, out, rows)


register_norm("layernorm", LayerNorm)
