"""A mixer whose state per head is a matrix: the matrix memory of xLSTM (mLSTM).

One product gives ``[q | k | v | gate | i | f]`` with 32-bit sums.  Per head, in 32-bit:
``i = cap tanh((i~ + b_i) / cap)``, ``f = logsigmoid(cap tanh((f~ + b_f) / cap))``, ``m' = max(f + m, i)``,
``S <- exp(f + m - m') S + exp(i - m') k v^T``, ``n`` likewise with ``k`` alone, and the head's output is
``S^T q / (max(|n . q|, exp(-m')) + floor)`` with ``q`` scaled by ``head_dim^(-1/2)``.  Every head's output
is divided by its root mean square, the heads side by side are multiplied by a gain and by
``sigmoid(gate)``, rounded to the compute type and projected back.  The cache holds, per sequence and
all zero at its start, ``S`` (stored column by column, ``[heads, v_head_dim, head_dim]``) and, once per
block of the kernel that walks the tokens, ``n`` and ``m``.  A prompt step and a step of one token
run the same kernel, the same arithmetic per token.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import MatrixMemorySpec
from ..errors import ConfigError
from .base import BuildContext, CompositeRequest, Mixer, ParamSpec, StateRequest
from .registry import register_mixer
from .residual import stream


class MatrixMemory(Mixer):
    adds_only = True
    prompt_graph_safe = True
    kernel_families = ("recurrent",)

    def __init__(self, spec: MatrixMemorySpec, ctx: BuildContext):
        if spec.head_dim > 256:
            raise ConfigError(f"a key size of {spec.head_dim} exceeds the 256 the matrix memory's kernel keeps in registers")
        if not spec.gate_cap > 0:
            raise ConfigError(f"the gates' cap must be positive, got {spec.gate_cap}")
        self.spec = spec
        self.dtype = ctx.dtype
        self.qk_dim = spec.n_heads * spec.head_dim
        self.v_dim = spec.n_heads * spec.v_head_dim
        # columns of the projection: q, k, v, the output gate, the two gates of the recurrence
        self.k_col = self.qk_dim
        self.v_col = 2 * self.qk_dim
        self.g_col = self.v_col + self.v_dim
        self.i_col = self.g_col + self.v_dim
        self.f_col = self.i_col + spec.n_heads
        self.proj_dim = self.f_col + spec.n_heads
        self.tiles = ops.mlstm_tiles(spec.v_head_dim)
        self.w_in: Optional[torch.Tensor] = None
        self.w_out: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        return {"q_proj.weight": ParamSpec((self.qk_dim, s.hidden)),
                "k_proj.weight": ParamSpec((self.qk_dim, s.hidden)),
                "v_proj.weight": ParamSpec((self.v_dim, s.hidden)),
                "g_proj.weight": ParamSpec((self.v_dim, s.hidden)),
                "i_proj.weight": ParamSpec((s.n_heads, s.hidden)),
                "f_proj.weight": ParamSpec((s.n_heads, s.hidden)),
                "i_proj.bias": ParamSpec((s.n_heads,), role="gain", init="normal"),
                "f_proj.bias": ParamSpec((s.n_heads,), role="gain", init="normal"),
                "norm.weight": ParamSpec((self.v_dim,), role="gain", init="gain"),
                "o_proj.weight": ParamSpec((s.hidden, self.v_dim))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = torch.cat([tensors[f"{p}_proj.weight"] for p in ("q", "k", "v", "g", "i", "f")], dim=0).contiguous()
        self.w_out = tensors["o_proj.weight"]
        self.i_bias, self.f_bias = tensors["i_proj.bias"], tensors["f_proj.bias"]
        self.norm_gain = tensors["norm.weight"]

    def cache_request(self) -> CompositeRequest:
        s = self.spec
        return CompositeRequest((StateRequest((s.n_heads, s.v_head_dim, s.head_dim)),
                                 StateRequest((s.n_heads, self.tiles, s.head_dim)),
                                 StateRequest((s.n_heads, self.tiles))))

    def flops(self, new_counts, starts) -> int:
        # the products with the weights; per token and head the state's update and its read
        s = self.spec
        return 2 * sum(new_counts) * (self.matrix_elements() + 2 * s.n_heads * s.head_dim * (s.v_head_dim + 1))

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * ((self.proj_dim + self.v_dim) * 4 + self.v_dim * size)

    def input_weight(self) -> Optional[torch.Tensor]:
        return self.w_in

    def adopt_input_weight(self, view: torch.Tensor) -> None:
        self.w_in = view

    def forward(self, step, xn, x_accum, cache, owns_cache: bool, projected=None) -> None:
        if not owns_cache:
            raise ConfigError("a recurrent layer cannot run on another layer's state")
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        s_state, n_state, m_state = cache.parts
        if projected is not None:        # the projection is columns c0 .. of a product shared with other mixers
            proj, c0 = projected
        else:
            proj, c0 = ws.get("memory.proj", (n, self.proj_dim), torch.float32), 0
            ops.gemm(xn, self.w_in, proj, workspace=ws.scratch())
        o = ws.get("memory.o", (n, self.v_dim), torch.float32)
        ops.mlstm_scan(proj, c0, c0 + self.k_col, c0 + self.v_col, c0 + self.i_col, c0 + self.f_col, self.i_bias, self.f_bias,
                       s.gate_cap, float(s.head_dim) ** -0.5, s.floor, s_state.state, n_state.state, m_state.state,
                       step.cu_seqlens, step.seq_slots, o, s.n_heads, s.head_dim, s.v_head_dim)
        gated = ws.get("memory.gated", (n, self.v_dim), self.dtype)
        ops.head_norm_gate(o, proj, c0 + self.g_col, self.norm_gain, gated, s.n_heads, s.eps)
        stream(step).add_product(gated, self.w_out, x_accum)


register_mixer("matrix_memory", MatrixMemory)
