"""A retention: linear attention with one fixed decay per head, without softmax or denominator.

One product gives ``[q | k | v | gate]`` with 32-bit sums.  q and k are rotated (the position
encoding's tables) and k is multiplied by ``head_dim^(-1/2)``, in place in that 32-bit buffer.  Per
head, in 32-bit, ``S <- decay_h S + k v^T`` and ``o = S^T q`` with the new state.  Every head's output
is divided by its root mean square, the heads side by side are multiplied by ``silu(gate)``, rounded
to the compute type and projected back.  The cache holds ``S`` per sequence, zero at its start
(stored column by column, ``[heads, v_head_dim, head_dim]``).  A prompt step and a step of one token
run the same kernel, the same arithmetic per token.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import RetentionSpec
from ..errors import ConfigError
from .base import BuildContext, Mixer, ParamSpec, StateRequest
from .registry import build_position, register_mixer
from .residual import stream

MAX_HEAD_DIM = 256      # key channels of a head that the recurrence kernel keeps in registers (16 per lane of a row of 16)


class Retention(Mixer):
    adds_only = True
    kernel_families = ("recurrent",)

    def __init__(self, spec: RetentionSpec, ctx: BuildContext):
        if len(spec.decay) != spec.n_heads:
            raise ConfigError(f"{len(spec.decay)} decays for {spec.n_heads} heads")
        if spec.head_dim > MAX_HEAD_DIM:
            raise ConfigError(f"a key size of {spec.head_dim} exceeds the {MAX_HEAD_DIM} the recurrence kernel keeps in registers")
        self.spec = spec
        self.dtype = ctx.dtype
        self.qk_dim = spec.n_heads * spec.head_dim
        self.v_dim = spec.n_heads * spec.v_head_dim
        self.k_col, self.v_col, self.g_col = self.qk_dim, 2 * self.qk_dim, 2 * self.qk_dim + self.v_dim
        self.proj_dim = self.g_col + self.v_dim
        self.position = build_position(spec.position, ctx) if spec.position is not None else None
        if self.position is not None and getattr(self.position, "pairing", "halves") != "halves":
            raise ConfigError("the retention's rotation pairs a head's halves")
        self.graph_safe = self.position is None or getattr(self.position, "graph_safe", True)
        self.prompt_graph_safe = self.graph_safe and (self.position is None or getattr(self.position, "prompt_graph_safe", False))
        self.decay: Optional[torch.Tensor] = None
        if torch.device(ctx.device).type != "meta":
            self.decay = torch.tensor(spec.decay, dtype=torch.float32, device=ctx.device)
        self.w_in: Optional[torch.Tensor] = None
        self.w_out: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        return {"q_proj.weight": ParamSpec((self.qk_dim, s.hidden)),
                "k_proj.weight": ParamSpec((self.qk_dim, s.hidden)),
                "v_proj.weight": ParamSpec((self.v_dim, s.hidden)),
                "g_proj.weight": ParamSpec((self.v_dim, s.hidden)),
                "o_proj.weight": ParamSpec((s.hidden, self.v_dim))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = torch.cat([tensors[f"{p}_proj.weight"] for p in ("q", "k", "v", "g")], dim=0).contiguous()
        self.w_out = tensors["o_proj.weight"]

    def cache_request(self) -> StateRequest:
        s = self.spec
        return StateRequest((s.n_heads, s.v_head_dim, s.head_dim))

    def flops(self, new_counts, starts) -> int:
        # the products with the weights; per token and head the state's update and its read
        s = self.spec
        return 2 * sum(new_counts) * (self.matrix_elements() + 2 * s.n_heads * s.head_dim * s.v_head_dim)

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * ((self.proj_dim + self.v_dim) * 4 + self.v_dim * size)

    def forward(self, step, xn, x_accum, cache, owns_cache: bool) -> None:
        if not owns_cache:
            raise ConfigError("a recurrent layer cannot run on another layer's state")
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        proj = ws.get("retention.proj", (n, self.proj_dim), torch.float32)
        ops.gemm(xn, self.w_in, proj, workspace=ws.scratch())
        cos = sin = None
        rot = 0
        if self.position is not None:
            cos, sin = self.position.tables(step)
            rot = self.position.rot_dim
        # q and k are neighbours in the projection: both rotated in one launch, in which the k heads are scaled too
        ops.rotate_rows(proj, 0, 2 * s.n_heads, s.head_dim, rot, cos, sin, 1.0, heads_first=s.n_heads,
                        scale_rest=float(s.head_dim) ** -0.5)
        o = ws.get("retention.o", (n, self.v_dim), torch.float32)
        ops.decay_scan(proj, 0, proj, self.k_col, proj, self.v_col, cache.state, step.cu_seqlens, step.seq_slots, o,
                       s.n_heads, s.head_dim, s.v_head_dim, head_decay=self.decay)
        gated = ws.get("retention.gated", (n, self.v_dim), self.dtype)
        ops.head_norm_gate(o, proj, self.g_col, None, gated, s.n_heads, s.eps, gate="silu")
        stream(step).add_product(gated, self.w_out, x_accum)


register_mixer("retention", Retention)
