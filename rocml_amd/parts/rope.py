"""Rotary position encoding with NEOX pairing (rocml-kernels/kernels/rope.hip:18-33):
``f_i = theta^(-2i/rot_dim)``, angle ``pos * f_i``, pair ``(i, i + rot_dim/2)``.  The part
owns the frequencies and prepares one cos/sin table per step from the step's token
positions; every mixer with the same spec shares it.

With a ``stretch`` (factor ``s``, original length ``L``, ``fast``, ``slow``) the frequencies are slowed
down for contexts beyond ``L`` positions: ``d(t) = rot_dim ln(L / (2 pi t)) / (2 ln theta)``,
``lo = max(floor(d(fast)), 0)``, ``hi = min(ceil(d(slow)), rot_dim - 1)``,
``r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``, ``f_i <- f_i / s * r_i + f_i (1 - r_i)``, and every
cosine and sine is multiplied by ``0.1 ln(s) + 1``."""
from __future__ import annotations

import math

import torch

from .. import ops
from ..config.spec import RopeSpec
from ..errors import ConfigError
from .base import BuildContext, PositionEncoding
from .registry import register_position


class RopeNeox(PositionEncoding):
    prompt_graph_safe = True

    def __init__(self, spec: RopeSpec, ctx: BuildContext):
        if spec.rot_dim % 2 != 0 or not 0 < spec.rot_dim <= spec.head_dim:
            raise ConfigError(f"rotary width {spec.rot_dim} must be even and at most the head size {spec.head_dim}")
        self.spec = spec
        self.rot_dim = spec.rot_dim
        half = spec.rot_dim // 2
        inv = [float(spec.theta) ** (-2.0 * i / spec.rot_dim) for i in range(half)]
        self.magnitude = 1.0
        st = getattr(spec, "stretch", None)
        if st is not None:
            if not (st.factor > 0 and st.original > 0 and st.fast > 0 and st.slow > 0 and spec.theta > 1):
                raise ConfigError("a stretch of the rotation's frequencies needs positive constants and a base above 1")

            def place(turns: float) -> float:      # the (fractional) frequency index that turns so often over the original length
                return spec.rot_dim * math.log(st.original / (2.0 * math.pi * turns)) / (2.0 * math.log(spec.theta))
            lo = max(math.floor(place(st.fast)), 0)
            hi = min(math.ceil(place(st.slow)), spec.rot_dim - 1)
            for i in range(half):
                r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                inv[i] = inv[i] / st.factor * r + inv[i] * (1.0 - r)
            self.magnitude = 0.1 * math.log(st.factor) + 1.0
        self.inv_freq = torch.tensor(inv, dtype=torch.float64, device=ctx.device)

    def tables(self, step):
        key = ("rope", self.spec)
        hit = step.memo.get(key)
        if hit is None:
            half = self.rot_dim // 2
            cos = step.workspace.get(f"rope.cos.{id(self)}", (step.n_tokens, half), torch.float32)
            sin = step.workspace.get(f"rope.sin.{id(self)}", (step.n_tokens, half), torch.float32)
            ops.rope_table(step.token_pos, self.inv_freq, cos, sin, self.magnitude)
            hit = (cos, sin)
            step.memo[key] = hit
        return hit


register_position("rope_neox", RopeNeox)
