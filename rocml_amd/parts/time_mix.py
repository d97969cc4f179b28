"""A recurrence whose decay depends on the token, per head and key channel (the time mixing of RWKV-6).

With ``h'`` the previous token's input (the sequence's kept row; zeros before its first token), each of r, k, v, the
gate and the decay reads a mix of its own, ``h + (h' - h) mu``, formed in 32-bit and rounded to the compute type for
the products.  ``r``, ``k``, ``v`` and the gate come from four products into one 32-bit buffer; the decay is
``w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))`` (two small products with ``tanh`` between them; the offset and both
exponentials in 32-bit, inside the recurrence kernel).  Per head, in 32-bit, ``o = (S + diag(u) k v^T)^T r`` and then ``S <- diag(w) S + k v^T``.
Every head's output is divided by its root mean square, the heads side by side are multiplied by a gain and by
``silu(gate)``, rounded to the compute type and projected back.  The cache holds two things per sequence, both zero
at its start: ``S`` (stored column by column, ``[heads, head_dim, head_dim]``) and the previous token's input.  A
prompt step and a step of one token run the same kernels.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import TimeMixSpec
from ..errors import ConfigError
from .base import BuildContext, CompositeRequest, Mixer, ParamSpec, StateRequest
from .registry import register_mixer
from .residual import stream

MIXES = ("r", "k", "v", "g", "w")


class TimeMix(Mixer):
    adds_only = True
    prompt_graph_safe = True
    kernel_families = ("recurrent",)

    def __init__(self, spec: TimeMixSpec, ctx: BuildContext):
        if spec.head_dim > 256:
            raise ConfigError(f"a key size of {spec.head_dim} exceeds the 256 the recurrence kernel keeps in registers")
        if spec.decay_rank <= 0:
            raise ConfigError(f"the decay's inner width must be positive, got {spec.decay_rank}")
        self.spec = spec
        self.dtype = ctx.dtype
        self.inner = spec.n_heads * spec.head_dim
        self.w_proj: Dict[str, torch.Tensor] = {}
        self.w_out: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        specs = {f"mu_{p}": ParamSpec((s.hidden,), role="gain", init="normal") for p in MIXES}
        for p in ("r", "k", "v", "g"):
            specs[f"{p}_proj.weight"] = ParamSpec((self.inner, s.hidden))
        specs.update({"w1.weight": ParamSpec((s.decay_rank, s.hidden)),
                      "w2.weight": ParamSpec((self.inner, s.decay_rank)),
                      "w0": ParamSpec((self.inner,), role="gain", init="normal"),
                      "u": ParamSpec((s.n_heads, s.head_dim), role="gain", init="normal"),
                      "norm.weight": ParamSpec((self.inner,), role="gain", init="gain"),
                      "o_proj.weight": ParamSpec((s.hidden, self.inner))})
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.mu = torch.stack([tensors[f"mu_{p}"] for p in MIXES]).contiguous()
        self.w_proj = {p: tensors[f"{p}_proj.weight"] for p in ("r", "k", "v", "g")}
        self.w1, self.w2 = tensors["w1.weight"], tensors["w2.weight"]
        self.w0, self.bonus = tensors["w0"], tensors["u"].reshape(-1).contiguous()
        self.norm_gain = tensors["norm.weight"]
        self.w_out = tensors["o_proj.weight"]

    def cache_request(self) -> CompositeRequest:
        s = self.spec
        return CompositeRequest((StateRequest((s.n_heads, s.head_dim, s.head_dim)), StateRequest((s.hidden,))))

    def flops(self, new_counts, starts) -> int:
        s = self.spec
        return 2 * sum(new_counts) * (self.matrix_elements() + 2 * s.n_heads * s.head_dim * s.head_dim)

    def activation_bytes(self, n_tokens: int) -> int:
        s = self.spec
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * (len(MIXES) * s.hidden * size + 6 * self.inner * 4 + s.decay_rank * (4 + size) + self.inner * size)

    def forward(self, step, xn, x_accum, cache, owns_cache: bool) -> None:
        if not owns_cache:
            raise ConfigError("a recurrent layer cannot run on another layer's state")
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        state, kept = cache.parts
        mixes = ws.get("timemix.mixes", (len(MIXES), n, s.hidden), self.dtype)
        ops.shift_mix(xn, self.mu, kept.state, step.token_seq, step.cu_seqlens, step.seq_slots, mixes)
        proj = ws.get("timemix.proj", (n, 4 * self.inner), torch.float32)
        for i, p in enumerate(("r", "k", "v", "g")):
            ops.gemm(mixes[i], self.w_proj[p], proj[:, i * self.inner:(i + 1) * self.inner], workspace=ws.scratch())
        low = ws.get("timemix.low", (n, s.decay_rank), torch.float32)
        ops.gemm(mixes[4], self.w1, low, workspace=ws.scratch())
        low_act = ws.get("timemix.low_act", (n, s.decay_rank), self.dtype)
        ops.tanh(low, low_act)
        decay = ws.get("timemix.decay", (n, self.inner), torch.float32)
        ops.gemm(low_act, self.w2, decay, workspace=ws.scratch())
        o = ws.get("timemix.o", (n, self.inner), torch.float32)
        # (the recurrence kernel turns the logits into decays, exp(-exp(x + w0)), on their way into its LDS)
        ops.decay_scan(proj, 0, proj, self.inner, proj, 2 * self.inner, state.state, step.cu_seqlens, step.seq_slots, o,
                       s.n_heads, s.head_dim, s.head_dim, decay=decay, decay_col0=0, bonus=self.bonus, decay_offset=self.w0)
        gated = ws.get("timemix.gated", (n, self.inner), self.dtype)
        ops.head_norm_gate(o, proj, 3 * self.inner, self.norm_gain, gated, s.n_heads, s.eps, gate="silu")
        stream(step).add_product(gated, self.w_out, x_accum)


register_mixer("time_mix", TimeMix)
