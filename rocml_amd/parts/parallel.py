"""A set of mixers that all run on one input: the result is ``weight * sum_b norm_b(out_b)``,
every branch's output normed over the model width with a gain of its own.

A branch is any registered mixer, built from its spec; each keeps what it needs in the cache
through a part of a composite request.  Branches whose first step is a product with the input
(``input_weight``) share one product over their matrices laid one under the other, and each finds
its columns in the result.  The branches' outputs stay in buffers of their own: a block
that norms after its sum takes them as they are (``branches``) and does the branches' norms, their
sum, the residual sum and its own norm in one kernel; in any other block ``forward`` adds the
weighted sum to the stream.

``normed`` false: the branches' outputs are summed as they are (no norms, no gains).  ``branch_weights``: a
factor per branch instead of one for all.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..config.spec import ParallelMixerSpec
from ..errors import ConfigError
from .base import BuildContext, CompositeRequest, Mixer, ParamSpec
from .registry import build_mixer, register_mixer
from .residual import stream


class ParallelMixer(Mixer):
    adds_only = True

    def __init__(self, spec: ParallelMixerSpec, ctx: BuildContext):
        if not 1 <= len(spec.branches) <= 4:
            raise ConfigError(f"a parallel mixer has one to four branches, got {len(spec.branches)}")
        names = [name for name, _ in spec.branches]
        if len(set(names)) != len(names):
            raise ConfigError(f"the branches of a parallel mixer need different names, got {names}")
        self.spec = spec
        self.dtype = ctx.dtype
        self.normed = bool(getattr(spec, "normed", True))
        weights = getattr(spec, "branch_weights", None)
        if weights is not None and len(weights) != len(spec.branches):
            raise ConfigError(f"{len(weights)} weights for {len(spec.branches)} branches")
        self.weights = tuple(float(w) for w in weights) if weights is not None else (float(spec.weight),) * len(spec.branches)
        if self.normed and len(set(self.weights)) > 1:
            raise ConfigError("branches that are normed share one weight")
        self.children = {name: build_mixer(sub, ctx) for name, sub in spec.branches}
        self.graph_safe = all(getattr(c, "graph_safe", True) for c in self.children.values())
        self.prompt_graph_safe = all(getattr(c, "prompt_graph_safe", False) for c in self.children.values())
        self.kernel_families = tuple(f for c in self.children.values() for f in getattr(c, "kernel_families", ()))
        self.gains: Dict[str, torch.Tensor] = {}
        self.w_in = None              # the branches' first matrices as one, if they share a product
        self.first_column: Dict[str, int] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {}
        for name, child in self.children.items():
            for p, ps in child.param_specs().items():
                specs[f"{name}.{p}"] = ps
            if self.normed:
                specs[f"{name}.out_norm.weight"] = ParamSpec((self.spec.hidden,), role="gain", init="gain")
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for name, child in self.children.items():
            prefix = name + "."
            own = {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
            self.gains[name] = own.pop("out_norm.weight") if self.normed else None
            child.bind(own)
        # One product for all branches that can take its result: their matrices one under the other, each
        # branch's own matrix replaced by its rows of the whole (no second copy stays).
        takers = [(name, child) for name, child in self.children.items()
                  if getattr(child, "input_weight", None) is not None and child.input_weight() is not None]
        if len(takers) >= 2 and len({w.dtype for w in (c.input_weight() for _, c in takers)}) == 1:
            self.w_in = torch.cat([child.input_weight() for _, child in takers], dim=0).contiguous()
            at = 0
            for name, child in takers:
                n_rows = child.input_weight().shape[0]
                self.first_column[name] = at
                child.adopt_input_weight(self.w_in[at:at + n_rows])
                at += n_rows

    def cache_request(self) -> CompositeRequest:
        return CompositeRequest(tuple(child.cache_request() for child in self.children.values()))

    def flops(self, new_counts, starts) -> int:
        return sum(child.flops(new_counts, starts) for child in self.children.values())

    def activation_bytes(self, n_tokens: int) -> int:
        return sum(child.activation_bytes(n_tokens) + n_tokens * self.spec.hidden * 4 for child in self.children.values())

    def branches(self, step, xn, cache, owns_cache: bool):
        """Runs every branch on ``xn`` and returns ``(outputs, gains, weight)``: the mixer's result is
        ``weight * sum_b rms(outputs[b]) * gains[b]``; the outputs are 32-bit ``[tokens, hidden]``."""
        ws = step.workspace
        rs = stream(step)
        before, before_defer = rs.overwrite, rs.defer_overwrite
        rs.defer_overwrite = False        # the branches' outputs are read by a kernel that takes whole sums
        views = cache.parts if cache is not None else (None,) * len(self.children)
        outs: List[torch.Tensor] = []
        proj = None
        if self.w_in is not None and owns_cache:
            proj = ws.get("parallel.proj", (step.n_tokens, self.w_in.shape[0]), torch.float32)
            ops.gemm(xn, self.w_in, proj, workspace=ws.scratch())
        for i, (name, child) in enumerate(self.children.items()):
            y = ws.get(f"parallel.y{i}", (step.n_tokens, self.spec.hidden), torch.float32)
            rs.overwrite = True
            if proj is not None and name in self.first_column:
                child.forward(step, xn, y, views[i], owns_cache, projected=(proj, self.first_column[name]))
            else:
                child.forward(step, xn, y, views[i], owns_cache)
            ws.flush_pending()
            outs.append(y)
        rs.overwrite, rs.defer_overwrite = before, before_defer
        return outs, [self.gains[name] for name in self.children], self.weights[0]

    def forward(self, step, xn, x_accum, cache, owns_cache: bool) -> None:
        outs, gains, weight = self.branches(step, xn, cache, owns_cache)
        step.workspace.flush_pending()
        if not self.normed:
            ops.weighted_sum(x_accum, outs, self.weights, alpha=0.0 if stream(step).overwrite else 1.0)
            return
        ops.sum_norm(x_accum, outs, gains, None, self.spec.eps, alpha=0.0 if stream(step).overwrite else 1.0, weight=weight)


register_mixer("parallel", ParallelMixer)
