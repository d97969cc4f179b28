"""Arrangement of a mixer and a feed-forward into one layer.

``pre_norm`` is the reference's wiring (rocml/src/forward/chunk_forward.rs:107-135):
``x += mixer(norm(x))``, then ``x += ffn(norm(x))``; the residual stream ``x`` stays
32-bit and the normalised copy has the activation type.

``post_norm`` norms after the sum: ``x <- norm(a x + mixer(x))``, then ``x <- norm(a x + ffn(x))`` with
``a`` the block's ``residual_scale``; the sublayers read the stream itself.

``sublayer_norm`` norms a sublayer's output alone: ``x += norm(mixer(x))``, ``x += norm(ffn(x))`` and, if the
layer has one, ``x += norm(side(x))``; the sublayers read the stream itself."""
from __future__ import annotations

from typing import Dict

from .. import ops

import torch

from ..config.spec import BlockSpec
from ..errors import ConfigError
from .base import BuildContext, FullNormHint, ParamSpec, Part
from .registry import build_feed_forward, build_mixer, build_norm, register_block
from .residual import stream


class PreNormBlock(Part):
    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        self.dtype = ctx.dtype
        self.hidden = spec.mixer_norm.size
        self.children = {"mixer_norm": build_norm(spec.mixer_norm, ctx),
                         "mixer": build_mixer(spec.mixer, ctx)}
        if spec.ffn is not None:          # a layer may be its mixer alone
            self.children["ffn_norm"] = build_norm(spec.ffn_norm, ctx)
            self.children["ffn"] = build_feed_forward(spec.ffn, ctx)
        self.mixer_norm = self.children["mixer_norm"]
        self.mixer = self.children["mixer"]
        self.ffn_norm = self.children.get("ffn_norm")
        self.ffn = self.children.get("ffn")
        self.graph_safe = all(getattr(c, "graph_safe", True) for c in self.children.values())
        self.prompt_graph_safe = all(getattr(c, "prompt_graph_safe", False) for c in self.children.values())

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {f"{name}.{p}": spec for name, child in self.children.items()
                for p, spec in child.param_specs().items()}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for name, child in self.children.items():
            prefix = name + "."
            child.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def cache_request(self):
        return self.mixer.cache_request()

    def flops(self, new_counts, starts) -> int:
        return self.mixer.flops(new_counts, starts) + (self.ffn.flops(new_counts, starts) if self.ffn is not None else 0)

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * self.hidden * size + self.mixer.activation_bytes(n_tokens) + \
            (self.ffn.activation_bytes(n_tokens) if self.ffn is not None else 0)

    takes_pending = True      # forward() may be handed a stream that still lacks deferred sums
    takes_next_norm = True    # forward() accepts the hint of the norm that reads the stream after it

    def entry_hint(self, step):
        """The norm this block reads the residual stream with first, for the product that completes
        the stream before it, if the block's mixer can apply the norm's scale itself in this step."""
        return self._hint(step, self.mixer_norm, self.mixer)

    def forward(self, step, x: torch.Tensor, cache, owns_cache: bool, next_norm=None) -> None:
        """``next_norm``: the hint of the norm that reads ``x`` after this block (``entry_hint`` of
        the block that runs next), or None."""
        ws = step.workspace
        rs = stream(step)
        xn, rs.row_scale = self._norm(step, self.mixer_norm, x)
        if not getattr(self.mixer, "adds_only", False):
            ws.flush_pending()
        rs.next_norm = self._hint(step, self.ffn_norm, self.ffn) if self.ffn is not None else next_norm
        self.mixer.forward(step, xn, x, cache, owns_cache)
        rs.next_norm = None
        if self.ffn is None:
            rs.row_scale = None
            return
        xn, rs.row_scale = self._norm(step, self.ffn_norm, x)
        if not getattr(self.ffn, "adds_only", False):
            ws.flush_pending()
        rs.next_norm = next_norm
        self.ffn.forward(step, xn, x)
        rs.next_norm = None
        rs.row_scale = None

    @staticmethod
    def _hint(step, norm, consumer):
        takes = getattr(consumer, "takes_row_scale", None)
        hint = getattr(norm, "prescale_hint", None)
        if takes is None or hint is None or not takes(step):
            return None
        return hint()

    def _norm(self, step, norm, x):
        """The norm's output and what is left to apply to it (None: nothing).  A part may leave the
        last step of its residual sum (adding split-K partial sums to x) to the norm that reads x
        next, or have prepared the norm's output itself; a norm that can use neither gets x
        completed."""
        ws = step.workspace
        gain = getattr(norm, "gain", None)
        prepared = stream(step).take_prescaled(x, gain) if gain is not None else None
        if prepared is not None:
            return prepared
        xn = ws.get("block.xn", tuple(x.shape), self.dtype)
        if getattr(norm, "fuses_pending", False):
            norm.forward(x, xn, pending=ws.take_pending(x))
        else:
            ws.flush_pending()
            norm.forward(x, xn)
        return xn, None


register_block("pre_norm", PreNormBlock)

_COPY_KEY = "post_norm.stream_copy"


class PostNormBlock(Part):
    """``x <- norm1(a x + mixer(x))``, ``x <- norm2(a x + ffn(x))``.  A sublayer reads the stream itself
    (in the compute type: a copy that the norm kernel before it wrote, the stream itself in 32-bit)
    and writes its result to a buffer of the block; one kernel then forms the scaled residual sum and
    its norm in 32-bit, in place, and the copy for the next sublayer.  A mixer that is a sum of normed
    branches hands its branches over as they are (``branches``) and the same kernel norms and sums
    them on the way."""
    takes_pending = False
    takes_next_norm = False

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        self.dtype = ctx.dtype
        self.hidden = spec.mixer_norm.size
        self.alpha = float(spec.residual_scale)
        self.children = {"mixer_norm": build_norm(spec.mixer_norm, ctx),
                         "mixer": build_mixer(spec.mixer, ctx)}
        if spec.ffn is not None:
            self.children["ffn_norm"] = build_norm(spec.ffn_norm, ctx)
            self.children["ffn"] = build_feed_forward(spec.ffn, ctx)
        self.mixer_norm = self.children["mixer_norm"]
        self.mixer = self.children["mixer"]
        self.ffn_norm = self.children.get("ffn_norm")
        self.ffn = self.children.get("ffn")
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and (not hasattr(norm, "gain") or not hasattr(norm, "eps")):
                raise ConfigError("a block that norms after the sum needs norms of the root-mean-square kind")
        self.graph_safe = all(getattr(c, "graph_safe", True) for c in self.children.values())
        self.prompt_graph_safe = all(getattr(c, "prompt_graph_safe", False) for c in self.children.values())
        self.kernel_families = tuple(f for c in self.children.values() for f in getattr(c, "kernel_families", ()))

    param_specs = PreNormBlock.param_specs
    bind = PreNormBlock.bind
    cache_request = PreNormBlock.cache_request
    flops = PreNormBlock.flops

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * self.hidden * (size + 4) + self.mixer.activation_bytes(n_tokens) + \
            (self.ffn.activation_bytes(n_tokens) if self.ffn is not None else 0)

    def _operand(self, step, x: torch.Tensor) -> torch.Tensor:
        """The stream as the products' operand."""
        if self.dtype == torch.float32:
            return x
        found = step.memo.get(_COPY_KEY)
        if found is not None and found[0] == x.data_ptr():
            return found[1]
        xb = step.workspace.get("block.stream_copy", tuple(x.shape), self.dtype)
        ops.convert(x, xb)
        step.memo[_COPY_KEY] = (x.data_ptr(), xb)
        return xb

    def _sum_norm(self, step, x, outs, gains, weight, norm) -> None:
        copy = None
        if self.dtype != torch.float32:
            copy = step.workspace.get("block.stream_copy", tuple(x.shape), self.dtype)
        ops.sum_norm(x, outs, gains, norm.gain, norm.eps, alpha=self.alpha, weight=weight, copy=copy)
        if copy is not None:
            step.memo[_COPY_KEY] = (x.data_ptr(), copy)

    def forward(self, step, x: torch.Tensor, cache, owns_cache: bool) -> None:
        ws = step.workspace
        rs = stream(step)
        ws.flush_pending()
        rs.row_scale = rs.next_norm = None
        xb = self._operand(step, x)
        rs.overwrite = True
        try:
            if hasattr(self.mixer, "branches"):
                outs, gains, weight = self.mixer.branches(step, xb, cache, owns_cache)
            else:
                y = ws.get("block.sublayer", tuple(x.shape), torch.float32)
                self.mixer.forward(step, xb, y, cache, owns_cache)
                outs, gains, weight = [y], [None], 1.0
            ws.flush_pending()
            self._sum_norm(step, x, outs, gains, weight, self.mixer_norm)
            if self.ffn is None:
                return
            xb = self._operand(step, x)
            y = ws.get("block.sublayer", tuple(x.shape), torch.float32)
            rs.overwrite = True
            self.ffn.forward(step, xb, y)
            ws.flush_pending()
            self._sum_norm(step, x, [y], [None], 1.0, self.ffn_norm)
        finally:
            rs.overwrite = False


register_block("post_norm", PostNormBlock)


class SublayerNormBlock(Part):
    """``x += norm1(mixer(x))``, ``x += norm2(ffn(x))``, ``x += norm3(side(x))`` (the last two may be absent).  A
    sublayer reads the stream itself (in the compute type: a copy that the kernel before it wrote, the stream
    itself in 32-bit) and writes its result to a buffer of the block; one kernel then norms that buffer, adds it
    to the 32-bit stream and writes the copy for the next sublayer.  The norms are layer norms (weight and bias)
    or root-mean-square norms (weight), each sublayer its own."""
    takes_pending = False
    takes_next_norm = False

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        self.dtype = ctx.dtype
        self.hidden = spec.mixer_norm.size
        self.children = {"mixer_norm": build_norm(spec.mixer_norm, ctx),
                         "mixer": build_mixer(spec.mixer, ctx)}
        if spec.ffn is not None:
            self.children["ffn_norm"] = build_norm(spec.ffn_norm, ctx)
            self.children["ffn"] = build_feed_forward(spec.ffn, ctx)
        if spec.side is not None:
            self.children["side_norm"] = build_norm(spec.side_norm, ctx)
            self.children["side"] = build_feed_forward(spec.side, ctx)
        self.mixer = self.children["mixer"]
        self.ffn = self.children.get("ffn")
        self.side = self.children.get("side")
        for name in ("mixer_norm", "ffn_norm", "side_norm"):
            norm = self.children.get(name)
            if norm is not None and (not hasattr(norm, "gain") or not hasattr(norm, "eps")):
                raise ConfigError("a block that norms its sublayers' outputs needs norms with a gain and an eps")
        self.graph_safe = all(getattr(c, "graph_safe", True) for c in self.children.values())
        self.prompt_graph_safe = all(getattr(c, "prompt_graph_safe", False) for c in self.children.values())
        self.kernel_families = tuple(f for c in self.children.values() for f in getattr(c, "kernel_families", ()))

    param_specs = PreNormBlock.param_specs
    bind = PreNormBlock.bind
    cache_request = PreNormBlock.cache_request

    def flops(self, new_counts, starts) -> int:
        return sum(part.flops(new_counts, starts) for part in (self.mixer, self.ffn, self.side) if part is not None)

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * self.hidden * (size + 4) + sum(part.activation_bytes(n_tokens)
                                                         for part in (self.mixer, self.ffn, self.side) if part is not None)

    _operand = PostNormBlock._operand

    def _norm_add(self, step, x, y, norm) -> None:
        copy = None
        if self.dtype != torch.float32:
            copy = step.workspace.get("block.stream_copy", tuple(x.shape), self.dtype)
        # (a product cut along K may have left its pieces for this kernel to add: they are all of y then)
        pending = step.workspace.take_pending_or_whole(y)
        partials, replace = pending if pending is not None else (None, False)
        ops.norm_add(x, y, norm.gain, getattr(norm, "bias", None), norm.eps, layer=bool(getattr(norm, "centred", False)), copy=copy,
                     partials=partials, replace=replace)
        if copy is not None:
            step.memo[_COPY_KEY] = (x.data_ptr(), copy)

    def _branches_norm_add(self, step, x, xb, cache, owns_cache: bool) -> bool:
        """A mixer that is a sum of normed branches hands them over as they are: one kernel norms the branches, sums
        them, norms the sum and adds it to the stream.  False: the mixer is of another kind, or its rows do not fit
        that kernel (the mixer then forms its sum itself)."""
        if not hasattr(self.mixer, "branches") or not ops.norm_add_branches_fits(self.hidden, len(self.mixer.children)):
            return False
        outs, gains, weight = self.mixer.branches(step, xb, cache, owns_cache)
        if any(g is None for g in gains):
            raise ConfigError("the branches of a parallel mixer come with a gain each")
        norm = self.children["mixer_norm"]
        copy = None
        if self.dtype != torch.float32:
            copy = step.workspace.get("block.stream_copy", tuple(x.shape), self.dtype)
        ops.norm_add_branches(x, outs, gains, weight, self.mixer.spec.eps, norm.gain, getattr(norm, "bias", None), norm.eps,
                              layer=bool(getattr(norm, "centred", False)), copy=copy)
        if copy is not None:
            step.memo[_COPY_KEY] = (x.data_ptr(), copy)
        return True

    def forward(self, step, x: torch.Tensor, cache, owns_cache: bool) -> None:
        ws = step.workspace
        rs = stream(step)
        ws.flush_pending()
        rs.row_scale = rs.next_norm = None
        try:
            xb = self._operand(step, x)
            y = ws.get("block.sublayer", tuple(x.shape), torch.float32)
            rs.overwrite = rs.defer_overwrite = True
            if not self._branches_norm_add(step, x, xb, cache, owns_cache):
                self.mixer.forward(step, xb, y, cache, owns_cache)
                self._norm_add(step, x, y, self.children["mixer_norm"])
            for part, norm in ((self.ffn, "ffn_norm"), (self.side, "side_norm")):
                if part is None:
                    continue
                xb = self._operand(step, x)
                y = ws.get("block.sublayer", tuple(x.shape), torch.float32)
                rs.overwrite = rs.defer_overwrite = True
                part.forward(step, xb, y)
                self._norm_add(step, x, y, self.children[norm])
        finally:
            rs.overwrite = rs.defer_overwrite = False


register_block("sublayer_norm", SublayerNormBlock)


class SandwichNormBlock(Part):
    """``x += out_norm1(mixer(norm1(x)))``, ``x += out_norm2(ffn(norm2(x)))``: a norm before and one after every
    sublayer (the feed-forward may be absent).  The first norm of a sublayer writes the products' operand in the
    compute type; the sublayer writes its result to a buffer of the block; one kernel then norms that buffer and
    adds it to the 32-bit stream (it takes a product's K pieces in place of the buffer) and, in the same pass over
    the row, forms the norm that reads the stream next: the feed-forward's first norm behind the mixer, the next
    layer's first norm behind the feed-forward when that layer is of this kind (``entry_hint``).  The norms are
    root-mean-square norms with a gain."""
    takes_pending = False
    takes_next_norm = True
    _READY = "sandwich_norm.operand"      # in step.memo: (stream, gain, operand) of a norm that the kernel before formed

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        if spec.mixer_out_norm is None or (spec.ffn is not None and (spec.ffn_norm is None or spec.ffn_out_norm is None)):
            raise ConfigError("a block with a norm before and after every sublayer needs both norms of each")
        self.dtype = ctx.dtype
        self.hidden = spec.mixer_norm.size
        self.children = {"mixer_norm": build_norm(spec.mixer_norm, ctx),
                         "mixer": build_mixer(spec.mixer, ctx),
                         "mixer_out_norm": build_norm(spec.mixer_out_norm, ctx)}
        if spec.ffn is not None:
            self.children["ffn_norm"] = build_norm(spec.ffn_norm, ctx)
            self.children["ffn"] = build_feed_forward(spec.ffn, ctx)
            self.children["ffn_out_norm"] = build_norm(spec.ffn_out_norm, ctx)
        self.mixer = self.children["mixer"]
        self.ffn = self.children.get("ffn")
        for name in ("mixer_out_norm", "ffn_out_norm"):
            norm = self.children.get(name)
            if norm is not None and (not hasattr(norm, "gain") or not hasattr(norm, "eps") or getattr(norm, "centred", False)):
                raise ConfigError("a block that norms its sublayers' outputs before adding them needs root-mean-square norms there")
        self.graph_safe = all(getattr(c, "graph_safe", True) for c in self.children.values())
        self.prompt_graph_safe = all(getattr(c, "prompt_graph_safe", False) for c in self.children.values())
        self.kernel_families = tuple(f for c in self.children.values() for f in getattr(c, "kernel_families", ()))

    param_specs = PreNormBlock.param_specs
    bind = PreNormBlock.bind
    cache_request = PreNormBlock.cache_request
    flops = PreNormBlock.flops

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * self.hidden * (size + 4) + self.mixer.activation_bytes(n_tokens) + \
            (self.ffn.activation_bytes(n_tokens) if self.ffn is not None else 0)

    def entry_hint(self, step):
        """The norm this block reads the stream with first, for the kernel that completes the stream before it."""
        norm = self.children["mixer_norm"]
        gain = getattr(norm, "gain", None)
        if gain is None or not hasattr(norm, "eps") or getattr(norm, "centred", False):
            return None
        return FullNormHint(gain, float(norm.eps), self.hidden)

    def _sublayer(self, step, x, norm, run, out_norm, following) -> None:
        """``following``: a ``FullNormHint`` of the norm that reads the stream after this sublayer, or None."""
        ws = step.workspace
        rs = stream(step)
        ready = step.memo.pop(self._READY, None)
        gain = getattr(norm, "gain", None)
        if ready is not None and gain is not None and ready[0] == x.data_ptr() and ready[1] == gain.data_ptr():
            xn = ready[2]           # the kernel that completed the stream formed this norm on its way
        else:
            xn = ws.get("block.xn", tuple(x.shape), self.dtype)
            norm.forward(x, xn)
        y = ws.get("block.sublayer", tuple(x.shape), torch.float32)
        rs.overwrite = rs.defer_overwrite = True
        run(xn, y)
        # (a product cut along K may have left its pieces for this kernel to add: they are all of y then)
        pending = ws.take_pending_or_whole(y)
        partials, replace = pending if pending is not None else (None, False)
        if isinstance(following, FullNormHint) and following.width == x.shape[1]:
            # (the sublayer is done with its operand: the buffer takes the next one)
            nxt = ws.get("block.xn", tuple(x.shape), self.dtype)
            ops.norm_add(x, y, out_norm.gain, None, out_norm.eps, layer=False, partials=partials, replace=replace, copy=nxt,
                         next_gain=following.gain, next_eps=following.eps)
            step.memo[self._READY] = (x.data_ptr(), following.gain.data_ptr(), nxt)
        else:
            ops.norm_add(x, y, out_norm.gain, None, out_norm.eps, layer=False, partials=partials, replace=replace)

    def forward(self, step, x: torch.Tensor, cache, owns_cache: bool, next_norm=None) -> None:
        rs = stream(step)
        step.workspace.flush_pending()
        rs.row_scale = rs.next_norm = None
        try:
            inner = None
            if self.ffn is not None:
                n2 = self.children["ffn_norm"]
                if getattr(n2, "gain", None) is not None and hasattr(n2, "eps") and not getattr(n2, "centred", False):
                    inner = FullNormHint(n2.gain, float(n2.eps), self.hidden)
            self._sublayer(step, x, self.children["mixer_norm"], lambda xn, y: self.mixer.forward(step, xn, y, cache, owns_cache),
                           self.children["mixer_out_norm"], inner if self.ffn is not None else next_norm)
            if self.ffn is not None:
                self._sublayer(step, x, self.children["ffn_norm"], lambda xn, y: self.ffn.forward(step, xn, y),
                               self.children["ffn_out_norm"], next_norm)
        finally:
            rs.overwrite = rs.defer_overwrite = False


register_block("sandwich_norm", SandwichNormBlock)
