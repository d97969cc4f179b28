"""Softmax attention with grouped key/value heads over the paged cache.

Order of work as in the reference's layer (rocml/src/forward/attention_chunk.rs:97-330):
projections without bias, per-head norm of q and k, rotation, append to the cache, causal
attention with the scale applied after the dot product, output projection, residual sum.
Here q, k and v come from one product over the concatenated weight, norm + rotation +
append are one kernel, and the residual sum is the output product's epilogue.  Head
counts, head size, scale, window, the optional norm and the optional position encoding
are the spec's, nothing is fixed here.

A layer may also ask for biased projections, a value head of another size than the key head,
blocks of positions instead of a window, a penalty on distance (a slope per head) and a sink in
the softmax.  Any of these takes the layer off the matrix-core attention kernels, which know none
of them, and onto the plain kernel, which takes them all as parameters; the projections and the
append kernel are the same ones.

Further options: a learned sink per head (``exp(sink_h)`` in the denominator), a soft cap on the scaled
scores, and a short causal convolution per channel on q, k and v right behind their projection (32-bit, with
the last ``taps - 1`` projected rows of a sequence kept as a state beside its keys and values).  The
matrix-core kernels take the first two; the convolution is a kernel of its own in front of the
norm-and-rotation kernel.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import AttentionSpec
from ..errors import ConfigError
from .base import BuildContext, CompositeRequest, KVCacheRequest, Mixer, ParamSpec, StateRequest
from .registry import build_position, register_mixer
from .residual import stream


class Attention(Mixer):
    adds_only = True
    FUSED_PREFILL_MIN_TOKENS = 1024
    SPAN_STATS_MIN_TOKENS = 64         # from so many tokens on, a kernel of its own forms the factors of a whole-row norm of q and k

    def __init__(self, spec: AttentionSpec, ctx: BuildContext):
        if spec.n_heads % spec.n_kv_heads != 0:
            raise ConfigError(f"{spec.n_heads} query heads are not a multiple of {spec.n_kv_heads} key/value heads")
        self.span = getattr(spec, "qk_norm_span", "head")
        if self.span not in ("head", "projection"):
            raise ConfigError(f"the norm of q and k spans a 'head' or the whole 'projection', got {self.span!r}")
        if spec.qk_norm is not None and spec.qk_norm.size != (spec.head_dim if self.span == "head" else spec.n_heads * spec.head_dim):
            raise ConfigError("the norm of q and k must span the head size, or with span 'projection' all query heads")
        if self.span == "projection" and (spec.qk_norm is None or not getattr(spec.qk_norm, "learned", True)):
            raise ConfigError("a norm over the whole projection needs learned gains")
        if spec.qk_norm is not None and spec.qk_norm.kind != "rmsnorm":
            # the norm of q and k runs inside the rotation and attention kernels, which know one kind
            raise ConfigError(f"the per-head norm must be of kind 'rmsnorm', got {spec.qk_norm.kind!r}")
        if spec.window is not None and spec.window <= 0:
            raise ConfigError(f"window must be positive, got {spec.window}")
        if spec.chunk is not None and (spec.chunk <= 0 or spec.window is not None):
            raise ConfigError("blocks of positions must be positive in size and exclude a window")
        if spec.distance_slopes is not None and len(spec.distance_slopes) != spec.n_heads:
            raise ConfigError(f"{len(spec.distance_slopes)} distance slopes for {spec.n_heads} heads")
        self.v_head_dim = spec.head_dim if spec.v_head_dim is None else spec.v_head_dim
        # what the matrix-core kernels do not know: such a layer runs the plain attention kernel
        self.extras = (self.v_head_dim != spec.head_dim or spec.chunk is not None
                       or spec.distance_slopes is not None or spec.sink or getattr(spec, "softcap", None) is not None)
        self.sink_learned = bool(getattr(spec, "sink_learned", False))
        if self.sink_learned and not spec.sink:
            raise ConfigError("learned sinks need the sink switched on")
        self.softcap = getattr(spec, "softcap", None)
        if self.softcap is not None and not self.softcap > 0:
            raise ConfigError(f"the soft cap of the scores must be positive, got {self.softcap}")
        self.conv = getattr(spec, "conv", None)
        if self.conv is not None and not 1 <= self.conv <= 8:
            raise ConfigError(f"the convolution on q, k and v has {self.conv} taps; 1 to 8 are supported")
        if self.conv is not None and (spec.bias or spec.qk_norm is not None and getattr(spec, "qk_norm_span", "head") != "head"):
            raise ConfigError("a convolution on q, k and v goes without biases and without a norm over the whole projection")
        if spec.q_temp is not None and not (spec.q_temp[1] > 0):
            raise ConfigError(f"the period of the query's stretch must be positive, got {spec.q_temp[1]}")
        # what only the norm-and-rotation kernel knows (the kernels that prepare their queries
        # themselves do not): a stretch of the query with its position, an output gate
        # (and a norm over a token's whole q and k rows, whose factors a kernel of their own forms first)
        self.separate_q = spec.q_temp is not None or spec.gate or self.span == "projection" or self.conv is not None \
            or self.sink_learned or self.softcap is not None
        self.gate_per_head = bool(getattr(spec, "gate_per_head", False))
        if self.gate_per_head and not spec.gate:
            raise ConfigError("a gate per head needs the output gate switched on")
        self.o_bias = spec.bias if getattr(spec, "o_bias", None) is None else bool(spec.o_bias)
        self.norm_learned = spec.qk_norm is None or getattr(spec.qk_norm, "learned", True)
        self.slopes: Optional[torch.Tensor] = None
        if spec.distance_slopes is not None and torch.device(ctx.device).type != "meta":
            self.slopes = torch.tensor(spec.distance_slopes, dtype=torch.float32, device=ctx.device)
        self.spec = spec
        self.dtype = ctx.dtype
        self.n_cus = ops.cu_count(ctx.device)
        self.q_dim = spec.n_heads * spec.head_dim
        self.kv_dim = spec.n_kv_heads * spec.head_dim
        self.v_dim = spec.n_kv_heads * self.v_head_dim
        self.o_dim = spec.n_heads * self.v_head_dim
        self.g_dim = 0 if not spec.gate else (spec.n_heads if self.gate_per_head else self.o_dim)
        self.position = build_position(spec.position, ctx) if spec.position is not None else None
        self.pairing = getattr(self.position, "pairing", "halves")
        if self.pairing not in ops.ROPE_PAIRINGS:
            raise ConfigError(f"unknown rotation pairing {self.pairing!r}; known: {sorted(ops.ROPE_PAIRINGS)}")
        # (what may be recorded as a graph: the attention's own launches always, its position
        # encoding's if that part says so)
        self.graph_safe = self.position is None or getattr(self.position, "graph_safe", True)
        self.prompt_graph_safe = self.graph_safe and (self.position is None or getattr(self.position, "prompt_graph_safe", False))
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.q_gain: Optional[torch.Tensor] = None
        self.k_gain: Optional[torch.Tensor] = None
        self.b_qkv: Optional[torch.Tensor] = None
        self.b_o: Optional[torch.Tensor] = None
        self.sinks: Optional[torch.Tensor] = None
        self.conv_w: Optional[torch.Tensor] = None
        if self.conv is not None:
            self.kernel_families = ("recurrent",)

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        specs = {"q_proj.weight": ParamSpec((self.q_dim, s.hidden)),
                 "k_proj.weight": ParamSpec((self.kv_dim, s.hidden)),
                 "v_proj.weight": ParamSpec((self.v_dim, s.hidden)),
                 "o_proj.weight": ParamSpec((s.hidden, self.o_dim))}
        if s.bias:       # added in 32-bit to the products' sums
            specs.update({"q_proj.bias": ParamSpec((self.q_dim,), role="gain", init="normal"),
                          "k_proj.bias": ParamSpec((self.kv_dim,), role="gain", init="normal"),
                          "v_proj.bias": ParamSpec((self.v_dim,), role="gain", init="normal")})
        if self.o_bias:
            specs["o_proj.bias"] = ParamSpec((s.hidden,), role="gain", init="normal")
        if s.qk_norm is not None and self.norm_learned:
            whole = self.span == "projection"       # one gain per column of the projection instead of one per head value
            specs["q_norm.weight"] = ParamSpec((self.q_dim if whole else s.head_dim,), role="gain", init="gain")
            specs["k_norm.weight"] = ParamSpec((self.kv_dim if whole else s.head_dim,), role="gain", init="gain")
        if s.gate:
            specs["g_proj.weight"] = ParamSpec((self.g_dim, s.hidden))
        if self.sink_learned:
            specs["sink"] = ParamSpec((s.n_heads,), role="gain", init="normal")
        if self.conv is not None:       # stored [channels, taps], the last tap the current token's
            specs["q_conv.weight"] = ParamSpec((self.q_dim, self.conv), role="gain", init="normal")
            specs["k_conv.weight"] = ParamSpec((self.kv_dim, self.conv), role="gain", init="normal")
            specs["v_conv.weight"] = ParamSpec((self.v_dim, self.conv), role="gain", init="normal")
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # One [Q + 2 KV, hidden] matrix: q rows first, so a layer that only reads another
        # layer's cache multiplies by the leading Q rows.
        # (an output gate's rows come last: its projection rides in the same product)
        self.w_qkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
                               + ([tensors["g_proj.weight"]] if self.spec.gate else []), dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        if self.spec.bias:
            # (an output gate's columns, which come last in the product, have no bias: zeros stand for it)
            self.b_qkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]]
                                   + ([torch.zeros(self.g_dim, dtype=torch.float32, device=self.w_o.device)] if self.g_dim else [])
                                   ).contiguous()
        if self.o_bias:
            self.b_o = tensors["o_proj.bias"]
        if self.sink_learned:
            self.sinks = tensors["sink"]
        if self.conv is not None:
            # [taps, channels] over q, k and v side by side, as the convolution kernel reads it
            self.conv_w = torch.cat([tensors["q_conv.weight"], tensors["k_conv.weight"], tensors["v_conv.weight"]], dim=0).t().contiguous()
        if self.spec.qk_norm is not None:
            if self.norm_learned:
                self.q_gain = tensors["q_norm.weight"]
                self.k_gain = tensors["k_norm.weight"]
            else:       # a norm without a weight: the kernels take a gain of ones
                self.q_gain = self.k_gain = torch.ones(self.spec.head_dim, dtype=torch.float32, device=self.w_o.device)

    def flops(self, new_counts, starts) -> int:
        # the products with the weights, and 4 * heads * head size per query and key it sees
        keys = 0
        w, c = self.spec.window, self.spec.chunk
        for n, s0 in zip(new_counts, starts):
            if c is not None:
                keys += sum((s0 + i) % c + 1 for i in range(n))
            elif w is None:
                keys += n * s0 + n * (n + 1) // 2
            else:
                keys += sum(min(s0 + i + 1, w) for i in range(n))
        return 2 * sum(new_counts) * self.matrix_elements() + \
            2 * self.spec.n_heads * (self.spec.head_dim + self.v_head_dim) * keys

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        rot = 0 if self.position is None else 2 * n_tokens * (self.position.rot_dim // 2) * 4
        return n_tokens * ((self.q_dim + self.kv_dim + self.v_dim) * 4 + (self.q_dim + self.o_dim) * size) + rot

    def _fused_decode(self, step) -> bool:
        rot = None if self.position is None else self.position.rot_dim
        # (blocks, slopes, a sink and biases ride in the fused kernel; a value head of another size does not)
        return not self.separate_q and self.v_head_dim == self.spec.head_dim and step.max_new == 1 and ops.attention_decode_fusable(
            self.dtype, self.spec.n_heads, self.spec.n_kv_heads, self.spec.head_dim, ops.FUSED_DECODE_PAGE, rot, self.pairing)

    def _fused_prefill(self, step, cache) -> bool:
        """Whether the prompt kernel prepares its queries itself: it pays from about a thousand
        tokens on (the preparation lengthens every attention block by some 6 us, the norm-and-rotation
        kernel's q rows cost 8 us per thousand tokens at 32 heads of 128)."""
        rot = None if self.position is None else self.position.rot_dim
        return (not self.extras and not self.separate_q and not self.spec.bias and step.max_new > 1 and step.n_tokens >= self.FUSED_PREFILL_MIN_TOKENS
                and step.cu_seqlens is not None and self.dtype == torch.bfloat16
                and ops.attention_prefill_fusable(cache.k.dtype, self.spec.head_dim, cache.k.shape[2], rot, self.pairing))

    def takes_row_scale(self, step) -> bool:
        # only the decode kernel that reads the projection's sums itself applies a scale to them
        return self._fused_decode(step)

    def cache_request(self):
        s = self.spec
        if s.v_head_dim is None and s.chunk is None:
            kv = KVCacheRequest(s.n_kv_heads, s.head_dim, s.window)
        else:
            kv = KVCacheRequest(s.n_kv_heads, s.head_dim, s.window, v_head_dim=self.v_head_dim, chunk=s.chunk)
        if self.conv is None or self.conv == 1:
            return kv
        # the convolution's last taps - 1 inputs live beside the keys and values
        return CompositeRequest((kv, StateRequest((self.conv - 1, self.q_dim + self.kv_dim + self.v_dim))))

    def _decode_splits(self, step, cache) -> int:
        """Splits of the key range in a decode step: enough blocks to fill the chip, at most one
        per page the block table has room for.  It depends on the step's shape only, never on
        the sequences' lengths, so a recorded step can be replayed as they grow."""
        if step.max_new != 1:
            return 0
        return ops.decode_splits(step.n_tokens * self.spec.n_kv_heads, self.n_cus, min(cache.block_table.shape[1], 64))

    def input_weight(self) -> Optional[torch.Tensor]:
        # only the path of the norm-and-rotation kernel, which takes rows of any stride; and the
        # projection must start at the buffer's first column
        return self.w_qkv if self.separate_q else None

    def adopt_input_weight(self, view: torch.Tensor) -> None:
        self.w_qkv = view

    def forward(self, step, xn, x_accum, cache, owns_cache: bool, projected=None) -> None:
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        rows = self.q_dim + self.kv_dim + self.v_dim + self.g_dim if owns_cache else self.q_dim
        if s.gate and not owns_cache:
            raise ConfigError("a gated attention layer that reads another layer's cache is not supported")
        conv_state = None
        if isinstance(getattr(cache, "parts", None), tuple) and cache.parts:
            cache, conv_state = cache.parts
        if self.conv is not None and not owns_cache:
            raise ConfigError("an attention layer with a convolution on q, k and v cannot read another layer's cache")
        scratch = ws.scratch()
        if projected is not None:
            qkv, first = projected
            if first != 0 or not owns_cache or qkv.shape[1] < rows:
                raise ConfigError("the attention takes a projection that starts at the buffer's first column")
            splits = 0
        else:
            qkv = ws.get("attn.qkv", (n, rows), torch.float32)
            # (the decode kernel that reads the projection adds four partial sums in one trip to memory
            # and further ones one after the other: K is cut into few pieces for it)
            # (the gate's columns are read where they lie: the product is then completed)
            splits = ops.gemm(xn, self.w_qkv[:rows], qkv, workspace=scratch,
                              defer=not s.gate and self.span == "head" and self.conv is None,
                              max_splits=ops.FUSED_DECODE_SPLITS if self._fused_decode(step) else 0)
        if splits:      # the product's split-K partial sums; the next kernel adds them
            qkv = scratch[:splits * n * rows * 4].view(torch.float32).view(splits, n, rows)
        if self.conv is not None:
            # q, k and v pass the convolution in 32-bit, channel by channel; what follows reads its output
            channels = self.q_dim + self.kv_dim + self.v_dim
            mixed = ws.get("attn.qkv_conv", (n, channels), torch.float32)
            if self.conv > 1:
                kept = conv_state.state
            else:
                kept = ws.get("attn.no_conv_state", (1, 0, channels), torch.float32)
            ops.causal_conv(qkv, 0, channels, self.conv_w, None, kept, step.token_seq, step.cu_seqlens, step.seq_slots, mixed,
                            silu=False)
            qkv = mixed
        cos = sin = None
        rot = 0
        if self.position is not None:
            cos, sin = self.position.tables(step)
            rot = self.position.rot_dim
        eps = s.qk_norm.eps if s.qk_norm is not None else 1.0
        o = ws.get("attn.o", (n, self.o_dim), self.dtype)
        if self._fused_decode(step) and cache.k.dtype == self.dtype and cache.k.shape[2] == ops.FUSED_DECODE_PAGE:
            # One token per sequence: norm, rotation, append and attention in one launch, straight
            # from the projection.  The attention's own partial results go behind the projection's.
            used = (splits * n * rows * 4 + 255) // 256 * 256 if splits else 0
            # (a step of one token per sequence numbers its tokens as its sequences)
            ops.attention_decode_fused(qkv, o, cache.k, cache.v, cache.block_table, None, step.token_pos,
                                       s.n_heads, s.n_kv_heads, s.head_dim, s.scale, self.q_gain, self.k_gain, eps,
                                       cos, sin, write_kv=owns_cache, window=s.window, workspace=scratch[used:],
                                       max_len=step.max_len, n_splits=self._decode_splits(step, cache),
                                       row_scale=stream(step).row_scale,
                                       bias=None if self.b_qkv is None else self.b_qkv[:rows], chunk=s.chunk,
                                       slopes=self.slopes, sink=s.sink)
        else:
            if stream(step).row_scale is not None:
                raise ConfigError("the attention was handed an input without its norm's scale in a step it cannot scale")
            if not splits and self._fused_prefill(step, cache):
                # A prompt step: keys and values are prepared and appended, the attention kernel
                # prepares its queries from the projection itself.
                if owns_cache:
                    ops.qk_norm_rope_append(qkv, s.n_heads, s.n_kv_heads, s.head_dim, self.q_gain, self.k_gain, eps,
                                            cos, sin, rot, None, cache.k, cache.v, cache.block_table, step.token_seq,
                                            step.token_pos, write_kv=True, pairing=self.pairing)
                ops.attention_prefill_fused(qkv, o, cache.k, cache.v, cache.block_table, step.token_pos, s.n_heads,
                                            s.n_kv_heads, s.head_dim, s.scale, self.q_gain, eps, cos, sin, s.window,
                                            step.cu_seqlens, step.new_counts, max_len=step.max_len)
            else:
                q = ws.get("attn.q", (n, self.q_dim), self.dtype)
                bias = None if self.b_qkv is None else self.b_qkv[:rows]
                span_inv, span_self = None, False
                if self.span == "projection":
                    if not owns_cache:
                        raise ConfigError("a norm over the whole projection needs the layer's own keys")
                    if n < self.SPAN_STATS_MIN_TOKENS:      # few tokens: every wave of the next kernel sums its token's row itself
                        span_self = True
                    else:
                        span_inv = ws.get("attn.span", (n, 2), torch.float32)
                        ops.qk_span_stats(qkv, self.q_dim, self.kv_dim, bias, eps, span_inv)
                ops.qk_norm_rope_append(qkv, s.n_heads, s.n_kv_heads, s.head_dim, self.q_gain, self.k_gain, eps,
                                        cos, sin, rot, q, cache.k, cache.v, cache.block_table, step.token_seq,
                                        step.token_pos, write_kv=owns_cache, n_splits=max(splits, 1), pairing=self.pairing,
                                        bias=bias, v_head_dim=self.v_head_dim, q_temp=s.q_temp, span_inv=span_inv, span_self=span_self)
                ops.attention(q, o, cache.k, cache.v, cache.block_table, step.token_seq, step.token_pos,
                              s.n_heads, s.n_kv_heads, s.head_dim, s.scale, s.window, workspace=ws.scratch(),
                              cu_seqlens=step.cu_seqlens, max_new=step.max_new, q_counts=step.new_counts,
                              max_len=step.max_len, n_splits=self._decode_splits(step, cache),
                              v_head_dim=self.v_head_dim, chunk=s.chunk, slopes=self.slopes, sink=s.sink, sinks=self.sinks,
                              softcap=self.softcap)
        if s.gate:
            ops.sigmoid_gate(o, qkv[:, rows - self.g_dim:rows], group=self.v_head_dim if self.gate_per_head else 1)
        if self.b_o is not None:
            ws.flush_pending()
            ops.add_row_vector(x_accum, self.b_o)
        stream(step).add_product(o, self.w_o, x_accum)


register_mixer("attention", Attention)
