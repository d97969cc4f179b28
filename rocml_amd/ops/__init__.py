"""Typed launch helpers over the compiled HIP libraries.

The counterpart of the reference's ``Kernels`` struct, which loads each code object
once and offers one typed method per kernel that fixes grid, block and LDS
(rocml/src/forward/kernels.rs:97-229,232-720).  Here the grid is chosen inside the
library; these helpers check devices, types and shapes, pass raw pointers and the
current stream, and turn a nonzero status into ``KernelError`` with the library's
message.  There is no fallback: a missing library is compiled, and if that fails the
call raises.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Sequence

import torch

from ..csrc import build as _build
from ..errors import KernelError

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
_LL = ctypes.c_longlong

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}

_SIGNATURES = {
    "elementwise": {
        "rocml_embed_gather": [_P, _I, _P, _P, _I, _I, _I, _F, _P, _P, _I, _P],
        "rocml_rmsnorm": [_P, _P, _P, _I, _P, _I, _I, _F, _P, _I, _LL, _P],
        "rocml_swiglu": [_P, _I, _P, _I, _I, _I, _I, _I, _F, _F, _P],
        "rocml_rope_table": [_P, _P, _P, _P, _I, _I, _F, _P],
        "rocml_qk_norm_rope_append": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _F, _P, _P, _I, _I, _P, _P, _P,
                                      _I, _P, _I, _P, _P, _I, _I, _I, _LL, _P, _I, _F, _I, _P, _I, _P],
        "rocml_qk_span_stats": [_P, _I, _I, _I, _I, _I, _P, _F, _P, _P],
        "rocml_norm_add": [_P, _P, _I, _I, _P, _P, _F, _I, _P, _I, _P, _I, _LL, _I, _P, _F, _P],
        "rocml_norm_add_branches": [_P, _P, _P, _P, _P, _F, _F, _I, _I, _P, _P, _F, _I, _P, _I, _P],
        "rocml_norm_add_branches_fits": [_I],
        "rocml_layernorm": [_P, _P, _I, _I, _P, _P, _F, _P, _I, _P],
        "rocml_token_side_gate": [_P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P, _I, _P],
        "rocml_add_into": [_P, _P, _I, _LL, _P],
        "rocml_add_row_vector": [_P, _P, _I, _I, _P],
        "rocml_latent_prepare": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _F, _P, _P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _P],
        "rocml_rope_heads": [_P, _I, _I, _I, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
        "rocml_latent_window_plan": [_P, _P, _P, _I, _I, _I, _I, _P, _I, _P, _I, _P],
        "rocml_latent_window_gather": [_P, _I, _I, _I, _P, _I, _P, _P],
        "rocml_gate_heads": [_P, _I, _I, _I, _P, _I, _P, _I, _I, _I, _P],
        "rocml_sigmoid_gate": [_P, _I, _P, _I, _I, _I, _I, _P],
        "rocml_sum_norm": [_P, _I, _I, _F, _F, _I, _P, _P, _P, _F, _P, _I, _P],
        "rocml_convert": [_P, _P, _I, _LL, _P],
        "rocml_softcap": [_P, _F, _LL, _P],
        "rocml_weighted_sum": [_P, _P, _P, _I, _F, _LL, _P],
        "rocml_row_gate_add": [_P, _P, _P, _I, _I, _I, _P],
    },
    "recurrent": {
        "rocml_causal_conv": [_P, _I, _I, _I, _I, _I, _P, _P, _P, _I, _P, _P, _P, _I, _P, _I, _P],
        "rocml_ssd_scan": [_P, _I, _P, _I, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P, _I, _I, _I, _I, _P],
        "rocml_gated_part_norm": [_P, _P, _I, _I, _P, _P, _I, _I, _I, _I, _F, _P],
        "rocml_mlstm_scan": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _F, _F, _F, _P, _P, _P, _I, _P, _P, _I, _I, _P, _I, _I, _I, _P],
        "rocml_mlstm_tile": [],
        "rocml_head_norm_gate": [_P, _P, _I, _I, _P, _P, _I, _I, _I, _I, _F, _I, _P],
        "rocml_decay_scan": [_P, _I, _I, _P, _I, _I, _P, _I, _I, _P, _I, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P, _I, _I, _I, _P],
        "rocml_rotate_rows": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _F, _I, _F, _P],
        "rocml_shift_mix": [_P, _I, _I, _I, _P, _I, _P, _I, _P, _P, _P, _I, _P, _P],
        "rocml_tanh": [_P, _P, _I, _LL, _P],
        "rocml_double_exp_decay": [_P, _P, _I, _I, _P],
    },
    "moe": {
        "rocml_moe_route": [_P, _I, _I, _I, _I, _I, _F, _P, _P, _P, _I, _P, _I, _I, _P],
        "rocml_moe_plan": [_P, _I, _I, _P, _P, _P, _P, _P, _I, _P],
        "rocml_moe_gemm": [_P, _I, _I, _I, _P, _I, _P, _P, _I, _LL, _I, _I, _P, _I, _I, _I, _I, _I, _P, _P, _P, _I, _I, _P],
        "rocml_moe_combine": [_P, _P, _P, _P, _I, _I, _I, _I, _P],
    },
    "gemm": {
        "rocml_gemm": [_P, _I, _I, _P, _I, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _LL, _P, _I, _F, _I, _P],
        "rocml_splitk_reduce": [_P, _P, _I, _I, _I, _I, _I, _I, _P],
        "rocml_gemm_batched": [_P, _I, _I, _LL, _P, _I, _I, _LL, _P, _I, _I, _LL, _I, _I, _I, _I, _P, _I, _LL, _P],
        "rocml_gemm_residual_prescale_pays": [_I, _I, _I],
        "rocml_gemm_residual_prescale": [_P, _I, _P, _I, _P, _I, _P, _P, _I, _P, _I, _I, _I, _I, _P],
    },
    "attention": {
        "rocml_attention": [_P, _P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I,
                            _P, _I, _I, _P, _I, _I, _P, _LL, _I, _I, _I, _P, _I, _P, _F, _P],
        "rocml_attention_decode_fused": [_P, _I, _I, _LL, _P, _P, _F, _P, _P, _I, _P, _P, _P, _P, _I, _P, _P,
                                         _I, _I, _I, _I, _I, _F, _I, _I, _I, _P, _LL, _P, _I, _F, _I, _P, _I, _P, _I, _P],
        "rocml_attention_prefill_fused": [_P, _I, _P, _F, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _I,
                                          _P, _I, _P, _P],
    },
    "sampling": {
        "rocml_sample": [_P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _P, _I, _P, _P],
        "rocml_argmax": [_P, _I, _I, _P, _P, _P],
    },
}

_libs: Dict[str, ctypes.CDLL] = {}


def library(family: str) -> ctypes.CDLL:
    """The family's shared library, compiled on first use if it is not there."""
    lib = _libs.get(family)
    if lib is None:
        lib = ctypes.CDLL(_build.ensure(family))
        for name, argtypes in _SIGNATURES[family].items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _I
        err = getattr(lib, f"{family}_last_error")
        err.restype = ctypes.c_char_p
        err.argtypes = []
        _libs[family] = lib
    return lib


MODEL_FAMILIES = ("elementwise", "gemm", "attention")   # what every model's step needs; sampling comes with generation,
                                                        # and a part with kernels of another family names it (``kernel_families``)


def prepare(families=tuple(_SIGNATURES)) -> None:
    """Loads the named families; those that are not built yet are compiled together first."""
    _build.build([f for f in families], force=False)
    for family in families:
        library(family)


def load_all() -> None:
    prepare()


def _check(family: str, status: int) -> None:
    if status != 0:
        msg = getattr(library(family), f"{family}_last_error")().decode("utf-8", "replace")
        raise KernelError(msg)


_cus = {}


def cu_count(device) -> int:
    """Compute units of ``device`` (256 on an MI355X, which is also the answer for a device that is
    not a GPU, where parts are built only to be counted); launch sizes are phrased in it."""
    device = torch.device(device)
    if device.type != "cuda":
        return 256
    if device not in _cus:
        _cus[device] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return _cus[device]


# The raw handle of the current device's current stream.  torch's public call builds a Stream
# object and checks the device on the way (8 us a call, a quarter of a prompt step's host time);
# the same answer comes from the two calls below in a fraction of a microsecond where torch has
# them.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
        if not t.is_contiguous():
            raise KernelError(f"kernel arguments must be contiguous, got strides {t.stride()} for shape {tuple(t.shape)}")


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported element type {t.dtype}") from None


def _want(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    if t.dtype != dtype:
        raise KernelError(f"{what} must be {dtype}, got {t.dtype}")


# ---- elementwise ---------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0,
                 pos_table: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None) -> None:
    """``out[t] = table[ids[t]] * scale`` and, with a table of positions ``[max_positions, hidden]``
    of the same type, ``+ pos_table[positions[t]]`` (not scaled)."""
    _dev(table, ids, out, pos_table, positions)
    max_pos = 0
    if pos_table is not None:
        if positions is None or positions.numel() != ids.numel() or pos_table.dtype != table.dtype \
                or pos_table.dim() != 2 or pos_table.shape[1] != table.shape[1]:
            raise KernelError("a table of positions needs one position per token and the token table's type and width")
        _want(positions, torch.int32, "positions")
        max_pos = pos_table.shape[0]
    _want(ids, torch.int32, "token ids")
    _want(out, torch.float32, "embedding output")
    vocab, hidden = table.shape
    n = ids.numel()
    if out.shape != (n, hidden):
        raise KernelError(f"embedding output is {tuple(out.shape)}, expected {(n, hidden)}")
    _check("elementwise", library("elementwise").rocml_embed_gather(
        _ptr(table), _code(table), _ptr(ids), _ptr(out), n, hidden, vocab, scale, _ptr(pos_table), _ptr(positions), max_pos,
        _stream()))


def rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None, partials: Optional[torch.Tensor] = None) -> None:
    """``partials`` ([splits, rows of x, n] float32) are split-K partial sums that belong to
    ``x``: the kernel adds them to ``x`` first (and stores the sum back unless rows are
    gathered)."""
    _dev(x, gain, out, rows, partials)
    _want(x, torch.float32, "norm input")
    _want(gain, torch.float32, "norm gain")
    n = x.shape[-1]
    if gain.numel() != n or out.shape[-1] != n:
        raise KernelError(f"norm sizes differ: input {n}, gain {gain.numel()}, output {out.shape[-1]}")
    n_rows = out.numel() // n
    if rows is not None:
        _want(rows, torch.int32, "row indices")
        if rows.numel() != n_rows:
            raise KernelError("one row index per output row is needed")
    elif x.numel() != out.numel():
        raise KernelError("norm input and output differ in size")
    n_splits, stride = 0, 0
    if partials is not None:
        _want(partials, torch.float32, "partial sums")
        if partials.dim() != 3 or partials.shape[1] * partials.shape[2] != x.numel():
            raise KernelError(f"partial sums {tuple(partials.shape)} do not fit the norm input {tuple(x.shape)}")
        n_splits, stride = partials.shape[0], x.numel()
    _check("elementwise", library("elementwise").rocml_rmsnorm(
        _ptr(x), _ptr(gain), _ptr(out), _code(out), _ptr(rows), n_rows, n, eps, _ptr(partials), n_splits,
        stride, _stream()))


GATE_ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2, "sigmoid_1702": 3}      # sigmoid_1702: g * sigmoid(1.702 g)


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, interleaved: bool = False, activation: str = "silu",
           limit: Optional[float] = None, up_offset: float = 0.0) -> None:
    """``out = act(gate) * (up + up_offset)``.  ``gate_up`` rows hold the gate half then the up half, or
    (gate, up) pairs when ``interleaved``; ``activation`` is one of ``GATE_ACTIVATIONS``.  ``limit``:
    the gate is cut off above at ``limit`` and the up value is held inside ``[-limit, limit]`` first."""
    if limit is not None and not limit > 0:
        raise KernelError(f"the limit of a gated activation must be positive, got {limit}")
    if activation not in GATE_ACTIVATIONS:
        raise KernelError(f"unknown activation {activation!r}; known: {sorted(GATE_ACTIVATIONS)}")
    _dev(gate_up, out)
    n_tokens, inter = out.shape
    if gate_up.shape != (n_tokens, 2 * inter):
        raise KernelError(f"gate/up is {tuple(gate_up.shape)}, expected {(n_tokens, 2 * inter)}")
    _check("elementwise", library("elementwise").rocml_swiglu(
        _ptr(gate_up), _code(gate_up), _ptr(out), _code(out), n_tokens, inter, 1 if interleaved else 0,
        GATE_ACTIVATIONS[activation], 0.0 if limit is None else float(limit), float(up_offset), _stream()))


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
               scale: float = 1.0) -> None:
    """``cos[t, i] = scale * cos(positions[t] * inv_freq[i])`` and the sines likewise (angles in 64-bit)."""
    _dev(positions, inv_freq, cos, sin)
    _want(positions, torch.int32, "positions")
    _want(inv_freq, torch.float64, "inverse frequencies")
    _want(cos, torch.float32, "cos table")
    _want(sin, torch.float32, "sin table")
    n, half = positions.numel(), inv_freq.numel()
    if cos.shape != (n, half) or sin.shape != (n, half):
        raise KernelError(f"rotation tables must be {(n, half)}")
    _check("elementwise", library("elementwise").rocml_rope_table(
        _ptr(positions), _ptr(inv_freq), _ptr(cos), _ptr(sin), n, half, float(scale), _stream()))


ROPE_PAIRINGS = {"halves": 0, "neighbours": 1}


def qk_norm_rope_append(qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                        q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                        cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot_dim: int,
                        q_out: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                        v_cache: Optional[torch.Tensor], block_table: Optional[torch.Tensor],
                        token_seq: torch.Tensor, token_pos: torch.Tensor, write_kv: bool = True,
                        n_splits: int = 1, pairing: str = "halves", bias: Optional[torch.Tensor] = None,
                        v_head_dim: Optional[int] = None, q_temp=None, span_inv: Optional[torch.Tensor] = None,
                        span_self: bool = False) -> None:
    """``qkv`` is ``[T, ld]`` with q, k, v side by side (k and v may be absent when
    ``write_kv`` is false).  Keys are ``[pages, Hkv, page_size, D]``, values
    ``[pages, Hkv, D, page_size]``.  ``pairing``: which two values of the rotated width turn
    together by the angle in column ``i`` of the tables: ``"halves"``, ``(i, i + rot_dim / 2)``,
    or ``"neighbours"``, ``(2 i, 2 i + 1)``.  ``q_out`` None: only keys and values are prepared
    and appended (the caller's attention kernel prepares its queries itself).  ``bias``: 32-bit,
    one number per column of ``qkv``, added to the projection's sums.  ``v_head_dim``: the size of a
    value head when it is not ``head_dim`` (the value columns then follow the ``Hq + Hkv`` heads of
    ``head_dim``).  ``q_temp``: ``(coef, every)``; the query at position ``p`` is multiplied by
    ``1 + coef * ln(floor((p + 1) / every) + 1)`` after its norm.  ``span_inv``: ``[T, 2]`` 32-bit, the
    factors of a norm over a token's whole q row and whole k row (``qk_span_stats``); the gains then
    have one number per column of the q and of the k projection.  ``span_self``: the same norm, its
    factors formed inside the kernel (for steps of few tokens)."""
    qt_coef, qt_every = (0.0, 0) if q_temp is None else (float(q_temp[0]), int(q_temp[1]))
    if q_temp is not None and qt_every <= 0:
        raise KernelError(f"the period of the query's stretch must be positive, got {qt_every}")
    dv = head_dim if v_head_dim is None else int(v_head_dim)
    if pairing not in ROPE_PAIRINGS:
        raise KernelError(f"unknown rotation pairing {pairing!r}; known: {sorted(ROPE_PAIRINGS)}")
    _dev(qkv, q_gain, k_gain, cos, sin, q_out, k_cache, v_cache, block_table, token_seq, token_pos, bias, span_inv)
    split_stride = 0
    if n_splits > 1:                      # [splits, T, ld] split-K partial sums, added in the kernel
        if qkv.dim() != 3 or qkv.shape[0] != n_splits:
            raise KernelError("partial sums of the projection must be [splits, tokens, width]")
        split_stride = qkv.shape[1] * qkv.shape[2]
        qkv = qkv[0]
    n_tokens, ld = qkv.shape
    if bias is not None:
        _want(bias, torch.float32, "projection bias")
        # (rows may be wider than the projection: a product shared with other mixers, whose columns follow)
        if bias.numel() > ld or bias.numel() < n_heads * head_dim + (n_kv_heads * (head_dim + dv) if write_kv else 0):
            raise KernelError(f"the bias has {bias.numel()} values for rows of {ld}")
    whole = span_inv is not None or span_self
    if span_inv is not None:
        _want(span_inv, torch.float32, "norm factors")
        if span_inv.shape != (n_tokens, 2) or span_self:
            raise KernelError("the factors of a norm over the whole projection are [tokens, 2], or formed by the kernel itself")
    if whole and (n_splits > 1 or q_gain is None or k_gain is None or not write_kv):
        raise KernelError("a norm over the whole projection needs a complete projection with its k columns and both gains")
    for g, heads in ((q_gain, n_heads), (k_gain, n_kv_heads)):
        if g is not None:
            _want(g, torch.float32, "head norm gain")
            if g.numel() != (heads * head_dim if whole else head_dim):
                raise KernelError(f"norm gain has {g.numel()} values for {heads} heads of size {head_dim}")
    if cos is not None:
        if cos.shape != (n_tokens, rot_dim // 2) or sin is None or sin.shape != cos.shape:
            raise KernelError(f"rotation tables must be {(n_tokens, rot_dim // 2)}")
    if q_out is None and not write_kv:
        raise KernelError("nothing to do: no q output and no append to the cache")
    if (q_out is not None and q_out.shape != (n_tokens, n_heads * head_dim)) or token_seq.numel() != n_tokens \
            or token_pos.numel() != n_tokens:
        raise KernelError("q output or token tables do not match the number of tokens")
    page_size = bt_width = 0
    if write_kv:
        if k_cache is None or v_cache is None or block_table is None:
            raise KernelError("appending to the cache needs the cache and the block table")
        if k_cache.shape[1:] != (n_kv_heads, k_cache.shape[2], head_dim) \
                or v_cache.shape != (k_cache.shape[0], n_kv_heads, dv, k_cache.shape[2]):
            raise KernelError(f"cache shape {tuple(k_cache.shape)} does not fit {n_kv_heads} heads of {head_dim}")
        if q_out is not None and k_cache.dtype != q_out.dtype:
            raise KernelError("cache and q output must share their type")
        _want(block_table, torch.int32, "block table")
        page_size, bt_width = k_cache.shape[2], block_table.shape[1]
    _check("elementwise", library("elementwise").rocml_qk_norm_rope_append(
        _ptr(qkv), _code(qkv), ld, n_tokens, n_heads, n_kv_heads, head_dim, _ptr(q_gain), _ptr(k_gain),
        eps, _ptr(cos), _ptr(sin), rot_dim if cos is not None else 0, ROPE_PAIRINGS[pairing], _ptr(q_out), _ptr(k_cache),
        _ptr(v_cache), _code(q_out if q_out is not None else k_cache), _ptr(block_table), bt_width, _ptr(token_seq),
        _ptr(token_pos), page_size, 1 if write_kv else 0, n_splits, split_stride, _ptr(bias), dv, qt_coef, qt_every,
        _ptr(span_inv), 1 if span_self else 0, _stream()))


def qk_span_stats(qkv: torch.Tensor, q_width: int, k_width: int, bias: Optional[torch.Tensor], eps: float,
                  out: torch.Tensor) -> None:
    """``out[t, 0] = 1 / sqrt(mean((qkv[t, :q_width] + bias)^2) + eps)`` and ``out[t, 1]`` the same over the
    ``k_width`` columns behind them: the factors of a norm over a token's whole q row and whole k row."""
    _dev(qkv, bias, out)
    _want(out, torch.float32, "norm factors")
    if qkv.dim() != 2 or out.shape != (qkv.shape[0], 2) or qkv.shape[1] < q_width + k_width:
        raise KernelError("qk_span_stats: shapes do not fit")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() < q_width + k_width):
        raise KernelError("qk_span_stats: the bias must be 32-bit and cover the q and k columns")
    _check("elementwise", library("elementwise").rocml_qk_span_stats(
        _ptr(qkv), _code(qkv), qkv.shape[1], qkv.shape[0], q_width, k_width, _ptr(bias), float(eps), _ptr(out), _stream()))


def norm_add(x: torch.Tensor, y: torch.Tensor, gain: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
             layer: bool, copy: Optional[torch.Tensor] = None, partials: Optional[torch.Tensor] = None,
             replace: bool = False, next_gain: Optional[torch.Tensor] = None, next_eps: float = 0.0) -> None:
    """``x += f(y)`` row by row in 32-bit: ``f`` a layer norm ``(y - mean) / sqrt(var + eps) * gain + bias``
    (``layer``) or ``y / sqrt(mean(y^2) + eps) * gain``.  ``copy`` gets the new ``x`` in its own type.
    ``partials`` (``[splits, rows, n]`` 32-bit): the K pieces of the product that made ``y``, added to ``y`` in
    split order first, or with ``replace`` all of ``y`` (what ``y`` holds is not read).  ``next_gain`` (with ``copy``):
    ``copy`` gets the root-mean-square norm of the new ``x`` instead, ``x / sqrt(mean(x^2) + next_eps) * next_gain``: the
    norm that reads the stream next."""
    _dev(x, y, gain, bias, copy, partials, next_gain)
    if next_gain is not None and (copy is None or next_gain.dtype != torch.float32 or next_gain.numel() != x.shape[1]):
        raise KernelError("norm_add: the next norm needs a 32-bit gain of the row's size and a place for its output")
    n_splits = split_stride = 0
    if partials is not None:
        _want(partials, torch.float32, "partial sums")
        if partials.dim() != 3 or tuple(partials.shape[1:]) != tuple(x.shape):
            raise KernelError("norm_add: partial sums must be [splits, rows, n]")
        n_splits, split_stride = partials.shape[0], x.numel()
    elif replace:
        raise KernelError("norm_add: nothing to replace the sublayer's output with")
    for t, what in ((x, "residual stream"), (y, "sublayer output"), (gain, "norm gain")):
        _want(t, torch.float32, what)
    if x.dim() != 2 or y.shape != x.shape or gain.numel() != x.shape[1] or (copy is not None and copy.shape != x.shape) \
            or (bias is not None and (bias.dtype != torch.float32 or bias.numel() != x.shape[1])):
        raise KernelError("norm_add: shapes do not fit")
    _check("elementwise", library("elementwise").rocml_norm_add(
        _ptr(x), _ptr(y), x.shape[0], x.shape[1], _ptr(gain), _ptr(bias), float(eps), 1 if layer else 0, _ptr(copy),
        _code(copy) if copy is not None else 0, _ptr(partials), n_splits, split_stride, 1 if replace else 0, _ptr(next_gain),
        float(next_eps), _stream()))


def norm_add_branches_fits(n: int, n_branches: int) -> bool:
    """Whether ``norm_add_branches`` takes rows of ``n`` values in ``n_branches`` branches."""
    return 1 <= n_branches <= 2 and bool(library("elementwise").rocml_norm_add_branches_fits(int(n)))


def norm_add_branches(x: torch.Tensor, branches: Sequence[torch.Tensor], branch_gains: Sequence[torch.Tensor], weight: float,
                      branch_eps: float, gain: torch.Tensor, bias: Optional[torch.Tensor], eps: float, layer: bool,
                      copy: Optional[torch.Tensor] = None) -> None:
    """``x += f(weight * sum_b rms(y_b) * gain_b)`` row by row in 32-bit for one or two branches ``y_b``, each divided by
    its own root mean square (``branch_eps`` inside the root) first; ``f`` as in ``norm_add``."""
    _dev(x, gain, bias, copy, *branches, *branch_gains)
    if not norm_add_branches_fits(x.shape[1], len(branches)) or len(branch_gains) != len(branches):
        raise KernelError(f"norm_add_branches takes one or two branches of rows it can keep in registers, got {len(branches)} of {x.shape[1]}")
    for t in (x, gain, *branches, *branch_gains):
        _want(t, torch.float32, "stream, branches and gains")
    n = x.shape[1]
    if any(y.shape != x.shape for y in branches) or any(g.numel() != n for g in branch_gains) or gain.numel() != n \
            or (bias is not None and (bias.dtype != torch.float32 or bias.numel() != n)) or (copy is not None and copy.shape != x.shape):
        raise KernelError("norm_add_branches: shapes do not fit")
    y1 = branches[1] if len(branches) > 1 else None
    g1 = branch_gains[1] if len(branches) > 1 else None
    _check("elementwise", library("elementwise").rocml_norm_add_branches(
        _ptr(x), _ptr(branches[0]), _ptr(y1), _ptr(branch_gains[0]), _ptr(g1), float(weight), float(branch_eps), x.shape[0], n,
        _ptr(gain), _ptr(bias), float(eps), 1 if layer else 0, _ptr(copy), _code(copy) if copy is not None else 0, _stream()))


def layernorm(x: torch.Tensor, gain: torch.Tensor, bias: Optional[torch.Tensor], eps: float, out: torch.Tensor,
              rows: Optional[torch.Tensor] = None) -> None:
    """``out[r] = (x[s] - mean) / sqrt(var + eps) * gain + bias`` with ``s = rows[r]`` (or ``r``), ``var`` the
    mean of the squared deviations; 32-bit ``x``, statistics 32-bit."""
    _dev(x, gain, bias, out, rows)
    _want(x, torch.float32, "norm input")
    _want(gain, torch.float32, "norm gain")
    n = x.shape[1]
    n_out = out.shape[0]
    if rows is not None:
        _want(rows, torch.int32, "row indices")
        if rows.numel() < n_out:
            raise KernelError("layernorm: fewer row indices than output rows")
    elif n_out != x.shape[0]:
        raise KernelError("layernorm: output rows differ from input rows")
    if out.shape[1] != n or gain.numel() != n or (bias is not None and (bias.dtype != torch.float32 or bias.numel() != n)):
        raise KernelError("layernorm: widths differ")
    _check("elementwise", library("elementwise").rocml_layernorm(
        _ptr(x), _ptr(rows), n_out, n, _ptr(gain), _ptr(bias), float(eps), _ptr(out), _code(out), _stream()))


SIDE_ACTIVATIONS = {"gelu_tanh": 0, "identity": 1}


def token_side_gate(g: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, col0: int, out: torch.Tensor,
                    activation: str = "gelu_tanh") -> None:
    """``out[t, j] = act(g[t, j]) * table[ids[t], col0 + j]`` for the 32-bit ``g [T, dim]``."""
    _dev(g, table, ids, out)
    _want(g, torch.float32, "gate")
    _want(ids, torch.int32, "token ids")
    if activation not in SIDE_ACTIVATIONS:
        raise KernelError(f"unknown activation {activation!r}; known: {sorted(SIDE_ACTIVATIONS)}")
    n, dim = g.shape
    if out.shape != g.shape or ids.numel() != n or table.dim() != 2 or col0 < 0 or col0 + dim > table.shape[1]:
        raise KernelError("token_side_gate: shapes do not fit")
    _check("elementwise", library("elementwise").rocml_token_side_gate(
        _ptr(g), _ptr(table), _code(table), _ptr(ids), n, table.shape[1], col0, dim, table.shape[0],
        SIDE_ACTIVATIONS[activation], _ptr(out), _code(out), _stream()))


def add_row_vector(x: torch.Tensor, b: torch.Tensor) -> None:
    """``x[t, :] += b`` for the 32-bit ``x [T, n]`` and ``b [n]``."""
    _dev(x, b)
    _want(x, torch.float32, "residual stream")
    _want(b, torch.float32, "row vector")
    if x.dim() != 2 or b.numel() != x.shape[1]:
        raise KernelError(f"a vector of {b.numel()} numbers does not fit rows of {tuple(x.shape)}")
    _check("elementwise", library("elementwise").rocml_add_row_vector(_ptr(x), _ptr(b), x.shape[0], x.shape[1], _stream()))


def latent_prepare(proj: torch.Tensor, q_rank: int, kv_rank: int, rot_part: int, rot_dims: int,
                   q_gain: torch.Tensor, kv_gain: torch.Tensor, eps: float, cos: Optional[torch.Tensor],
                   sin: Optional[torch.Tensor], cq_out: torch.Tensor, cache: Optional[torch.Tensor],
                   block_table: Optional[torch.Tensor], token_seq: torch.Tensor, token_pos: torch.Tensor,
                   write_cache: bool = True) -> None:
    """What follows a latent attention's first projection.  A row of ``proj`` (32-bit) holds the
    query latent (``q_rank``), the key/value latent (``kv_rank``) and the shared rotated key part
    (``rot_part``, of which the first ``rot_dims`` turn in pairs ``(i, i + rot_dims/2)``).  Both
    latents get their root-mean-square norm; the query latent goes to ``cq_out [T, q_rank]``, the
    other two into the token's row of ``cache [pages, page_size, kv_rank + rot_part]``."""
    _dev(proj, q_gain, kv_gain, cos, sin, cq_out, cache, block_table, token_seq, token_pos)
    _want(proj, torch.float32, "projection output")
    _want(q_gain, torch.float32, "latent norm gain")
    _want(kv_gain, torch.float32, "latent norm gain")
    n_tokens, ld = proj.shape
    if q_gain.numel() != q_rank or kv_gain.numel() != kv_rank or cq_out.shape != (n_tokens, q_rank):
        raise KernelError("latent gains or the query latent's output do not fit the ranks")
    if rot_dims:
        if cos is None or sin is None or cos.shape != (n_tokens, rot_dims // 2) or sin.shape != cos.shape \
                or cos.dtype != torch.float32 or sin.dtype != torch.float32:
            raise KernelError(f"rotation tables must be float32 {(n_tokens, rot_dims // 2)}")
    page_size = bt_width = 0
    if write_cache:
        if cache is None or block_table is None:
            raise KernelError("appending to the cache needs the cache and the block table")
        if cache.dim() != 3 or cache.shape[2] != kv_rank + rot_part or cache.dtype != cq_out.dtype:
            raise KernelError(f"latent cache {tuple(cache.shape)} {cache.dtype} does not fit rows of {kv_rank + rot_part}")
        _want(block_table, torch.int32, "block table")
        page_size, bt_width = cache.shape[1], block_table.shape[1]
    _want(token_seq, torch.int32, "token sequence table")
    _want(token_pos, torch.int32, "token position table")
    if token_seq.numel() != n_tokens or token_pos.numel() != n_tokens:
        raise KernelError("one sequence index and one position per token are needed")
    _check("elementwise", library("elementwise").rocml_latent_prepare(
        _ptr(proj), ld, n_tokens, q_rank, kv_rank, rot_part, rot_dims, _ptr(q_gain), _ptr(kv_gain), eps, _ptr(cos),
        _ptr(sin), _ptr(cq_out), _ptr(cache), _code(cq_out), _ptr(block_table), bt_width, _ptr(token_seq),
        _ptr(token_pos), page_size, 1 if write_cache else 0, _stream()))


def rope_heads(q: torch.Tensor, n_heads: int, head_stride: int, offset: int, rot_part: int, rot_dims: int,
               cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], out: torch.Tensor, out_stride: int,
               out_offset: int, lead: int = 0) -> None:
    """The part of every head of ``q [T, n_heads * head_stride]`` (32-bit) that starts at ``offset``
    and is ``rot_part`` wide, rotated (its first ``rot_dims`` numbers, pairs ``(i, i + rot_dims/2)``),
    written to ``out [T, n_heads * out_stride]`` at ``out_offset`` of every head.  ``lead``: so many
    numbers before the part are copied unchanged in front of it (``out_offset`` is where they start)."""
    _dev(q, cos, sin, out)
    _want(q, torch.float32, "queries")
    n_tokens = q.shape[0]
    if q.dim() != 2 or out.dim() != 2 or out.shape[0] != n_tokens:
        raise KernelError("queries and output must be [tokens, width]")
    if rot_dims and (cos is None or sin is None or cos.shape != (n_tokens, rot_dims // 2) or sin.shape != cos.shape
                     or cos.dtype != torch.float32 or sin.dtype != torch.float32):
        raise KernelError(f"rotation tables must be float32 {(n_tokens, rot_dims // 2)}")
    _check("elementwise", library("elementwise").rocml_rope_heads(
        _ptr(q), q.shape[1], head_stride, offset, rot_part, rot_dims, _ptr(cos), _ptr(sin), _ptr(out), _code(out),
        out.shape[1], out_stride, out_offset, n_tokens, n_heads, int(lead), _stream()))


def latent_window_plan(cu_seqlens: torch.Tensor, token_pos: torch.Tensor, block_table: torch.Tensor, window: Optional[int],
                       page_size: int, table: torch.Tensor, plan: torch.Tensor) -> None:
    """For a prompt step over a cache of rows per position: which pages hold the positions the step's
    queries see (per sequence its new tokens and up to ``window - 1`` before them; all without a
    window), numbered as scratch pages in sequence order.  Writes ``table [sequences, width]``
    (a sequence's page index -> scratch page, -1 elsewhere) and ``plan [4, max_pages]`` int32: per
    scratch page the pool page it mirrors (-1: unused), its first position, and the first and one past
    the last position that count."""
    _dev(cu_seqlens, token_pos, block_table, table, plan)
    for t, name in ((cu_seqlens, "sequence offsets"), (token_pos, "token positions"), (block_table, "block table"),
                    (table, "scratch table"), (plan, "plan")):
        _want(t, torch.int32, name)
    n_seqs = cu_seqlens.numel() - 1
    if table.dim() != 2 or table.shape[0] != n_seqs or plan.dim() != 2 or plan.shape[0] != 4 or block_table.shape[0] < n_seqs:
        raise KernelError("the scratch table must be [sequences, width] and the plan [4, pages]")
    _check("elementwise", library("elementwise").rocml_latent_window_plan(
        _ptr(cu_seqlens), _ptr(token_pos), _ptr(block_table), block_table.shape[1], n_seqs, 0 if window is None else int(window),
        page_size, _ptr(table), table.shape[1], _ptr(plan), plan.shape[1], _stream()))


def latent_window_gather(cache: torch.Tensor, plan: torch.Tensor, out: torch.Tensor) -> None:
    """The rows ``latent_window_plan`` planned, ``cache [pages, page_size, row]`` -> ``out [max_pages *
    page_size, row]`` in scratch-page order, zeros where a position does not count."""
    _dev(cache, plan, out)
    _want(plan, torch.int32, "plan")
    pages, page_size, row = cache.shape
    if out.dtype != cache.dtype or out.shape != (plan.shape[1] * page_size, row):
        raise KernelError(f"gathered rows must be {(plan.shape[1] * page_size, row)} of the cache's type")
    _check("elementwise", library("elementwise").rocml_latent_window_gather(
        _ptr(cache), _code(cache), row, page_size, _ptr(plan), plan.shape[1], _ptr(out), _stream()))


def gate_heads(x: torch.Tensor, x_stride: int, gate: Optional[torch.Tensor], out: torch.Tensor, n_heads: int, n: int) -> None:
    """``out[t, h * n + i] = x[t, h * x_stride + i] * sigmoid(gate[t, h * n + i])`` (``gate`` None: the
    plain copy): the leading ``n`` numbers of every head of ``x``, gated and packed."""
    _dev(x, out)
    if gate is not None and (not gate.is_cuda or gate.dtype != torch.float32 or gate.stride(1) != 1 or gate.shape != out.shape):
        raise KernelError("the gate must be 32-bit and of the output's shape")
    if x.dtype != out.dtype or out.shape != (x.shape[0], n_heads * n) or x.shape[1] < n_heads * x_stride:
        raise KernelError("gate_heads: shapes do not fit")
    ldg = 0 if gate is None else (gate.stride(0) if x.shape[0] > 1 else max(gate.stride(0), gate.shape[1]))
    _check("elementwise", library("elementwise").rocml_gate_heads(
        _ptr(x), _code(x), x.shape[1], x_stride, _ptr(gate), ldg, _ptr(out), x.shape[0], n_heads, n, _stream()))


def sigmoid_gate(y: torch.Tensor, gate: torch.Tensor, group: int = 1) -> None:
    """``y *= sigmoid(gate)`` for ``y [T, n]`` and the 32-bit ``gate [T, n / group]``, whose rows may be a
    column range of a wider matrix; a gate value covers ``group`` neighbouring values of ``y`` (a head)."""
    _dev(y)
    if not gate.is_cuda:
        raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
    _want(gate, torch.float32, "gate")
    if y.dim() != 2 or group <= 0 or y.shape[1] % group != 0 or gate.shape != (y.shape[0], y.shape[1] // group) \
            or gate.stride(1) != 1:
        raise KernelError(f"gate {tuple(gate.shape)} does not fit {tuple(y.shape)} in groups of {group}")
    ldg = gate.stride(0) if y.shape[0] > 1 else max(gate.stride(0), gate.shape[1])
    _check("elementwise", library("elementwise").rocml_sigmoid_gate(_ptr(y), _code(y), _ptr(gate), ldg, y.shape[0],
                                                                   y.shape[1], group, _stream()))


def sum_norm(x: torch.Tensor, branches: Sequence[torch.Tensor], branch_gains: Sequence[Optional[torch.Tensor]],
             gain: Optional[torch.Tensor], eps: float, alpha: float = 1.0, weight: float = 1.0,
             copy: Optional[torch.Tensor] = None) -> None:
    """``x <- rms(alpha * x + weight * sum_b f_b(y_b)) * gain`` in place (32-bit; without ``gain`` the
    sum itself, and with ``alpha`` zero ``x`` is only written), where
    ``f_b(y) = rms(y) * gain_b`` for a branch with a gain and ``y`` itself for one without;
    ``rms(v) = v / sqrt(mean(v^2) + eps)``.  ``copy`` gets the new ``x`` in its own type."""
    _dev(x, gain, copy, *branches, *[g for g in branch_gains if g is not None])
    _want(x, torch.float32, "residual stream")
    if gain is not None:
        _want(gain, torch.float32, "norm gain")
    rows, n = x.shape
    if not 1 <= len(branches) <= 4 or len(branch_gains) != len(branches):
        raise KernelError("sum_norm takes one to four branches and a gain (or None) for each")
    for y, g in zip(branches, branch_gains):
        _want(y, torch.float32, "a branch's output")
        if y.shape != x.shape or (g is not None and (g.dtype != torch.float32 or g.numel() != n)):
            raise KernelError(f"a branch is {tuple(y.shape)} for a stream of {tuple(x.shape)}, or its gain does not fit")
    if (gain is not None and gain.numel() != n) or (copy is not None and copy.shape != x.shape):
        raise KernelError("sum_norm: gain or copy do not fit the stream")
    ys = (ctypes.c_void_p * len(branches))(*[y.data_ptr() for y in branches])
    gs = (ctypes.c_void_p * len(branches))(*[None if g is None else g.data_ptr() for g in branch_gains])
    _check("elementwise", library("elementwise").rocml_sum_norm(
        _ptr(x), rows, n, float(alpha), float(weight), len(branches), ys, gs, _ptr(gain), float(eps), _ptr(copy),
        _code(copy) if copy is not None else 0, _stream()))


def convert(x: torch.Tensor, out: torch.Tensor) -> None:
    """``out = x`` in ``out``'s type, for 32-bit ``x``."""
    _dev(x, out)
    _want(x, torch.float32, "the values to copy")
    if x.numel() != out.numel():
        raise KernelError("convert: sizes differ")
    _check("elementwise", library("elementwise").rocml_convert(_ptr(x), _ptr(out), _code(out), x.numel(), _stream()))


def softcap(x: torch.Tensor, cap: float) -> None:
    """``x <- cap * tanh(x / cap)`` in place, 32-bit."""
    _dev(x)
    _want(x, torch.float32, "the values to cap")
    _check("elementwise", library("elementwise").rocml_softcap(_ptr(x), float(cap), x.numel(), _stream()))


def weighted_sum(out: torch.Tensor, branches: Sequence[torch.Tensor], weights: Sequence[float], alpha: float = 0.0) -> None:
    """``out <- alpha * out + sum_b weights[b] * branches[b]``, all 32-bit and of one shape."""
    _dev(out, *branches)
    if not 1 <= len(branches) <= 4 or len(weights) != len(branches):
        raise KernelError("weighted_sum takes one to four branches and a weight for each")
    for y in (out, *branches):
        _want(y, torch.float32, "a summand")
        if y.shape != out.shape:
            raise KernelError("weighted_sum: shapes differ")
    ys = (ctypes.c_void_p * len(branches))(*[y.data_ptr() for y in branches])
    ws = (ctypes.c_float * len(branches))(*[float(w) for w in weights])
    _check("elementwise", library("elementwise").rocml_weighted_sum(_ptr(out), ys, ws, len(branches), float(alpha), out.numel(),
                                                                   _stream()))


def row_gate_add(x: torch.Tensor, y: torch.Tensor, gate: torch.Tensor) -> None:
    """``x[t] += sigmoid(gate[t]) * y[t]`` for 32-bit ``x``, ``y [T, n]`` and one 32-bit gate logit per row (a column
    of a matrix: ``gate [T, 1]`` with any row stride)."""
    _dev(x, y)
    if not gate.is_cuda:
        raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
    for t, what in ((x, "the stream"), (y, "the summand"), (gate, "the gate")):
        _want(t, torch.float32, what)
    rows, n = x.shape
    if y.shape != x.shape or gate.dim() != 2 or gate.shape != (rows, 1):
        raise KernelError("row_gate_add: sizes differ")
    _check("elementwise", library("elementwise").rocml_row_gate_add(_ptr(x), _ptr(y), _ptr(gate), max(gate.stride(0), 1), rows, n,
                                                                   _stream()))


def add_into(x: torch.Tensor, y: torch.Tensor) -> None:
    _dev(x, y)
    _want(x, torch.float32, "residual")
    if x.numel() != y.numel():
        raise KernelError("residual add of different sizes")
    _check("elementwise", library("elementwise").rocml_add_into(_ptr(x), _ptr(y), _code(y), x.numel(), _stream()))


# ---- matrix product ------------------------------------------------------------------
GEMM_AUTO, GEMM_PLAIN = 0, 1
# epilogues of a product whose weight rows are (gate, up) pairs: act(gate) * up
GEMM_EPILOGUES = {None: 0, "swiglu": 1, "relu_glu": 2}
ROW_SCALE_MAX_ROWS = 16     # most rows of a product whose consumer applies a row scale


class RowScale:
    """What is left of a norm whose operand ``bfloat16(x * gain)`` was prepared by the product that
    completed ``x`` (``gemm_residual_prescale``): ``ssq [rows, parts]`` float32 sums of squares
    whose total over a row, divided by ``width`` and with ``eps`` added, is the square of what the
    row still has to be divided by.  The consumer of the next product applies it to its sums."""

    def __init__(self, ssq: torch.Tensor, eps: float, width: int):
        _dev(ssq)
        _want(ssq, torch.float32, "sums of squares")
        if ssq.dim() != 2:
            raise KernelError("sums of squares must be [rows, parts]")
        self.ssq, self.eps, self.width = ssq, float(eps), int(width)


def gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         algo: int = GEMM_AUTO, workspace: Optional[torch.Tensor] = None, epilogue: Optional[str] = None,
         defer: bool = False, row_scale: Optional["RowScale"] = None, max_splits: int = 0) -> int:
    """``out (+)= x @ w.T`` for ``x [M, K]``, ``w [N, K]``, ``out [M, N]`` (rows may be
    strided views with unit inner stride).  ``epilogue="swiglu"``: ``w``'s rows are (gate, up)
    pairs and ``out`` is ``[M, N/2] = silu(gate) * up``.  With ``defer`` a product that was
    split along K leaves its partial sums ``[splits, M, N]`` at the start of ``workspace`` and
    returns their number for the caller's next kernel to add; it returns 0 when ``out`` is
    complete.  ``row_scale``: ``x`` lacks its norm's scale (see ``RowScale``), which the gated
    epilogue applies; at most ``ROW_SCALE_MAX_ROWS`` rows.  ``max_splits``: the most pieces K may
    be cut into (0: as the kernels see fit)."""
    for t in (x, w, out):
        if not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
        if t.dim() != 2 or t.stride(1) != 1:
            raise KernelError("matrix product operands must be 2-D with unit inner stride")
    if epilogue not in GEMM_EPILOGUES:
        raise KernelError(f"unknown epilogue {epilogue!r}")
    m, k = x.shape
    n = w.shape[0]
    cols = n // 2 if epilogue else n
    if w.shape[1] != k or out.shape != (m, cols):
        raise KernelError(f"matrix product shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    ws_ptr, ws_bytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    deferred = ctypes.c_int(0)
    ssq_ptr, parts, eps = None, 0, 0.0
    if row_scale is not None:
        if epilogue is None or m > ROW_SCALE_MAX_ROWS or row_scale.width != k or row_scale.ssq.shape[0] < m:
            raise KernelError("a row scale goes with the gated epilogue of at most 16 rows whose K is the norm's width")
        ssq_ptr, parts, eps = row_scale.ssq.data_ptr(), row_scale.ssq.shape[1], row_scale.eps
    _check("gemm", library("gemm").rocml_gemm(
        _ptr(x), _code(x), x.stride(0) if m > 1 else max(x.stride(0), k), _ptr(w), _code(w), w.stride(0),
        _ptr(out), _code(out), out.stride(0) if m > 1 else max(out.stride(0), cols), m, n, k,
        1 if accumulate else 0, algo, GEMM_EPILOGUES[epilogue], 1 if defer else 0, ctypes.byref(deferred), ws_ptr,
        ws_bytes, ssq_ptr, parts, eps, int(max_splits), _stream()))
    return deferred.value


def gemm_batched_gate_fusable(w: torch.Tensor, x: torch.Tensor) -> bool:
    """Whether ``gemm_batched`` can apply an output gate itself (its matrix-core kernel runs)."""
    return (w.dtype == torch.bfloat16 and w.shape[2] % 8 == 0 and x.shape[1] % (4 if x.dtype == torch.float32 else 8) == 0)


def gemm_batched(x: torch.Tensor, x_head_stride: int, w: torch.Tensor, out: torch.Tensor, out_head_stride: int,
                 gate: Optional[torch.Tensor] = None) -> None:
    """One small product per head: ``out[:, h * out_head_stride : ... + N] = x[:, h * x_head_stride :
    ... + K] @ w[h].T`` for ``w [heads, N, K]``; ``x`` and ``out`` are ``[tokens, width]`` matrices
    that hold the heads side by side.  32-bit accumulation; ``x`` may be 32-bit with bfloat16 weights.
    ``gate`` (32-bit ``[tokens, heads * N]``, rows may be a column range of a wider matrix): the
    product is multiplied by ``sigmoid(gate)``; only where ``gemm_batched_gate_fusable``."""
    _dev(x, w, out)
    ldg = g_stride = 0
    if gate is not None:
        if not gate.is_cuda or gate.dtype != torch.float32 or gate.stride(1) != 1 or gate.shape != (x.shape[0], w.shape[0] * w.shape[1]) \
                or out_head_stride != w.shape[1] or not gemm_batched_gate_fusable(w, x) or x_head_stride % 4:
            raise KernelError("the gate must be 32-bit [tokens, heads * N] for an output without gaps, on the matrix-core kernel")
        ldg, g_stride = (gate.stride(0) if x.shape[0] > 1 else max(gate.stride(0), gate.shape[1])), w.shape[1]
    if x.dim() != 2 or out.dim() != 2 or w.dim() != 3 or x.shape[0] != out.shape[0]:
        raise KernelError("gemm_batched takes x [T, width], w [heads, N, K], out [T, width]")
    heads, n, k = w.shape
    if (heads - 1) * x_head_stride + k > x.shape[1] or (heads - 1) * out_head_stride + n > out.shape[1]:
        raise KernelError(f"{heads} heads of K={k} / N={n} do not fit rows of {x.shape[1]} / {out.shape[1]}")
    _check("gemm", library("gemm").rocml_gemm_batched(
        _ptr(x), _code(x), x.shape[1], x_head_stride, _ptr(w), _code(w), k, n * k, _ptr(out), _code(out),
        out.shape[1], out_head_stride, heads, x.shape[0], n, k, _ptr(gate), ldg, g_stride, _stream()))


PRESCALE_MAX_ROWS = 16      # most rows gemm_residual_prescale takes
PRESCALE_TILE = 16          # columns whose squares one entry of its sums of squares covers


def gemm_residual_prescale_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_residual_prescale`` takes this product."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 1 <= x.shape[0] <= PRESCALE_MAX_ROWS
            and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0)


def gemm_residual_prescale_pays(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether it takes the product and is the faster way (the library's own rule)."""
    return gemm_residual_prescale_fits(x, w) and \
        library("gemm").rocml_gemm_residual_prescale_pays(x.shape[0], w.shape[0], x.shape[1]) != 0


def gemm_residual_prescale(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, gain: torch.Tensor,
                           xg: torch.Tensor, ssq: torch.Tensor, waves: int = 0) -> None:
    """``resid += x @ w.T`` (whole sums, at most 16 rows of bfloat16 operands) and, for the norm
    with ``gain`` that reads ``resid`` next: ``xg = bfloat16(resid * gain)`` and ``ssq[row][j]`` =
    the sum of squares of columns ``16 j .. 16 j + 15`` of the row.  The norm's output is
    ``xg * (1 / sqrt(ssq[row].sum() / N + eps))``; the scale commutes with the next product."""
    _dev(gain, ssq)
    for t in (x, w, resid, xg):
        if not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
        if t.dim() != 2 or t.stride(1) != 1:
            raise KernelError("matrix product operands must be 2-D with unit inner stride")
    m, k = x.shape
    n = w.shape[0]
    if not gemm_residual_prescale_fits(x, w):
        raise KernelError(f"gemm_residual_prescale does not take x {tuple(x.shape)} {x.dtype}, w {tuple(w.shape)} {w.dtype}")
    _want(resid, torch.float32, "residual stream")
    _want(gain, torch.float32, "norm gain")
    _want(xg, torch.bfloat16, "prepared operand")
    _want(ssq, torch.float32, "sums of squares")
    tiles = (n + PRESCALE_TILE - 1) // PRESCALE_TILE
    if w.shape[1] != k or resid.shape != (m, n) or xg.shape != (m, n) or gain.numel() != n or ssq.shape != (m, tiles):
        raise KernelError(f"shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, residual {tuple(resid.shape)}, "
                          f"prepared {tuple(xg.shape)}, gain {gain.numel()}, sums {tuple(ssq.shape)} (need {(m, tiles)})")
    _check("gemm", library("gemm").rocml_gemm_residual_prescale(
        _ptr(x), max(x.stride(0), k), _ptr(w), w.stride(0), _ptr(resid), max(resid.stride(0), n), _ptr(gain), _ptr(xg),
        max(xg.stride(0), n), _ptr(ssq), m, n, k, waves, _stream()))


def splitk_reduce(partials: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """``out (+)= partials.sum(0)`` in split order, for ``partials [splits, M, N]`` float32."""
    _dev(partials, out)
    _want(partials, torch.float32, "partial sums")
    splits, m, n = partials.shape
    if out.shape != (m, n):
        raise KernelError("partial sums and output differ in shape")
    _check("gemm", library("gemm").rocml_splitk_reduce(_ptr(partials), _ptr(out), _code(out), out.stride(0), m, n,
                                                       splits, 1 if accumulate else 0, _stream()))


# ---- attention -----------------------------------------------------------------------
ATTN_AUTO, ATTN_PLAIN, ATTN_MFMA = 0, 1, 2


def attention(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              block_table: torch.Tensor, token_seq: torch.Tensor, token_pos: torch.Tensor,
              n_heads: int, n_kv_heads: int, head_dim: int, scale: float, window: Optional[int] = None,
              algo: int = ATTN_AUTO, workspace: Optional[torch.Tensor] = None,
              cu_seqlens: Optional[torch.Tensor] = None, max_new: int = 0,
              q_counts: Optional[Sequence[int]] = None, max_len: int = 0, n_splits: int = 0,
              v_head_dim: Optional[int] = None, values_in_keys: bool = False, chunk: Optional[int] = None,
              slopes: Optional[torch.Tensor] = None, sink: bool = False, sinks: Optional[torch.Tensor] = None,
              softcap: Optional[float] = None) -> None:
    """Attention of the step's query tokens over the cache.  Keys are ``[pages, Hkv, page, D]``,
    values ``[pages, Hkv, D, page]``.  ``cu_seqlens`` (device), ``q_counts`` (the same knowledge on
    the host: query tokens of each sequence), ``max_new`` (the most of them) and ``max_len``
    (longest context) describe the step to the fast kernels; without them the plain kernel runs.

    ``v_head_dim``: size of a value head when it is not ``head_dim``.  ``values_in_keys``: there is
    no value cache (``v_cache`` None) and a key's value is the first ``v_head_dim`` numbers of its
    row.  ``chunk``: blocks of so many positions, counted from 0, instead of a window: a query sees
    its own block up to itself.  ``slopes`` (32-bit, one per query head): ``slope * (i - j)`` is
    taken off the score of query ``i`` and key ``j``.  ``sink``: the denominator of the softmax has
    one more term ``exp(0)``, or with ``sinks`` (32-bit, one per query head) ``exp(sinks[h])``.
    ``softcap``: the scaled score ``s`` becomes ``softcap * tanh(s / softcap)`` before the mask."""
    _dev(q, out, k_cache, v_cache, block_table, token_seq, token_pos, cu_seqlens, slopes, sinks)
    if sinks is not None:
        _want(sinks, torch.float32, "sinks")
        if sinks.numel() != n_heads or not sink:
            raise KernelError("one sink per query head is needed, and the sink switched on")
    if softcap is not None and not softcap > 0:
        raise KernelError(f"the soft cap of the scores must be positive, got {softcap}")
    n_tokens = q.shape[0]
    dv = head_dim if v_head_dim is None else int(v_head_dim)
    if q.shape != (n_tokens, n_heads * head_dim) or out.shape != (n_tokens, n_heads * dv) or out.dtype != q.dtype:
        raise KernelError("attention input must be [tokens, heads * head_dim] and its output [tokens, heads * value size], of one type")
    page = k_cache.shape[2]
    if k_cache.dtype != q.dtype or k_cache.shape[1:] != (n_kv_heads, page, head_dim):
        raise KernelError(f"key cache {tuple(k_cache.shape)} {k_cache.dtype} does not fit the queries")
    if values_in_keys:
        if v_cache is not None or dv > head_dim:
            raise KernelError("values taken from the key rows: no value cache, and a value no longer than a key")
    elif v_cache is None or v_cache.dtype != q.dtype or v_cache.shape != (k_cache.shape[0], n_kv_heads, dv, page):
        raise KernelError(f"value cache does not fit keys {tuple(k_cache.shape)} and a value size of {dv}")
    if slopes is not None:
        _want(slopes, torch.float32, "distance slopes")
        if slopes.numel() != n_heads:
            raise KernelError("one distance slope per query head is needed")
    if chunk is not None and window is not None:
        raise KernelError("a layer has a window or blocks of positions, not both")
    _want(block_table, torch.int32, "block table")
    _want(token_seq, torch.int32, "token sequence table")
    _want(token_pos, torch.int32, "token position table")
    if token_seq.numel() != n_tokens or token_pos.numel() != n_tokens:
        raise KernelError("one sequence index and one position per token are needed")
    n_seqs = 0
    counts = None
    if cu_seqlens is not None:
        _want(cu_seqlens, torch.int32, "sequence offsets")
        n_seqs = cu_seqlens.numel() - 1
        if q_counts is not None:
            if len(q_counts) != n_seqs:
                raise KernelError(f"{len(q_counts)} query counts for {n_seqs} sequences")
            counts = (ctypes.c_int * n_seqs)(*[int(c) for c in q_counts])
    ws_ptr, ws_bytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    _check("attention", library("attention").rocml_attention(
        _ptr(q), _ptr(out), _ptr(k_cache), _ptr(v_cache), _code(q), _ptr(block_table),
        block_table.shape[1], _ptr(token_seq), _ptr(token_pos), n_tokens, n_heads, n_kv_heads, head_dim,
        page, scale, 0 if window is None else int(window), algo, _ptr(cu_seqlens), n_seqs, max_new,
        counts, max_len, n_splits, ws_ptr, ws_bytes, dv, 1 if values_in_keys else 0,
        0 if chunk is None else int(chunk), _ptr(slopes), 1 if sink else 0, _ptr(sinks),
        0.0 if softcap is None else float(softcap), _stream()))


FUSED_DECODE_HEAD_DIMS = (64, 128, 192, 256)
FUSED_DECODE_PAGE = 64
# The most partial sums of the projection the fused decode attention should be handed: it adds four in
# one trip to memory and each further one in a trip of its own.  Measured at 64 sequences (8B shape,
# decoded tokens a second): at most 4 pieces 8,022, 5 8,073, 6 8,003, 8 7,932, no limit 7,960; at 16
# to 48 sequences the limit makes no difference.
FUSED_DECODE_SPLITS = 5


def decode_splits(pairs: int, n_cus: int, most: int) -> int:
    """Splits of the key range for ``pairs`` (token, kv head) pairs of a decode step, at most
    ``most``.  A CU works at its full rate with two blocks on it, or with one whose waves keep two
    pieces on their way (which the kernel does when the chip holds at most a block a CU); every
    block costs about three pages' time beside its own pages, a merge of splits as much again and
    a little per split.  The choice is the count with the least work on the busiest CU by that
    account, for a nominal 32 pages a sequence: it must not follow the lengths, so that a recorded
    step can be replayed as the sequences grow.  Measured at the Qwen3-8B shape, 2,048-token
    contexts (decoded tokens a second): 14 sequences 3,040 with 2 or 4 splits, 2,850 with 9;
    18 sequences 3,555 with 3, 3,375 with 5; 24 sequences 4,480 with none, 4,310 with 4;
    32 sequences 5,620 with none, 5,375 with 2; 40 sequences 5,990 with 3, 5,720 with none;
    56 sequences 7,330 with none, 7,000 with 2.  Below 8 sequences' worth of pairs (64) the
    rule is about a block a CU."""
    if pairs * 4 < n_cus:
        # a few sequences: about a block a CU (two pieces of each wave are then on their way); measured,
        # one block a CU against two: one sequence 277.5 against 274.8 tokens a second, two 542 against
        # 532, four 1,050 against 1,029, six 1,518 against 1,501
        return max(1, min(n_cus // pairs, most))
    pages, per_block, merge, per_split = 32.0, 3.0, 3.0, 0.3
    best, best_cost = 1, float("inf")
    for s in range(1, max(1, min(most, 16)) + 1):
        blocks = pairs * s
        cost = -(-blocks // n_cus) * (pages / s + per_block) + (merge + per_split * s if s > 1 else 0.0)
        if cost < best_cost - 1e-9:
            best, best_cost = s, cost
    return best


def attention_decode_fusable(dtype: torch.dtype, n_heads: int, n_kv_heads: int, head_dim: int, page: int,
                             rot_dim: Optional[int], pairing: str = "halves") -> bool:
    """Whether ``attention_decode_fused`` takes this layer: bfloat16 cache in pages of 64, a head
    size it has a kernel for, at most 16 query heads per kv head, and a rotation (if any) of the
    whole head in pairs ``(i, i + head_dim / 2)``."""
    return (dtype == torch.bfloat16 and page == 64 and head_dim in FUSED_DECODE_HEAD_DIMS
            and n_heads // n_kv_heads <= 16 and (rot_dim is None or (rot_dim == head_dim and pairing == "halves")))


PREFILL_FUSED_PAGE = 64
PREFILL_FUSED_HEAD_DIMS = (32, 64, 96, 128, 192, 256)


def attention_prefill_fusable(dtype: torch.dtype, head_dim: int, page_size: int, rot_dim: Optional[int],
                              pairing: str = "halves") -> bool:
    """Whether ``attention_prefill_fused`` takes a layer: a bfloat16 cache with pages of 64 positions,
    a head size the MFMA kernels know, and a rotation of the whole head with halves as pairs (or none)."""
    return (dtype == torch.bfloat16 and page_size == PREFILL_FUSED_PAGE and head_dim in PREFILL_FUSED_HEAD_DIMS
            and (rot_dim is None or (rot_dim == head_dim and pairing == "halves")))


def attention_prefill_fused(qkv: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_table: torch.Tensor, token_pos: torch.Tensor, n_heads: int, n_kv_heads: int,
                            head_dim: int, scale: float, q_gain: Optional[torch.Tensor], eps: float,
                            cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], window: Optional[int],
                            cu_seqlens: torch.Tensor, q_counts: Sequence[int], max_len: int = 0) -> None:
    """A prompt step's attention with the queries taken from the q/k/v projection ``qkv`` (float32
    ``[tokens, ld]``, complete sums, a token's q heads first): per-head norm, rotation and rounding
    of the queries happen in the attention kernel.  The new tokens' keys and values are in the
    cache already (``qk_norm_rope_append`` without a q output puts them there).  ``max_len``
    (the longest context) is what ``--profile`` prices the call with; the kernel does not need it."""
    _dev(qkv, out, k_cache, v_cache, block_table, token_pos, q_gain, cos, sin, cu_seqlens)
    _want(qkv, torch.float32, "projection output")
    if qkv.dim() != 2:
        raise KernelError("the projection must be [tokens, width] (complete sums)")
    n_tokens, ld = qkv.shape
    page = k_cache.shape[2]
    if not attention_prefill_fusable(k_cache.dtype, head_dim, page, None if cos is None else 2 * cos.shape[-1]):
        raise KernelError(f"fused prefill attention does not take this layer (cache {k_cache.dtype}, pages of {page}, "
                          f"head size {head_dim})")
    if out.shape != (n_tokens, n_heads * head_dim) or out.dtype != k_cache.dtype:
        raise KernelError("attention output must be [tokens, heads * head_dim] of the cache's type")
    if v_cache.dtype != k_cache.dtype or k_cache.shape[1:] != (n_kv_heads, page, head_dim) \
            or v_cache.shape != (k_cache.shape[0], n_kv_heads, head_dim, page):
        raise KernelError(f"cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)} does not fit {n_kv_heads} heads of {head_dim}")
    if q_gain is not None:
        _want(q_gain, torch.float32, "head norm gain")
        if q_gain.numel() != head_dim:
            raise KernelError(f"head norm gain has {q_gain.numel()} values for head size {head_dim}")
    if cos is not None:
        _want(cos, torch.float32, "rotation table")
        if cos.shape != (n_tokens, head_dim // 2) or sin is None or sin.shape != cos.shape or sin.dtype != cos.dtype:
            raise KernelError(f"rotation tables must be float32 {(n_tokens, head_dim // 2)}")
    _want(block_table, torch.int32, "block table")
    _want(token_pos, torch.int32, "token position table")
    _want(cu_seqlens, torch.int32, "sequence offsets")
    n_seqs = cu_seqlens.numel() - 1
    if token_pos.numel() != n_tokens or len(q_counts) != n_seqs or block_table.shape[0] < n_seqs:
        raise KernelError("one position per token, one query count and one block table row per sequence are needed")
    counts = (ctypes.c_int * n_seqs)(*[int(c) for c in q_counts])
    _check("attention", library("attention").rocml_attention_prefill_fused(
        _ptr(qkv), ld, _ptr(q_gain), eps, _ptr(cos), _ptr(sin), _ptr(out), _ptr(k_cache), _ptr(v_cache),
        _ptr(block_table), block_table.shape[1], _ptr(token_pos), n_tokens, n_heads, n_kv_heads, head_dim, page,
        scale, 0 if window is None else int(window), _ptr(cu_seqlens), n_seqs, counts, _stream()))


def attention_decode_fused(qkv: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_table: torch.Tensor, token_seq: Optional[torch.Tensor], token_pos: torch.Tensor,
                           n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                           q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                           cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], write_kv: bool = True,
                           window: Optional[int] = None, workspace: Optional[torch.Tensor] = None,
                           max_len: int = 0, n_splits: int = 0, row_scale: Optional[RowScale] = None,
                           bias: Optional[torch.Tensor] = None, chunk: Optional[int] = None,
                           slopes: Optional[torch.Tensor] = None, sink: bool = False) -> None:
    """A decode step's attention straight from the q/k/v projection ``qkv`` (float32
    ``[tokens, ld]``, or its split-K partial sums ``[splits, tokens, ld]``): per-head norm,
    rotation, append of the new key and value to the cache and attention over the cache in one
    launch.  ``token_seq`` None: token ``t`` is the one token of the step's sequence ``t`` (row
    ``t`` of the block table).  ``workspace`` must not overlap ``qkv``.  ``row_scale``: the
    projection's operand lacked its norm's scale, which is applied to the projection's sums here.
    ``bias`` (32-bit, one number per column of a projection row) is added behind that scale;
    ``chunk``, ``slopes`` and ``sink`` as in ``attention``."""
    _dev(qkv, out, k_cache, v_cache, block_table, token_seq, token_pos, q_gain, k_gain, cos, sin, bias, slopes)
    if bias is not None:
        _want(bias, torch.float32, "projection bias")
        if bias.numel() < (n_heads + 2 * n_kv_heads) * head_dim and (write_kv or bias.numel() < n_heads * head_dim):
            raise KernelError("the bias is shorter than a projection row")
    if slopes is not None:
        _want(slopes, torch.float32, "distance slopes")
        if slopes.numel() != n_heads:
            raise KernelError("one distance slope per query head is needed")
    _want(qkv, torch.float32, "projection output")
    qkv_splits, split_stride = 1, 0
    if qkv.dim() == 3:
        qkv_splits, split_stride = qkv.shape[0], qkv.shape[1] * qkv.shape[2]
        qkv = qkv[0]
    n_tokens, ld = qkv.shape
    page = k_cache.shape[2]
    if not attention_decode_fusable(k_cache.dtype, n_heads, n_kv_heads, head_dim, page,
                                    None if cos is None else 2 * cos.shape[-1]):
        raise KernelError(f"fused decode attention does not take this layer (cache {k_cache.dtype}, pages of {page}, "
                          f"head size {head_dim}, {n_heads} heads over {n_kv_heads})")
    if out.shape != (n_tokens, n_heads * head_dim) or out.dtype != k_cache.dtype:
        raise KernelError("attention output must be [tokens, heads * head_dim] of the cache's type")
    if v_cache.dtype != k_cache.dtype or k_cache.shape[1:] != (n_kv_heads, page, head_dim) \
            or v_cache.shape != (k_cache.shape[0], n_kv_heads, head_dim, page):
        raise KernelError(f"cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)} does not fit {n_kv_heads} heads of {head_dim}")
    for g in (q_gain, k_gain):
        if g is not None:
            _want(g, torch.float32, "head norm gain")
            if g.numel() != head_dim:
                raise KernelError(f"head norm gain has {g.numel()} values for head size {head_dim}")
    if cos is not None:
        _want(cos, torch.float32, "rotation table")
        if cos.shape != (n_tokens, head_dim // 2) or sin is None or sin.shape != cos.shape or sin.dtype != cos.dtype:
            raise KernelError(f"rotation tables must be float32 {(n_tokens, head_dim // 2)}")
    _want(block_table, torch.int32, "block table")
    _want(token_pos, torch.int32, "token position table")
    if token_seq is not None:
        _want(token_seq, torch.int32, "token sequence table")
    elif block_table.shape[0] < n_tokens:
        raise KernelError(f"the block table has {block_table.shape[0]} rows for {n_tokens} sequences")
    if (token_seq is not None and token_seq.numel() != n_tokens) or token_pos.numel() != n_tokens:
        raise KernelError("one sequence index and one position per token are needed")
    ws_ptr, ws_bytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    ssq_ptr, parts, row_eps, width = None, 0, 0.0, 0
    if row_scale is not None:
        if row_scale.ssq.shape[0] < n_tokens:
            raise KernelError("the row scale has fewer rows than the step has tokens")
        ssq_ptr, parts, row_eps, width = row_scale.ssq.data_ptr(), row_scale.ssq.shape[1], row_scale.eps, row_scale.width
    _check("attention", library("attention").rocml_attention_decode_fused(
        _ptr(qkv), ld, qkv_splits, split_stride, _ptr(q_gain), _ptr(k_gain), eps, _ptr(cos), _ptr(sin),
        1 if write_kv else 0, _ptr(out), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
        _ptr(token_seq), _ptr(token_pos), n_tokens, n_heads, n_kv_heads, head_dim, page, scale,
        0 if window is None else int(window), max_len, n_splits, ws_ptr, ws_bytes, ssq_ptr, parts, row_eps, width,
        _ptr(bias), 0 if chunk is None else int(chunk), _ptr(slopes), 1 if sink else 0, _stream()))


# ---- sampling ------------------------------------------------------------------------
ARGMAX_WORK_WORDS = 64      # 32-bit words of workspace per row for the two-stage argmax
SAMPLE_SMALL_K = 64         # the largest top-k that the slice kernels of the sampler take


def argmax(logits: torch.Tensor, out: torch.Tensor, work: Optional[torch.Tensor] = None) -> None:
    """First index of each row's maximum.  With ``work`` (``ARGMAX_WORK_WORDS`` 32-bit words
    per row) long rows are searched by several blocks."""
    _dev(logits, out, work)
    _want(logits, torch.float32, "logits")
    _want(out, torch.int32, "token output")
    batch, vocab = logits.shape
    if work is not None and work.numel() * work.element_size() < batch * ARGMAX_WORK_WORDS * 4:
        raise KernelError("argmax workspace is too small")
    _check("sampling", library("sampling").rocml_argmax(_ptr(logits), batch, vocab, _ptr(out), _ptr(work), _stream()))


def sample(logits: torch.Tensor, work: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           out: torch.Tensor, top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           penalty: Optional[torch.Tensor] = None, history: Optional[torch.Tensor] = None,
           history_len: Optional[torch.Tensor] = None, small_k: int = 0) -> None:
    """``small_k``: 0, or a bound of at most 64 such that every sequence with a positive
    temperature has its top_k in ``[1, small_k]``: the caller's promise, which lets the selection
    run on slices of the vocabulary instead of whole rows."""
    _dev(logits, work, temperature, uniform, out, top_k, top_p, penalty, history, history_len)
    _want(logits, torch.float32, "logits")
    _want(work, torch.float32, "sampling workspace")
    batch, vocab = logits.shape
    if work.numel() < logits.numel():
        raise KernelError("sampling workspace is smaller than the logits")
    for t, dt, name in ((temperature, torch.float32, "temperature"), (uniform, torch.float32, "uniform"),
                        (top_p, torch.float32, "top_p"), (penalty, torch.float32, "penalty"),
                        (top_k, torch.int32, "top_k"), (history, torch.int32, "history"),
                        (history_len, torch.int32, "history lengths"), (out, torch.int32, "token output")):
        if t is not None:
            _want(t, dt, name)
            if name != "history" and t.numel() != batch:
                raise KernelError(f"{name} needs one value per sequence")
    if penalty is not None and (history is None or history_len is None or history.shape[0] != batch):
        raise KernelError("a repeat penalty needs the history and its lengths")
    _check("sampling", library("sampling").rocml_sample(
        _ptr(logits), _ptr(work), batch, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
        _ptr(penalty), _ptr(history), 0 if history is None else history.shape[1], _ptr(history_len),
        int(small_k), _ptr(out), _stream()))


# ---- recurrent ---------------------------------------------------------------------------
def causal_conv(u: torch.Tensor, col0: int, n_channels: int, w: torch.Tensor, bias: Optional[torch.Tensor],
                state: torch.Tensor, token_seq: torch.Tensor, cu_seqlens: torch.Tensor, seq_slots: torch.Tensor,
                out: torch.Tensor, silu: bool = True) -> None:
    """Causal convolution per channel over columns ``col0 .. col0 + n_channels - 1`` of the 32-bit
    ``u [T, ld]``: ``out[t, c] = act(bias[c] + sum_j w[j, c] in(t - (taps - 1) + j, c))``; ``w`` is
    ``[taps, channels]``, its last row the current token's.  ``state``
    ``[slots, taps - 1, channels]`` holds every sequence's last ``taps - 1`` inputs (zeros at its
    start), is read for the inputs before the step's first token and brought up to date."""
    _dev(u, w, bias, state, token_seq, cu_seqlens, seq_slots, out)
    for t, what in ((u, "convolution input"), (w, "convolution weights"), (state, "convolution state"), (out, "convolution output")):
        _want(t, torch.float32, what)
    n_tokens, ld = u.shape
    taps = w.shape[0]
    n_seqs = seq_slots.numel()
    if w.shape != (taps, n_channels) or (bias is not None and (bias.dtype != torch.float32 or bias.numel() != n_channels)):
        raise KernelError(f"convolution weights {tuple(w.shape)} or bias do not fit {n_channels} channels")
    if out.shape != (n_tokens, n_channels) or token_seq.numel() != n_tokens or cu_seqlens.numel() != n_seqs + 1:
        raise KernelError("convolution output or token tables do not fit the step")
    if state.dim() != 3 or state.shape[1:] != (max(taps - 1, 0), n_channels):
        raise KernelError(f"convolution state {tuple(state.shape)} does not fit {taps} taps of {n_channels} channels")
    _check("recurrent", library("recurrent").rocml_causal_conv(
        _ptr(u), ld, col0, n_tokens, n_channels, taps, _ptr(w), _ptr(bias), _ptr(state), state.shape[0], _ptr(token_seq),
        _ptr(cu_seqlens), _ptr(seq_slots), n_seqs, _ptr(out), 1 if silu else 0, _stream()))


def ssd_scan(xbc: torch.Tensor, dt_src: torch.Tensor, dt_col0: int, dt_bias: torch.Tensor, a_log: torch.Tensor,
             d_skip: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor, seq_slots: torch.Tensor, y: torch.Tensor,
             n_heads: int, head_dim: int, n_state: int, n_groups: int) -> None:
    """The recurrence with a scalar decay per head over the step's tokens, per sequence in order:
    ``dt = softplus(raw + dt_bias)``, ``S <- exp(-exp(A_log) dt) S + dt B x^T``, ``y = S^T C + D x``.
    ``xbc [T, H P + 2 G N]`` holds x, B and C side by side, the raw step sizes are columns
    ``dt_col0 .. dt_col0 + H - 1`` of ``dt_src``; ``state [slots, H, P, N]``; all 32-bit."""
    _dev(xbc, dt_src, dt_bias, a_log, d_skip, state, cu_seqlens, seq_slots, y)
    for t, what in ((xbc, "recurrence inputs"), (dt_src, "step sizes"), (dt_bias, "dt_bias"), (a_log, "A_log"),
                    (d_skip, "D"), (state, "recurrent state"), (y, "recurrence output")):
        _want(t, torch.float32, what)
    n_tokens = xbc.shape[0]
    n_seqs = seq_slots.numel()
    if state.dim() != 4 or state.shape[1:] != (n_heads, head_dim, n_state):
        raise KernelError(f"recurrent state {tuple(state.shape)} does not fit {n_heads} heads of {head_dim} x {n_state}")
    if y.shape != (n_tokens, n_heads * head_dim) or dt_src.shape[0] != n_tokens or cu_seqlens.numel() != n_seqs + 1:
        raise KernelError("recurrence output or tables do not fit the step")
    if min(dt_bias.numel(), a_log.numel(), d_skip.numel()) != n_heads or max(dt_bias.numel(), a_log.numel(), d_skip.numel()) != n_heads:
        raise KernelError("dt_bias, A_log and D must have one number per head")
    _check("recurrent", library("recurrent").rocml_ssd_scan(
        _ptr(xbc), xbc.shape[1], _ptr(dt_src), dt_src.shape[1], dt_col0, _ptr(dt_bias), _ptr(a_log), _ptr(d_skip),
        _ptr(state), state.shape[0], _ptr(cu_seqlens), _ptr(seq_slots), n_seqs, n_tokens, _ptr(y), n_heads, head_dim,
        n_state, n_groups, _stream()))


def gated_part_norm(y: torch.Tensor, z: torch.Tensor, z_col0: int, gain: torch.Tensor, out: torch.Tensor, parts: int,
                    eps: float) -> None:
    """``out = rms_parts(y * silu(z)) * gain``: the gate first, then each of the ``parts`` equal parts
    of a row divided by its own root mean square.  ``z`` is columns ``z_col0 ..`` of a 32-bit matrix."""
    _dev(y, z, gain, out)
    for t, what in ((y, "norm input"), (z, "gate"), (gain, "norm gain")):
        _want(t, torch.float32, what)
    rows, n = y.shape
    if gain.numel() != n or out.shape != y.shape or z.shape[0] != rows:
        raise KernelError("gated_part_norm: sizes differ")
    _check("recurrent", library("recurrent").rocml_gated_part_norm(
        _ptr(y), _ptr(z), z.shape[1], z_col0, _ptr(gain), _ptr(out), _code(out), rows, n, parts, float(eps), _stream()))


MLSTM_COLUMNS = 32      # values of a head that one block of the matrix memory's kernel owns


def mlstm_tiles(v_head_dim: int) -> int:
    """Blocks per head of the matrix memory's kernel; each keeps the head's ``n`` and ``m`` for itself."""
    return (v_head_dim + MLSTM_COLUMNS - 1) // MLSTM_COLUMNS


def mlstm_scan(proj: torch.Tensor, q_col0: int, k_col0: int, v_col0: int, i_col0: int, f_col0: int,
               i_bias: Optional[torch.Tensor], f_bias: Optional[torch.Tensor], cap: float, q_scale: float, floor: float,
               s_state: torch.Tensor, n_state: torch.Tensor, m_state: torch.Tensor, cu_seqlens: torch.Tensor,
               seq_slots: torch.Tensor, out: torch.Tensor, n_heads: int, head_dim: int, v_head_dim: int) -> None:
    """The matrix memory over the step's tokens, per sequence in order: with ``q`` (times ``q_scale``), ``k``,
    ``v`` and the raw gates taken from columns of the 32-bit ``proj [T, ld]``,
    ``i = cap tanh((raw_i + i_bias) / cap)``, ``f = logsigmoid(cap tanh((raw_f + f_bias) / cap))``,
    ``m' = max(f + m, i)``, ``S <- exp(f + m - m') S + exp(i - m') k v^T``, ``n`` likewise with ``k`` alone,
    ``out = S^T q / (max(|n . q|, exp(-m')) + floor)``.  States per slot: ``s_state [slots, H, dv, dk]``,
    ``n_state [slots, H, tiles, dk]``, ``m_state [slots, H, tiles]`` with ``tiles = mlstm_tiles(dv)``; all 32-bit."""
    _dev(proj, i_bias, f_bias, s_state, n_state, m_state, cu_seqlens, seq_slots, out)
    for t, what in ((proj, "projection"), (s_state, "matrix state"), (n_state, "vector state"), (m_state, "maximum state"),
                    (out, "memory output")):
        _want(t, torch.float32, what)
    lib = library("recurrent")
    if lib.rocml_mlstm_tile() != MLSTM_COLUMNS:
        raise KernelError("the matrix memory's kernel and its launcher disagree about a block's columns")
    n_tokens, n_seqs, tiles = proj.shape[0], seq_slots.numel(), mlstm_tiles(v_head_dim)
    slots = s_state.shape[0]
    if s_state.shape != (slots, n_heads, v_head_dim, head_dim) or n_state.shape != (slots, n_heads, tiles, head_dim) \
            or m_state.shape != (slots, n_heads, tiles):
        raise KernelError(f"matrix memory states {tuple(s_state.shape)}, {tuple(n_state.shape)}, {tuple(m_state.shape)} "
                          f"do not fit {n_heads} heads of {head_dim} x {v_head_dim}")
    if out.shape != (n_tokens, n_heads * v_head_dim) or cu_seqlens.numel() != n_seqs + 1:
        raise KernelError("matrix memory output or tables do not fit the step")
    for b in (i_bias, f_bias):
        if b is not None and (b.dtype != torch.float32 or b.numel() != n_heads):
            raise KernelError("gate biases must be 32-bit with one number per head")
    _check("recurrent", lib.rocml_mlstm_scan(
        _ptr(proj), proj.shape[1], q_col0, k_col0, v_col0, i_col0, f_col0, _ptr(i_bias), _ptr(f_bias), float(cap),
        float(q_scale), float(floor), _ptr(s_state), _ptr(n_state), _ptr(m_state), slots, _ptr(cu_seqlens), _ptr(seq_slots),
        n_seqs, n_tokens, _ptr(out), n_heads, head_dim, v_head_dim, _stream()))


HEAD_GATES = {"sigmoid": 0, "silu": 1}


def head_norm_gate(o: torch.Tensor, g: torch.Tensor, g_col0: int, gain: Optional[torch.Tensor], out: torch.Tensor, n_heads: int,
                   eps: float, gate: str = "sigmoid") -> None:
    """``out = rms_heads(o) * gain * act(g)``: every one of the ``n_heads`` equal parts of a row of the 32-bit
    ``o [T, n]`` divided by its own root mean square; ``g`` is columns ``g_col0 ..`` of a 32-bit matrix; ``act`` is
    ``sigmoid`` or ``silu``; without ``gain`` the normed values are only gated."""
    _dev(o, g, gain, out)
    for t, what in ((o, "norm input"), (g, "gate")) + (((gain, "norm gain"),) if gain is not None else ()):
        _want(t, torch.float32, what)
    if gate not in HEAD_GATES:
        raise KernelError(f"unknown gate {gate!r}; known: {sorted(HEAD_GATES)}")
    rows, n = o.shape
    if n % n_heads != 0 or (gain is not None and gain.numel() != n) or out.shape != o.shape or g.shape[0] != rows \
            or g.shape[1] < g_col0 + n:
        raise KernelError("head_norm_gate: sizes differ")
    _check("recurrent", library("recurrent").rocml_head_norm_gate(
        _ptr(o), _ptr(g), g.shape[1], g_col0, _ptr(gain), _ptr(out), _code(out), rows, n_heads, n // n_heads, float(eps),
        HEAD_GATES[gate], _stream()))


def decay_scan(q: torch.Tensor, q_col0: int, k: torch.Tensor, k_col0: int, v: torch.Tensor, v_col0: int,
               state: torch.Tensor, cu_seqlens: torch.Tensor, seq_slots: torch.Tensor, out: torch.Tensor,
               n_heads: int, head_dim: int, v_head_dim: int, head_decay: Optional[torch.Tensor] = None,
               decay: Optional[torch.Tensor] = None, decay_col0: int = 0, bonus: Optional[torch.Tensor] = None,
               decay_offset: Optional[torch.Tensor] = None) -> None:
    """A recurrence whose state per head, ``S [dk, dv]``, decays row by row, over the step's tokens, per sequence in
    order: ``S <- diag(w_t) S + k_t v_t^T``.  With ``head_decay`` (one number per head) ``w_t`` is that constant and
    the output reads the new state, ``o_t = S_t^T q_t``; with ``decay`` (per token and key channel, columns
    ``decay_col0 ..`` of a 32-bit matrix) and ``bonus`` ``u [H * dk]`` the output reads the state before the update,
    ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t``.  With ``decay_offset`` (``[H * dk]``) ``decay`` holds logits ``x`` and the
    decay is ``exp(-exp(x + decay_offset))``.  q, k, v are column ranges of 32-bit matrices ``[T, ld]``;
    ``state [slots, H, dv, dk]``; ``out [T, H * dv]``; all 32-bit."""
    _dev(q, k, v, state, cu_seqlens, seq_slots, out, head_decay, decay, bonus, decay_offset)
    for t, what in ((q, "queries"), (k, "keys"), (v, "values"), (state, "recurrent state"), (out, "recurrence output")):
        _want(t, torch.float32, what)
    n_tokens, n_seqs = out.shape[0], seq_slots.numel()
    if state.dim() != 4 or state.shape[1:] != (n_heads, v_head_dim, head_dim):
        raise KernelError(f"recurrent state {tuple(state.shape)} does not fit {n_heads} heads of {head_dim} x {v_head_dim}")
    if out.shape != (n_tokens, n_heads * v_head_dim) or cu_seqlens.numel() != n_seqs + 1 \
            or any(t.dim() != 2 or t.shape[0] != n_tokens for t in (q, k, v)):
        raise KernelError("recurrence inputs, output or tables do not fit the step")
    if (head_decay is None) == (decay is None) or (decay is None) != (bonus is None):
        raise KernelError("the recurrence takes one decay per head, or a decay per token and channel together with a bonus")
    if decay_offset is not None and decay is None:
        raise KernelError("an offset of the decays' logits goes with decays per token")
    for t, n, what in ((head_decay, n_heads, "the heads' decays"), (bonus, n_heads * head_dim, "the bonus"),
                       (decay_offset, n_heads * head_dim, "the offset of the decays' logits")):
        if t is not None and (t.dtype != torch.float32 or t.numel() != n):
            raise KernelError(f"{what} must be 32-bit with {n} numbers")
    if decay is not None and (decay.dtype != torch.float32 or decay.dim() != 2 or decay.shape[0] != n_tokens):
        raise KernelError("the decays per token must be a 32-bit matrix with a row per token")
    _check("recurrent", library("recurrent").rocml_decay_scan(
        _ptr(q), q.shape[1], q_col0, _ptr(k), k.shape[1], k_col0, _ptr(v), v.shape[1], v_col0, _ptr(decay),
        0 if decay is None else decay.shape[1], decay_col0, _ptr(decay_offset), _ptr(head_decay), _ptr(bonus), _ptr(state),
        state.shape[0],
        _ptr(cu_seqlens), _ptr(seq_slots), n_seqs, n_tokens, _ptr(out), n_heads, head_dim, v_head_dim, _stream()))


def rotate_rows(buf: torch.Tensor, col0: int, n_heads: int, head_dim: int, rot_dim: int, cos: Optional[torch.Tensor],
                sin: Optional[torch.Tensor], scale: float = 1.0, heads_first: Optional[int] = None, scale_rest: float = 1.0) -> None:
    """In place on columns ``col0 .. col0 + n_heads * head_dim - 1`` of the 32-bit ``buf [T, ld]``: of every head the
    first ``rot_dim`` numbers turn (number ``i`` with ``i + rot_dim / 2``, angles from the tables ``[T, rot_dim / 2]``),
    then the heads are multiplied by ``scale`` (with ``heads_first``: the heads from that one on by ``scale_rest``)."""
    _dev(buf, cos, sin)
    _want(buf, torch.float32, "the matrix to rotate")
    n_tokens = buf.shape[0]
    if rot_dim:
        if cos is None or sin is None or cos.shape != (n_tokens, rot_dim // 2) or sin.shape != cos.shape:
            raise KernelError(f"rotation tables must be {(n_tokens, rot_dim // 2)}")
    _check("recurrent", library("recurrent").rocml_rotate_rows(_ptr(buf), buf.shape[1], col0, n_tokens, n_heads, head_dim, rot_dim,
                                                             _ptr(cos), _ptr(sin), float(scale),
                                                             n_heads if heads_first is None else int(heads_first), float(scale_rest),
                                                             _stream()))


def shift_mix(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, token_seq: torch.Tensor, cu_seqlens: torch.Tensor,
              seq_slots: torch.Tensor, out: torch.Tensor) -> None:
    """``out[m, t] = h_t + (h_(t-1) - h_t) * mu[m]`` for every row of the 32-bit ``mu [mixes, n]``, in 32-bit, written in
    ``h``'s type.  Before a sequence's first token of the step stands its kept row ``state [slots, n]`` (32-bit, zeros
    at its start), which is replaced by the sequence's last row of the step."""
    _dev(h, mu, state, token_seq, cu_seqlens, seq_slots, out)
    _want(mu, torch.float32, "mix weights")
    _want(state, torch.float32, "the kept row")
    n_tokens, n = h.shape
    n_seqs = seq_slots.numel()
    if mu.dim() != 2 or mu.shape[1] != n or out.shape != (mu.shape[0], n_tokens, n) or out.dtype != h.dtype \
            or state.dim() != 2 or state.shape[1] != n or token_seq.numel() != n_tokens or cu_seqlens.numel() != n_seqs + 1:
        raise KernelError("shift_mix: sizes differ")
    _check("recurrent", library("recurrent").rocml_shift_mix(
        _ptr(h), _code(h), n_tokens, n, _ptr(mu), mu.shape[0], _ptr(state), state.shape[0], _ptr(token_seq), _ptr(cu_seqlens),
        _ptr(seq_slots), n_seqs, _ptr(out), _stream()))


def tanh(x: torch.Tensor, out: torch.Tensor) -> None:
    """``out = tanh(x)`` in ``out``'s type, for 32-bit ``x``."""
    _dev(x, out)
    _want(x, torch.float32, "the values")
    if x.numel() != out.numel():
        raise KernelError("tanh: sizes differ")
    _check("recurrent", library("recurrent").rocml_tanh(_ptr(x), _ptr(out), _code(out), x.numel(), _stream()))


def double_exp_decay(x: torch.Tensor, offset: torch.Tensor) -> None:
    """``x <- exp(-exp(x + offset))`` in place for the 32-bit ``x [T, n]`` and ``offset [n]``."""
    _dev(x, offset)
    _want(x, torch.float32, "decay logits")
    _want(offset, torch.float32, "decay offsets")
    if x.dim() != 2 or offset.numel() != x.shape[1]:
        raise KernelError("double_exp_decay: sizes differ")
    _check("recurrent", library("recurrent").rocml_double_exp_decay(_ptr(x), _ptr(offset), x.shape[0], x.shape[1], _stream()))


# ---- experts -----------------------------------------------------------------------------
MOE_TILE_ROWS = 128


def moe_max_tiles(n_pairs: int, n_experts: int) -> int:
    """Room for the tiles of a plan: an expert's last tile may be short."""
    return max(1, min(n_pairs, n_pairs // MOE_TILE_ROWS + n_experts))


def moe_route(logits: torch.Tensor, top: int, groups, sum_eps: float, chosen: torch.Tensor, weight: torch.Tensor,
              bias: Optional[torch.Tensor] = None, sigmoid: bool = False, correction: Optional[torch.Tensor] = None,
              group_top2: bool = False) -> None:
    """Softmax over all experts, the ``top`` best (of the experts of the ``groups[1]`` best of
    ``groups[0]`` equal groups of neighbours, a group's score being its largest, if ``groups`` is
    given), weights = chosen scores / (their sum + ``sum_eps``).  ``chosen`` int32, ``weight`` float32,
    both ``[T, top]``.  ``bias``: 32-bit, one number per expert, added to the logits first.  ``sigmoid``: an
    expert's score is ``sigmoid(logit)`` instead of the softmax.  ``correction``: 32-bit, one number per expert,
    added to the scores for the choice of groups and experts only.  ``group_top2``: a group's score is the sum of
    its two largest (corrected) scores."""
    _dev(chosen, weight, bias, correction)
    if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("the router's logits must be a GPU matrix with unit inner stride (rows may be the leading columns of a wider one)")
    if correction is not None and (correction.dtype != torch.float32 or correction.numel() != logits.shape[1]):
        raise KernelError("the correction of the experts' scores must be 32-bit with one number per expert")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != logits.shape[1]):
        raise KernelError("the router's bias must be 32-bit with one number per expert")
    _want(logits, torch.float32, "router logits")
    _want(chosen, torch.int32, "chosen experts")
    _want(weight, torch.float32, "expert weights")
    n_tokens, n_experts = logits.shape
    if chosen.shape != (n_tokens, top) or weight.shape != (n_tokens, top):
        raise KernelError("moe_route: outputs must be [tokens, top]")
    count, keep = (0, 0) if groups is None else (int(groups[0]), int(groups[1]))
    _check("moe", library("moe").rocml_moe_route(_ptr(logits), n_tokens, n_experts, top, count, keep, float(sum_eps),
                                                 _ptr(chosen), _ptr(weight), _ptr(bias), 1 if sigmoid else 0,
                                                 _ptr(correction), 1 if group_top2 else 0,
                                                 logits.stride(0) if n_tokens > 1 else max(logits.stride(0), n_experts), _stream()))


def moe_plan(chosen: torch.Tensor, n_experts: int, plan: torch.Tensor):
    """Sorts the (token, choice) pairs by expert.  ``plan`` is int32 scratch of at least
    ``moe_plan_words(pairs, experts)`` words; returns its views
    ``(offsets [E + 1], order [pairs], place [pairs], tiles [2 * max_tiles], n_tiles [1], max_tiles)``."""
    _dev(chosen, plan)
    _want(chosen, torch.int32, "chosen experts")
    _want(plan, torch.int32, "plan")
    n_pairs = chosen.numel()
    max_tiles = moe_max_tiles(n_pairs, n_experts)
    if plan.numel() < moe_plan_words(n_pairs, n_experts):
        raise KernelError("moe_plan: the plan's scratch is too small")
    at = 0
    views = []
    for n in (n_experts + 1, n_pairs, n_pairs, 2 * max_tiles, 1):
        views.append(plan[at:at + n])
        at += n
    offsets, order, place, tiles, n_tiles = views
    _check("moe", library("moe").rocml_moe_plan(_ptr(chosen), n_pairs, n_experts, _ptr(offsets), _ptr(order), _ptr(place),
                                                _ptr(tiles), _ptr(n_tiles), max_tiles, _stream()))
    return offsets, order, place, tiles, n_tiles, max_tiles


def moe_plan_words(n_pairs: int, n_experts: int) -> int:
    return n_experts + 1 + 2 * n_pairs + 2 * moe_max_tiles(n_pairs, n_experts) + 1


def moe_gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, plan, top: int, gather: bool,
             w2: Optional[torch.Tensor] = None, plain: bool = False) -> None:
    """The products of all experts over the plan's order: row ``r`` of ``out`` (a place of expert
    ``e``) is ``w[e] @ a_r``, with ``a_r`` the row of the pair's token when ``gather`` (``a`` holds the
    step's tokens) and row ``r`` of ``a`` otherwise.  With ``w2``: ``silu(w[e] a_r) * (w2[e] a_r)``.
    ``w`` is ``[experts, n, k]``."""
    offsets, order, place, tiles, n_tiles, max_tiles = plan
    _dev(a, w, w2, out)
    n_experts, n, k = w.shape
    if w2 is not None and (w2.shape != w.shape or w2.dtype != w.dtype):
        raise KernelError("moe_gemm: the second matrix must have the first one's shape and type")
    n_pairs = order.numel()
    if a.shape[1] != k or out.shape != (n_pairs, n) or a.dtype != w.dtype:
        raise KernelError(f"moe_gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit {n_pairs} pairs")
    _check("moe", library("moe").rocml_moe_gemm(
        _ptr(a), _code(a), a.shape[1], a.shape[0], _ptr(order) if gather else None, top, _ptr(w), _ptr(w2), _code(w), n * k, k,
        n_experts, _ptr(out), _code(out), n, n_pairs, n, k, _ptr(offsets), _ptr(tiles), _ptr(n_tiles), max_tiles,
        1 if plain else 0, _stream()))


def moe_combine(y: torch.Tensor, plan, weight: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """``out[t] (+)= sum_c weight[t, c] * y[place[t * top + c]]`` (32-bit, choices in order)."""
    offsets, order, place, tiles, n_tiles, max_tiles = plan
    _dev(y, weight, out)
    for t, what in ((y, "expert outputs"), (weight, "expert weights"), (out, "feed-forward output")):
        _want(t, torch.float32, what)
    n_tokens, top = weight.shape
    if y.shape != (n_tokens * top, out.shape[1]) or out.shape[0] != n_tokens:
        raise KernelError("moe_combine: sizes differ")
    _check("moe", library("moe").rocml_moe_combine(_ptr(y), _ptr(place), _ptr(weight), _ptr(out), n_tokens, top, out.shape[1],
                                                   1 if accumulate else 0, _stream()))
