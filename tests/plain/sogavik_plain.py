"""A plain, slow Sogavik decoder in torch on the CPU, one function per mechanism.

It is the oracle of the tests: written from the design's equations, sharing no code with the
library (it reads the configuration dictionary and the checkpoint's tensor names directly, and
keeps no cache: every call runs whole sequences, the matrix memory token by token).

Notation: ``h`` a sublayer's input ``[T, width]``, positions ``0 .. T-1``, ``W x`` for a matrix
stored ``[out, in]``.  The arithmetic type is the type of the tensors handed in (the tests use
64-bit floats so that the oracle's own rounding does not count).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w + b, var the mean squared deviation."""
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(dim=-1, keepdim=True) + eps) * w + b


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def log_sigmoid(z):
    return -(torch.log1p(torch.exp(-z.abs())) + torch.clamp(-z, min=0.0))


def rotary_frequencies(rot: Dict) -> tuple:
    """``(f, magnitude)``: ``f_i = base^(-2i/dims)`` for ``i < dims/2``.  With a ``scaling`` table
    (factor s, original length L, fast, slow): ``d(t) = dims ln(L / (2 pi t)) / (2 ln base)``,
    ``lo = max(floor(d(fast)), 0)``, ``hi = min(ceil(d(slow)), dims - 1)``,
    ``r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``, ``f_i <- f_i / s * r_i + f_i (1 - r_i)``,
    and cosines and sines are multiplied by ``0.1 ln(s) + 1``."""
    dims, base = rot["dims"], float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    mag = 1.0
    sc = rot.get("scaling")
    if sc is not None:
        def d(t):
            return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))
        lo = max(math.floor(d(sc["fast"])), 0)
        hi = min(math.ceil(d(sc["slow"])), dims - 1)
        for i in range(half):
            r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / sc["factor"] * r + f[i] * (1.0 - r)
        mag = 0.1 * math.log(sc["factor"]) + 1.0
    return f, mag


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: Dict) -> torch.Tensor:
    """``x [T, heads, d]``: of every head the first ``dims`` numbers turn, number ``i`` together with
    number ``i + dims/2`` by the angle ``p f_i``; the rest stays."""
    dims = rot["dims"]
    half = dims // 2
    f, mag = rotary_frequencies(rot)
    ang = positions.to(torch.float64)[:, None] * torch.tensor(f, dtype=torch.float64)[None, :]
    c, s = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int]) -> torch.Tensor:
    """Softmax attention of one sequence: ``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]``; query head
    ``a`` uses key/value head ``a // (H / G)``; position ``i`` sees ``j`` with ``0 <= i - j < window``."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    dist = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    visible = dist >= 0
    if window is not None:
        visible = visible & (dist < window)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def window_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float,
                     head_gate: bool) -> torch.Tensor:
    """Biased q, k, v; q and k normed over their whole rows (all heads at once) with a weight each,
    then rotated; windowed softmax attention; optionally every head's output times the sigmoid of one
    number per head projected from ``h``; output matrix."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ t[pre + "q"].T + t[pre + "q.b"]
    k = h @ t[pre + "k"].T + t[pre + "k.b"]
    v = h @ t[pre + "v"].T + t[pre + "v.b"]
    q = (rms(q, eps) * t[pre + "q.norm"]).reshape(T, H, d)
    k = (rms(k, eps) * t[pre + "k.norm"]).reshape(T, G, d)
    pos = torch.arange(T)
    if m.get("rot") is not None:
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    mask = m.get("mask")
    out = attend(q, k, v.reshape(T, G, dv), m["scale"], None if mask is None else mask["size"])
    if head_gate:
        out = out * torch.sigmoid(h @ t[pre + "g"].T)[:, :, None]
    return out.reshape(T, H * dv) @ t[pre + "o"].T


def matrix_memory_gates(h, t, pre, cap):
    """Log input gate ``cap tanh(a / cap)`` and log forget gate ``logsigmoid(cap tanh(b / cap))``."""
    a = h @ t[pre + "i"].T + t[pre + "i.b"]
    b = h @ t[pre + "f"].T + t[pre + "f.b"]
    return cap * torch.tanh(a / cap), log_sigmoid(cap * torch.tanh(b / cap))


def matrix_memory_scan(q, k, v, ig, fg):
    """``q, k [T, H, d]``, ``v [T, H, dv]``, gates ``[T, H]``.  Per head, with ``S`` (d x dv), ``n`` (d)
    and ``m`` all zero at the start: ``m' = max(f + m, i)``, ``S' = exp(f + m - m') S + exp(i - m') k v^T``,
    ``n'`` the same with ``k``, output ``S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)``."""
    T, H, d = q.shape
    dv = v.shape[2]
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for a in range(H):
        S = torch.zeros(d, dv, dtype=q.dtype)
        n = torch.zeros(d, dtype=q.dtype)
        m = torch.zeros((), dtype=q.dtype)
        for r in range(T):
            m_new = torch.maximum(fg[r, a] + m, ig[r, a])
            keep, take = torch.exp(fg[r, a] + m - m_new), torch.exp(ig[r, a] - m_new)
            S = keep * S + take * torch.outer(k[r, a], v[r, a])
            n = keep * n + take * k[r, a]
            m = m_new
            den = torch.maximum((n @ q[r, a]).abs(), torch.exp(-m)) + 1e-6
            out[r, a] = (S.T @ q[r, a]) / den
    return out


def matrix_memory(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict, eps: float) -> torch.Tensor:
    """Queries scaled by ``dim^(-1/2)``; the scan; every head's output divided by its root mean square,
    the heads side by side times a weight, times ``sigmoid(W_g h)``, then the output matrix."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ t[pre + "k"].T).reshape(T, H, d)
    v = (h @ t[pre + "v"].T).reshape(T, H, dv)
    ig, fg = matrix_memory_gates(h, t, pre, float(m["gate_cap"]))
    o = rms(matrix_memory_scan(q, k, v, ig, fg), eps).reshape(T, H * dv)
    return (o * t[pre + "norm"] * torch.sigmoid(h @ t[pre + "g"].T)) @ t[pre + "o"].T


def parallel_mixer(h, t, pre, m, eps):
    """Half the sum of the two mixers' outputs, each normed over the width with a weight of its own."""
    left = window_attention(h, t, pre + "left.", m["left"], eps, head_gate=False)
    right = matrix_memory(h, t, pre + "right.", m["right"], eps)
    return 0.5 * (rms(left, eps) * t[pre + "left.out"] + rms(right, eps) * t[pre + "right.out"])


def choose(logits: torch.Tensor, top: int):
    """The ``top`` largest logits and the softmax over them alone."""
    picked, chosen = torch.topk(logits, top, dim=-1)
    return chosen, torch.softmax(picked, dim=-1)


def expert_ff(h, t, pre):
    return (silu(h @ t[pre + "gate"].T) * (h @ t[pre + "up"].T)) @ t[pre + "down"].T


def routed_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], pre: str, m: Dict) -> torch.Tensor:
    chosen, weight = choose(h @ t[pre + "router"].T + t[pre + "router.b"], m["router"]["top"])
    out = torch.zeros_like(h)
    for r in range(h.shape[0]):
        for e, w in zip(chosen[r].tolist(), weight[r]):
            out[r] = out[r] + w * expert_ff(h[r:r + 1], t, f"{pre}e{e}.")[0]
    return out


def token_side(x, t, pre, rows, eps):
    """``rows [T, dim]``: the layer's part of every token's side row.  ``y = W_proj (gelu(W_gate x) * rows)``
    and the result is ``rms(y) * weight``."""
    y = (gelu_tanh(x @ t[pre + "gate"].T) * rows) @ t[pre + "proj"].T
    return rms(y, eps) * t[pre + "norm"]


def layer(x, t, i, spec, cfg, tokens) -> torch.Tensor:
    """Each sublayer reads the stream itself and its output is normed before it is added:
    ``x += norm1(mixer(x))``, ``x += norm2(ff(x))``, then the token's side input is added."""
    pre, eps = f"l{i}.", cfg["norm"]["eps"]
    if spec["type"] == "attention":
        y = window_attention(x, t, pre + "mix.", spec["mixer"], eps, head_gate=True)
    elif spec["type"] == "parallel":
        y = parallel_mixer(x, t, pre + "mix.", spec["mixer"], eps)
    else:
        raise ValueError(f"unknown layer type {spec['type']!r}")
    x = x + layer_norm(y, t[pre + "norm1"], t[pre + "norm1.b"], eps)
    mlp = spec.get("mlp")
    if mlp is not None:
        if mlp["kind"] != "moe":
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        x = x + layer_norm(routed_ff(x, t, pre + "mlp.", mlp), t[pre + "norm2"], t[pre + "norm2.b"], eps)
    side = cfg.get("token_side")
    if side is not None:
        ids = torch.tensor(list(tokens), dtype=torch.long)
        rows = t["side.embed"][ids][:, i * side["dim"]:(i + 1) * side["dim"]]
        x = x + token_side(x, t, pre + "side.", rows, eps)
    return x


def forward(cfg: Dict, t: Dict[str, torch.Tensor], tokens: Sequence[int], streams: Optional[List] = None) -> torch.Tensor:
    """Logits at every position ``[T, vocab]``; with ``streams`` a list, the residual stream
    after every layer is appended to it."""
    x = t["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    for i, spec in enumerate(cfg["layers"]):
        x = layer(x, t, i, spec, cfg, tokens)
        if streams is not None:
            streams.append(x)
    return layer_norm(x, t["final.norm"], t["final.norm.b"], cfg["norm"]["eps"]) @ t["head"].T


def greedy(cfg: Dict, t: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int) -> List[int]:
    ids, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(forward(cfg, t, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
