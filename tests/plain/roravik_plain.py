"""A plain, slow Roravik decoder in torch on the CPU, one function per mechanism.

It is the oracle of the tests: written from the design's equations, sharing no code with the
library (it reads the configuration dictionary and the checkpoint's tensor names directly, and
keeps no cache: every call runs whole sequences, the recurrences token by token).

Notation: ``h`` a sublayer's input ``[T, width]``, positions ``0 .. T-1``, ``W x`` for a matrix
stored ``[out, in]``.  The arithmetic type is the type of the tensors handed in (the tests use
64-bit floats so that the oracle's own rounding does not count).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """Root-mean-square norm whose stored weight is the gain's distance from one."""
    return rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: Dict) -> torch.Tensor:
    """``x [T, heads, d]``: of every head the first ``dims`` numbers turn, number ``i`` together with
    number ``i + dims/2`` by the angle ``p base^(-2i/dims)``; the rest stays."""
    dims, base = rot["dims"], float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def short_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``u [T, C]``, ``w [C, taps]``: ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j][None, :]
    return y


def recurrence_read_after(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay) -> torch.Tensor:
    """``q, k [T, H, d]``, ``v [T, H, dv]``, one decay per head: ``S_t = decay S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``."""
    T, H, d = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for a in range(H):
        S = torch.zeros(d, v.shape[-1], dtype=q.dtype)
        for t in range(T):
            S = float(decay[a]) * S + torch.outer(k[t, a], v[t, a])
            out[t, a] = S.T @ q[t, a]
    return out


def recurrence_read_before(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, w: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    """``r, k, w [T, H, d]``, ``v [T, H, dv]``, ``u [H, d]``: ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``, then
    ``S_t = diag(w_t) S_(t-1) + k_t v_t^T``."""
    T, H, d = r.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=r.dtype)
    for a in range(H):
        S = torch.zeros(d, v.shape[-1], dtype=r.dtype)
        for t in range(T):
            kv = torch.outer(k[t, a], v[t, a])
            out[t, a] = (S + u[a][:, None] * kv).T @ r[t, a]
            S = w[t, a][:, None] * S + kv
    return out


def capped_window_softmax(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, cap: float, window: int,
                          sink: torch.Tensor) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]`` of one sequence: ``s = cap tanh(scale (q . k) / cap)``, position
    ``i`` sees ``j`` with ``0 <= i - j < window``, and the denominator has one more term ``exp(sink_a)``."""
    T, H, _ = q.shape
    G = k.shape[1]
    pos = torch.arange(T)
    dist = pos[:, None] - pos[None, :]
    seen = (dist >= 0) & (dist < window)
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * scale
        s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~seen, float("-inf"))
        top = torch.maximum(s.max(dim=-1, keepdim=True).values, sink[a])
        e = torch.exp(s - top)
        out[:, a] = (e @ v[:, g]) / (e.sum(dim=-1, keepdim=True) + torch.exp(sink[a] - top))
    return out


def retention(h: torch.Tensor, p: Dict[str, torch.Tensor], m: Dict, eps: float) -> torch.Tensor:
    """Linear attention with one fixed decay per head, no softmax and no denominator: per head
    ``S_t = decay S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``; q and k rotated, k times ``dim^(-1/2)``
    after the rotation; every head's ``o`` over its root mean square, the heads side by side times
    ``silu(W_g h)``, then ``W_o``."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rotate((h @ p["q"].T).view(T, H, d), pos, m["rot"])
    k = rotate((h @ p["k"].T).view(T, H, d), pos, m["rot"]) * d ** -0.5
    v = (h @ p["v"].T).view(T, H, dv)
    out = recurrence_read_after(q, k, v, m["decay"])
    out = rms(out, eps).reshape(T, H * dv) * silu(h @ p["g"].T)
    return out @ p["o"].T


def window_attention(h: torch.Tensor, p: Dict[str, torch.Tensor], m: Dict) -> torch.Tensor:
    """Grouped softmax attention: projections, a short causal convolution on every channel of q, k and v,
    rotation of q and k, ``s = cap tanh(scale (q . k) / cap)``, a window of ``mask.size`` positions (the
    query's own among them), and a denominator with one more term ``exp(sink_a)`` per head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = short_conv(h @ p["q"].T, p["q.conv"]).view(T, H, d)
    k = short_conv(h @ p["k"].T, p["k.conv"]).view(T, G, d)
    v = short_conv(h @ p["v"].T, p["v.conv"]).view(T, G, dv)
    q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    out = capped_window_softmax(q, k, v, float(m["scale"]), float(m["softcap"]), m["mask"]["size"], p["sink"])
    return out.reshape(T, H * dv) @ p["o"].T


def time_mix(h: torch.Tensor, p: Dict[str, torch.Tensor], m: Dict, eps: float) -> torch.Tensor:
    """A recurrence with a decay per key channel that depends on the token: every projection reads its
    own mix ``h + (h' - h) mu`` of the token's and the previous token's input; ``w = exp(-exp(W_w2
    tanh(W_w1 mix_w) + w0))``; per head ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``, then
    ``S_t = diag(w_t) S_(t-1) + k_t v_t^T``; every head's ``o`` over its root mean square, times a gain,
    times ``silu(W_g mix_g)``, then ``W_o``."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, h.shape[1], dtype=h.dtype), h[:-1]], dim=0)

    def mix(name):
        return h + (prev - h) * p["mu." + name][None, :]
    r = (mix("r") @ p["r"].T).view(T, H, d)
    k = (mix("k") @ p["k"].T).view(T, H, d)
    v = (mix("v") @ p["v"].T).view(T, H, d)
    gate = silu(mix("g") @ p["g"].T)
    w = torch.exp(-torch.exp(torch.tanh(mix("w") @ p["w1"].T) @ p["w2"].T + p["w0"][None, :])).view(T, H, d)
    out = recurrence_read_before(r, k, v, w, p["u"])
    out = rms(out, eps).reshape(T, H * d) * p["norm"][None, :] * gate
    return out @ p["o"].T


def parallel_mixer(h: torch.Tensor, p: Dict[str, torch.Tensor], m: Dict, eps: float) -> torch.Tensor:
    """Two mixers on one input, each with a weight of its own from the configuration."""
    left = {k[len("left."):]: v for k, v in p.items() if k.startswith("left.")}
    right = {k[len("right."):]: v for k, v in p.items() if k.startswith("right.")}
    return float(m["left_scale"]) * window_attention(h, left, m["left"]) + float(m["right_scale"]) * time_mix(h, right, m["right"], eps)


def dense_ff(h: torch.Tensor, p: Dict[str, torch.Tensor], mlp: Dict) -> torch.Tensor:
    """``g = min(W_gate h, limit)``, ``u = clamp(W_up h, -limit, limit)``, ``W_down (g sigmoid(1.702 g) (u + 1))``."""
    limit = float(mlp["limit"])
    g = torch.clamp(h @ p["gate"].T, max=limit)
    u = torch.clamp(h @ p["up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ p["down"].T


def small_ff(h: torch.Tensor, p: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """An expert: ``W_down (silu(W_gate h) * (W_up h))``."""
    return (silu(h @ p[prefix + "gate"].T) * (h @ p[prefix + "up"].T)) @ p[prefix + "down"].T


def choose_experts(z: torch.Tensor, correction: torch.Tensor, router: Dict):
    """``z [T, E]`` router logits.  Scores ``s = sigmoid(z)``; the choice goes by ``s + correction``, among
    the experts of the ``keep`` groups whose two largest such numbers have the largest sum; the weights
    are the chosen experts' ``s`` over their sum (+ 1e-20).  Returns ``(chosen [T, top], weights [T, top])``."""
    T, E = z.shape
    s = torch.sigmoid(z)
    c = s + correction[None, :]
    groups = router.get("groups")
    if groups is not None:
        count, keep = groups["count"], groups["keep"]
        per = E // count
        grouped = c.view(T, count, per)
        score = grouped.topk(min(2, per), dim=-1).values.sum(dim=-1)
        kept = score.topk(keep, dim=-1).indices
        allowed = torch.zeros(T, count, dtype=torch.bool)
        allowed.scatter_(1, kept, True)
        c = c.masked_fill(~allowed[:, :, None].expand(T, count, per).reshape(T, E), float("-inf"))
    chosen = c.topk(router["top"], dim=-1).indices
    w = s.gather(1, chosen)
    return chosen, w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def moe_ff(h: torch.Tensor, p: Dict[str, torch.Tensor], mlp: Dict) -> torch.Tensor:
    """The weighted sum of every token's chosen experts, plus a shared expert that every token uses,
    times ``sigmoid(W_sg h)`` (one number per token)."""
    chosen, w = choose_experts(h @ p["router"].T, p["correction"], mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(chosen.shape[1]):
            out[t] = out[t] + w[t, c] * small_ff(h[t:t + 1], p, f"e{int(chosen[t, c])}.")[0]
    if mlp.get("shared") is not None:
        out = out + torch.sigmoid(h @ p["shared.sg"].T) * small_ff(h, p, "shared.")
    return out


def layer_order(cfg: Dict) -> List[tuple]:
    """``(layer, first of a later pass)`` in run order: layers ``start .. stop - 1`` run ``times`` times in a
    row, the others once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if loop is None:
        return [(i, False) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(start)]
    for rep in range(times):
        order += [(i, rep > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(cfg: Dict, tensors: Dict[str, torch.Tensor], tokens, collect: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence.  ``collect``: a list that receives the stream after every layer run."""
    eps = float(cfg["norm"]["eps"])
    x0 = tensors["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    x = x0
    for i, again in layer_order(cfg):
        layer = cfg["layers"][i]
        pre = f"l{i}."
        if again:
            x = x + x0
        mp = {k[len(pre + "mix."):]: v for k, v in tensors.items() if k.startswith(pre + "mix.")}
        h = offset_norm(x, tensors[pre + "norm1"], eps)
        if layer["type"] == "retention":
            y = retention(h, mp, layer["mixer"], eps)
        else:
            y = parallel_mixer(h, mp, layer["mixer"], eps)
        x = x + offset_norm(y, tensors[pre + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            fp = {k[len(pre + "mlp."):]: v for k, v in tensors.items() if k.startswith(pre + "mlp.")}
            h = offset_norm(x, tensors[pre + "norm2"], eps)
            y = dense_ff(h, fp, mlp) if mlp["kind"] == "dense" else moe_ff(h, fp, mlp)
            x = x + offset_norm(y, tensors[pre + "norm2b"], eps)
        if collect is not None:
            collect.append(x)
    z = offset_norm(x, tensors["final.norm"], eps) @ tensors["embed"].T
    cap = float(cfg["logit_softcap"])
    return cap * torch.tanh(z / cap)


def greedy(cfg: Dict, tensors: Dict[str, torch.Tensor], prompt, n_new: int) -> List[int]:
    """``n_new`` tokens, each the largest logit after the prompt and the tokens before it."""
    tokens = list(prompt)
    out = []
    for _ in range(n_new):
        out.append(int(forward(cfg, tensors, tokens)[-1].argmax()))
        tokens.append(out[-1])
    return out
