"""Small Sogavik configurations and random weights for the tests.

The weights are drawn here and not by the library's own initialiser, with spreads that keep activations of
order one and make every mechanism count: attention scales well above 1/sqrt(dim) so that single keys stand
out, norm weights and biases clearly away from one and zero, gates of the matrix memory that forget between a
few percent and almost nothing, router matrices and biases that spread the tokens over the experts.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch


def attention(heads, kv_heads, dim, vdim, scale, window=None, rot=None, stretch=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
        if stretch is not None:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    return m


def memory(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def moe(experts, ff, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def attention_layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def parallel_layer(left, right, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def config(vocab, width, layers, side_dim: Optional[int], eps=1e-5) -> Dict:
    cfg = {"architecture": "Sogavik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if side_dim is not None:
        cfg["token_side"] = {"dim": side_dim}
    return cfg


# A: every size differs from its neighbours and none is a multiple of 8 where it need not be: value heads narrower
# and wider than key heads, windows of 7, 33, 70 (across a page of the cache) and 5, rotations of a part of the
# head and of all of it, with and without stretched frequencies, a matrix memory whose values need two blocks of
# the kernel (36 > 32) and one with odd sizes, a layer without a feed-forward, one chosen expert and all of them.
CFG_A = config(211, 72, [
    attention_layer(attention(4, 2, 24, 16, 0.9, 7, (5000.0, 12), (3.0, 64, 8.0, 2.0)), moe(6, 24, 2)),
    parallel_layer(attention(3, 3, 16, 40, 1.1, 33, (10000.0, 16)), memory(2, 20, 36, 8.0), None),
    attention_layer(attention(6, 1, 12, 12, 1.3, 70, (300.0, 4)), moe(5, 40, 1)),
    parallel_layer(attention(2, 1, 40, 24, 0.6, 5, (20000.0, 40), (2.0, 32, 4.0, 0.5)), memory(3, 17, 9, 2.5), moe(3, 16, 3)),
], side_dim=5, eps=3e-6)

# B: sizes the matrix-core kernels know: key heads of 64, 128 and 32 with value heads of the same size, widths that
# are multiples of 8, windows of 64, 65 and 130 (a page, a page and one, two pages and two), the parallel layers
# first and last.  Its attention scales are twice 1/sqrt(dim): it is the model that bfloat16 runs are judged on.
CFG_B = config(300, 128, [
    parallel_layer(attention(4, 1, 64, 64, 0.25, 65, (10000.0, 64)), memory(2, 64, 64, 12.0), moe(8, 64, 3)),
    attention_layer(attention(2, 2, 128, 128, 0.18, 130, (200000.0, 64), (5.0, 128, 16.0, 1.0)), moe(16, 32, 4)),
    attention_layer(attention(8, 4, 32, 32, 0.35, 64, (10000.0, 32), (8.0, 64, 8.0, 2.0)), None),
    parallel_layer(attention(4, 2, 64, 64, 0.3, 200, (500.0, 16)), memory(4, 128, 32, 30.0), moe(4, 96, 2)),
], side_dim=8)

# C: the values that make mechanisms vanish or coincide: one head everywhere, a window of one (a token sees itself
# alone), a layer without window and one without rotation, a rotation of a single pair, a stretch by a factor of
# one, every expert chosen and a single expert, a matrix memory of one number per key and of one value, a side
# input of one column, and a model without side input comes with D.
CFG_C = config(131, 36, [
    attention_layer(attention(1, 1, 10, 10, 1.0, 1, (10000.0, 2)), moe(2, 20, 2)),
    parallel_layer(attention(2, 2, 12, 6, 0.8, None, None), memory(1, 1, 12, 1.0), moe(1, 12, 1)),
    attention_layer(attention(1, 1, 20, 20, 0.5, 1000, (100.0, 20), (1.0, 16, 2.0, 1.0)), None),
    parallel_layer(attention(1, 1, 8, 8, 0.7, 3, (50.0, 8)), memory(4, 6, 1, 100.0), moe(3, 12, 3)),
], side_dim=1, eps=1e-3)

# D: no side input at all, one layer of each kind.
CFG_D = config(97, 48, [
    parallel_layer(attention(2, 1, 16, 24, 0.7, 9, (1000.0, 8)), memory(2, 12, 20, 4.0), moe(4, 24, 2)),
    attention_layer(attention(3, 1, 16, 8, 0.9, 12, (1000.0, 16)), moe(4, 24, 1)),
], side_dim=None)

# E: a width that is no multiple of 4 (no kernel takes its rows as 16-byte pieces, and the pair of mixers forms its sum in
# a kernel of its own), both kinds of layer.
CFG_E = config(90, 70, [
    parallel_layer(attention(2, 1, 12, 10, 0.8, 6, (100.0, 6)), memory(2, 5, 7, 3.0), moe(3, 10, 2)),
    attention_layer(attention(2, 2, 10, 14, 0.9, 20, (100.0, 10), (2.0, 8, 4.0, 1.0)), moe(2, 18, 1)),
], side_dim=3)

CONFIGS = {"A": (CFG_A, 31), "B": (CFG_B, 32), "C": (CFG_C, 33), "D": (CFG_D, 34), "E": (CFG_E, 35)}


def _attention_shapes(p: str, m: Dict, w: int, gate: bool) -> Dict[str, tuple]:
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    shapes = {p + "q": (H * d, w), p + "q.b": (H * d,), p + "k": (G * d, w), p + "k.b": (G * d,), p + "v": (G * dv, w),
              p + "v.b": (G * dv,), p + "q.norm": (H * d,), p + "k.norm": (G * d,), p + "o": (w, H * dv)}
    if gate:
        shapes[p + "g"] = (H, w)
    return shapes


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    w = cfg["width"]
    side = cfg.get("token_side")
    shapes = {"embed": (cfg["vocab"], w), "final.norm": (w,), "final.norm.b": (w,), "head": (cfg["vocab"], w)}
    if side is not None:
        shapes["side.embed"] = (cfg["vocab"], side["dim"] * len(cfg["layers"]))
    for i, lay in enumerate(cfg["layers"]):
        p = f"l{i}."
        shapes.update({p + "norm1": (w,), p + "norm1.b": (w,), p + "norm2": (w,), p + "norm2.b": (w,)})
        if lay["type"] == "attention":
            shapes.update(_attention_shapes(p + "mix.", lay["mixer"], w, gate=True))
        else:
            shapes.update(_attention_shapes(p + "mix.left.", lay["mixer"]["left"], w, gate=False))
            r = lay["mixer"]["right"]
            H, d, dv = r["heads"], r["dim"], r["vdim"]
            q = p + "mix.right."
            shapes.update({q + "q": (H * d, w), q + "k": (H * d, w), q + "v": (H * dv, w), q + "g": (H * dv, w),
                           q + "o": (w, H * dv), q + "norm": (H * dv,), q + "i": (H, w), q + "i.b": (H,), q + "f": (H, w),
                           q + "f.b": (H,), p + "mix.left.out": (w,), p + "mix.right.out": (w,)})
        mlp = lay.get("mlp")
        if mlp is not None:
            ff = mlp["expert"]["ff"]
            shapes[p + "mlp.router"] = (mlp["router"]["experts"], w)
            shapes[p + "mlp.router.b"] = (mlp["router"]["experts"],)
            for e in range(mlp["router"]["experts"]):
                shapes.update({p + f"mlp.e{e}.gate": (ff, w), p + f"mlp.e{e}.up": (ff, w), p + f"mlp.e{e}.down": (w, ff)})
        if side is not None:
            shapes.update({p + "side.gate": (side["dim"], w), p + "side.proj": (w, side["dim"]), p + "side.norm": (w,)})
    return shapes


def random_tensors(cfg: Dict, seed: int) -> Dict[str, torch.Tensor]:
    """Values that bfloat16 holds exactly (so both compute types read the same weights)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        def n(std=1.0, mean=0.0):
            return mean + std * torch.randn(shape, generator=gen)
        if name.endswith(("norm1", "norm2", ".norm", ".out")):
            t = n(0.3, 1.0)
        elif name.endswith(("norm1.b", "norm2.b", "final.norm.b")):
            t = n(0.3)
        elif name in ("embed", "side.embed"):
            t = n(1.0)
        elif name.endswith("f.b"):
            t = n(1.5, 2.0)              # forget gates from a half to almost one
        elif name.endswith(("i.b", "router.b", "q.b", "k.b", "v.b")):
            t = n(0.5)
        elif name.endswith("router"):
            t = n(3.0 / shape[-1] ** 0.5)
        else:
            t = n(1.5 / shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    return out


def write_model(path: str, cfg: Dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def as_double(tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: v.double() for k, v in tensors.items()}
