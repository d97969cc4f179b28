"""Small Roravik configurations and random weights for the tests.

The weights are drawn here and not by the library's own initialiser, with spreads that keep activations of
order one and make every mechanism count: attention scales well above 1/sqrt(dim) so that single keys stand
out, soft caps that bend the larger scores, sinks from far below the scores to above them, norm weights clearly
away from zero, decays of the recurrences from almost nothing kept to almost nothing lost, bonuses and mixes of
order one, router matrices and corrections that spread the tokens over the experts and let the correction
change the choice.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch


def attention(heads, kv_heads, dim, vdim, scale, window, rot, conv, softcap):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap, "conv": conv,
            "mask": {"size": window}, "rot": {"base": rot[0], "dims": rot[1]}}


def time_mix(heads, dim, rank):
    return {"heads": heads, "dim": dim, "decay_rank": rank}


def retention_layer(heads, dim, vdim, decay, rot, mlp):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay),
                                           "rot": {"base": rot[0], "dims": rot[1]}}, "mlp": mlp}


def parallel_layer(left, right, left_scale, right_scale, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, ff, top, groups=None, shared=None):
    router = {"experts": experts, "top": top, "groups": None if groups is None else {"count": groups[0], "keep": groups[1]}}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router, "shared": None if shared is None else {"ff": shared}}


def config(vocab, width, layers, loop=None, eps=1e-5, embed_scale=1.0, logit_softcap=30.0) -> Dict:
    cfg = {"architecture": "Roravik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
           "logit_softcap": logit_softcap, "layers": layers}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


# A: every size differs from its neighbours and few are multiples of 8: value heads narrower and wider than key heads,
# windows of 7, 33 and 70 (across a page of the cache), convolutions of 2, 3 and 4 taps, rotations of a part of the
# head and of all of it, retentions whose keys need two entries a lane (20) and whose values need three blocks of the
# kernel (36), time mixing with heads of 17, groups of experts of which one and two are kept, with and without a shared
# expert, a layer without a feed-forward, and the two middle layers run twice.
CFG_A = config(211, 72, [
    parallel_layer(attention(4, 2, 24, 16, 0.9, 7, (5000.0, 12), 3, 8.0), time_mix(3, 17, 5), 0.6, 0.9, moe(6, 24, 2, (2, 1), 40)),
    retention_layer(2, 20, 36, (0.9, 0.995), (10000.0, 20), dense(88, 1.5)),
    parallel_layer(attention(3, 3, 16, 40, 1.1, 33, (10000.0, 16), 2, 20.0), time_mix(2, 24, 8), 1.3, 0.4, None),
    retention_layer(3, 12, 8, (0.5, 0.97, 0.999), (300.0, 4), moe(6, 16, 3, (3, 2), None)),
    parallel_layer(attention(6, 1, 12, 12, 1.3, 70, (300.0, 4), 4, 5.0), time_mix(1, 40, 3), 0.5, 0.5, moe(5, 40, 1, None, 24)),
], loop=(1, 3, 2), eps=3e-6, embed_scale=8.5, logit_softcap=12.0)

# B: sizes the matrix-core kernels know: key heads of 64, 128 and 32 with value heads of the same size, widths that are
# multiples of 8, windows of 64, 65 and 130 (a page, a page and one, two pages and two), the first layer run three
# times.  Its attention scales are about twice 1/sqrt(dim): it is the model that bfloat16 runs are judged on.
CFG_B = config(300, 128, [
    parallel_layer(attention(4, 1, 64, 64, 0.25, 65, (10000.0, 64), 4, 30.0), time_mix(2, 64, 16), 0.6, 0.9, moe(8, 64, 3, (2, 1), 96)),
    retention_layer(4, 32, 32, (0.98, 0.99, 0.998, 0.9995), (1000000.0, 32), dense(256, 1.0)),
    parallel_layer(attention(2, 2, 128, 128, 0.18, 130, (200000.0, 64), 4, 50.0), time_mix(4, 32, 8), 0.7, 0.7, moe(16, 32, 4, (4, 2), 64)),
    parallel_layer(attention(8, 4, 32, 32, 0.35, 64, (10000.0, 32), 2, 15.0), time_mix(1, 128, 32), 1.0, 0.5, dense(192, 2.0)),
], loop=(0, 1, 3), embed_scale=11.3)

# C: the values that make mechanisms vanish or coincide: one head everywhere, a window of one (a token sees itself
# alone), a convolution of one tap, a rotation of a single pair, decays of one (nothing is forgotten) and of zero
# (nothing is kept), every expert chosen, a single expert, groups of one expert each and one group of all, a branch
# weight of zero, a loop that runs once, an embedding scale of one, a soft cap far above every score and one far below.
CFG_C = config(131, 36, [
    parallel_layer(attention(1, 1, 10, 10, 1.0, 1, (10000.0, 2), 1, 1000.0), time_mix(1, 1, 1), 1.0, 1.0, moe(2, 20, 2, (1, 1), 12)),
    retention_layer(2, 6, 1, (1.0, 0.0), (100.0, 2), moe(1, 12, 1, None, None)),
    parallel_layer(attention(2, 2, 12, 6, 0.8, 1000, (100.0, 12), 8, 0.05), time_mix(4, 6, 2), 0.0, 1.0, moe(4, 8, 2, (4, 2), 8)),
    retention_layer(1, 2, 12, (0.75,), (50.0, 2), dense(20, 100.0)),
], loop=(2, 3, 1), eps=1e-3, embed_scale=1.0, logit_softcap=1000.0)

# D: no loop at all, a width that is no multiple of 4 (no kernel takes its rows as 16-byte pieces), one layer of each kind.
CFG_D = config(97, 70, [
    retention_layer(2, 10, 14, (0.9, 0.99), (1000.0, 6), moe(4, 24, 2, (2, 2), 10)),
    parallel_layer(attention(2, 1, 12, 10, 0.8, 9, (100.0, 6), 3, 6.0), time_mix(2, 5, 4), 0.8, 1.1, dense(50, 0.7)),
], eps=1e-5, embed_scale=5.0, logit_softcap=8.0)

CONFIGS = {"A": (CFG_A, 41), "B": (CFG_B, 42), "C": (CFG_C, 43), "D": (CFG_D, 44)}


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    w = cfg["width"]
    shapes = {"embed": (cfg["vocab"], w), "final.norm": (w,)}
    for i, lay in enumerate(cfg["layers"]):
        p = f"l{i}."
        shapes.update({p + "norm1": (w,), p + "norm1b": (w,), p + "norm2": (w,), p + "norm2b": (w,)})
        m = lay["mixer"]
        if lay["type"] == "retention":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            q = p + "mix."
            shapes.update({q + "q": (H * d, w), q + "k": (H * d, w), q + "v": (H * dv, w), q + "g": (H * dv, w), q + "o": (w, H * dv)})
        else:
            left, right = m["left"], m["right"]
            H, G, d, dv, taps = left["heads"], left["kv_heads"], left["dim"], left["vdim"], left["conv"]
            q = p + "mix.left."
            shapes.update({q + "q": (H * d, w), q + "k": (G * d, w), q + "v": (G * dv, w), q + "o": (w, H * dv), q + "sink": (H,),
                           q + "q.conv": (H * d, taps), q + "k.conv": (G * d, taps), q + "v.conv": (G * dv, taps)})
            H, d, rank = right["heads"], right["dim"], right["decay_rank"]
            q = p + "mix.right."
            for s in ("r", "k", "v", "g", "w"):
                shapes[q + "mu." + s] = (w,)
            for s in ("r", "k", "v", "g"):
                shapes[q + s] = (H * d, w)
            shapes.update({q + "w1": (rank, w), q + "w2": (H * d, rank), q + "w0": (H * d,), q + "u": (H, d), q + "norm": (H * d,),
                           q + "o": (w, H * d)})
        mlp = lay.get("mlp")
        if mlp is None:
            continue
        q = p + "mlp."
        if mlp["kind"] == "dense":
            shapes.update({q + "gate": (mlp["ff"], w), q + "up": (mlp["ff"], w), q + "down": (w, mlp["ff"])})
            continue
        ff, n = mlp["expert"]["ff"], mlp["router"]["experts"]
        shapes.update({q + "router": (n, w), q + "correction": (n,)})
        for e in range(n):
            shapes.update({q + f"e{e}.gate": (ff, w), q + f"e{e}.up": (ff, w), q + f"e{e}.down": (w, ff)})
        if mlp.get("shared") is not None:
            ff = mlp["shared"]["ff"]
            shapes.update({q + "shared.gate": (ff, w), q + "shared.up": (ff, w), q + "shared.down": (w, ff), q + "shared.sg": (1, w)})
    return shapes


def random_tensors(cfg: Dict, seed: int) -> Dict[str, torch.Tensor]:
    """Values that bfloat16 holds exactly (so both compute types read the same weights)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        def n(std=1.0, mean=0.0):
            return mean + std * torch.randn(shape, generator=gen)
        last = name.rsplit(".", 1)[-1]
        if last in ("norm1", "norm2", "norm1b", "norm2b") or name == "final.norm":
            t = n(0.3)                                   # stored around zero
        elif name.endswith("right.norm"):
            t = n(0.3, 1.0)
        elif name == "embed":
            t = n(1.0 / max(cfg["embedding"]["scale"], 1.0))
        elif last == "sink":
            t = n(3.0)                                   # from far below the scores to above them
        elif last == "conv":
            t = n(0.6)
        elif ".mu." in name:
            t = torch.rand(shape, generator=gen)
        elif last == "w0":
            t = n(1.5, -1.0)                             # decays from almost zero to almost one
        elif last == "w2":
            t = n(1.0)
        elif last == "u":
            t = n(1.0)
        elif last == "correction":
            t = n(0.5)
        elif last == "router":
            t = n(3.0 / shape[-1] ** 0.5)
        else:
            t = n(1.5 / shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    return out


def write_model(path: str, cfg: Dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16, keep_rank: bool = False) -> str:
    """A model folder.  Unless ``keep_rank``, config.json goes without the decay's inner width, which the loader
    then takes from the tensors' shapes."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    cfg = json.loads(json.dumps(cfg))
    if not keep_rank:
        for lay in cfg["layers"]:
            if lay["type"] == "parallel":
                lay["mixer"]["right"].pop("decay_rank", None)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def as_double(tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: v.double() for k, v in tensors.items()}
