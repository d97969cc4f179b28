"""Catalog of named models and the rule that tells a name from a folder.

The reference keeps a compiled-in table of checkpoints with a default context
and a sampling preset each (rocml/src/registry/catalog.rs:25-37,216-258) and
resolves ``--model`` as a path if it looks like one, else as a catalog name,
listing all names when it is unknown (rocml/src/registry/mod.rs:42-84,123-127).
Here an entry carries the whole configuration, so a model with random weights
needs no file.  Sizes of the 8B, 14B and 32B entries are the ones the
benchmark configurations name; the two tiny entries are the test models.  The
reference's other dense names (0.6B, 1.7B, 4B; rocml/src/registry/catalog.rs:216-248)
come without sizes in its files, which read them from each checkpoint: the sizes
here are the ones published with those checkpoints and nothing in the reference
pins them.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional

from ..errors import UnknownModelError
from ..sampling.params import SamplingParams

# Sampling preset the reference attaches to every dense Qwen3 entry
# (rocml/src/registry/catalog.rs:44-51).
QWEN_THINKING_SAMPLING = SamplingParams(temperature=0.6, top_k=20, top_p=0.95)

DEFAULT_CTX = 4096


@dataclass(frozen=True)
class ModelEntry:
    name: str
    config: Dict
    default_ctx: int = DEFAULT_CTX
    sampling: Optional[SamplingParams] = None
    init_norm_jitter: bool = False   # norm gains 1 + N(0, 0.02) instead of 1


def _qwen3(vocab, hidden, inter, layers, heads, kv_heads, head_dim, theta, eps, tied, max_pos):
    return {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": vocab,
            "hidden_size": hidden, "intermediate_size": inter, "num_hidden_layers": layers,
            "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
            "rope_theta": theta, "rms_norm_eps": eps, "tie_word_embeddings": tied,
            "max_position_embeddings": max_pos, "hidden_act": "silu", "attention_bias": False}


CATALOG: List[ModelEntry] = [
    ModelEntry("tiny-a", _qwen3(256, 64, 128, 2, 4, 2, 16, 10000.0, 1e-6, True, 128),
               default_ctx=128, init_norm_jitter=True),
    ModelEntry("tiny-b", _qwen3(384, 96, 224, 3, 6, 2, 32, 1000000.0, 1e-5, False, 512),
               default_ctx=512, init_norm_jitter=True),
    ModelEntry("qwen3-0.6b", _qwen3(151936, 1024, 3072, 28, 16, 8, 128, 1000000.0, 1e-6, True, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-1.7b", _qwen3(151936, 2048, 6144, 28, 16, 8, 128, 1000000.0, 1e-6, True, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-4b", _qwen3(151936, 2560, 9728, 36, 32, 8, 128, 1000000.0, 1e-6, True, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-8b", _qwen3(151936, 4096, 12288, 36, 32, 8, 128, 1000000.0, 1e-6, False, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-14b", _qwen3(151936, 5120, 17408, 40, 40, 8, 128, 1000000.0, 1e-6, False, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-32b", _qwen3(151936, 5120, 25600, 64, 64, 8, 128, 1000000.0, 1e-6, False, 40960),
               sampling=QWEN_THINKING_SAMPLING),
]



def _dokulix(vocab, width, ff, heads, kv_heads, dim, q_rank, kv_rank, rot_dim, window, chunk, n_layers, loop=None):
    """A Dokulix configuration whose layers are block attention and latent attention in turn."""
    att = {"type": "attention", "mlp": {"kind": "dense", "ff": ff},
           "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": chunk},
                     "scale": dim ** -0.5}}
    lat = {"type": "latent_attention", "mlp": {"kind": "dense", "ff": ff},
           "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": dim, "q_rank": q_rank, "kv_rank": kv_rank,
                     "mask": {"size": window}, "rot": {"base": 10000.0, "dims": rot_dim}, "scale": (dim + rot_dim) ** -0.5}}
    cfg = {"architecture": "Dokulix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
           "layers": [att if i % 2 == 0 else lat for i in range(n_layers)], "max_positions": 40960}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# The second architecture: a test-sized model whose middle layers run twice, and the layer sizes of a
# 2B-class model (random weights; no checkpoint of this design exists).
CATALOG += [
    ModelEntry("dokulix-tiny", _dokulix(320, 96, 160, 4, 2, 32, 48, 32, 16, 40, 48, 4, loop=(1, 3, 2)),
               default_ctx=512, init_norm_jitter=True),
    ModelEntry("dokulix-2b", _dokulix(32768, 2048, 6144, 16, 8, 128, 768, 512, 64, 1024, 1024, 24)),
]



def felovik_config(vocab, width, heads, kv_heads, dim, ssm_heads, ssm_dim, state, groups, ff, experts, expert_ff, top, n_layers,
                   max_positions=8192, dense_every=4):
    """A Felovik configuration: every layer the attention and the recurrence next to each other, a dense
    feed-forward in every ``dense_every``-th layer (the first among them) and routed experts in the others."""
    mixer = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                      "q_temp": {"coef": 0.1, "every": 1024}},
             "right": {"heads": ssm_heads, "vdim": ssm_dim, "state": state, "groups": groups, "conv": 4, "norm_groups": groups}}
    dense = {"kind": "dense", "ff": ff, "limit": 7.0}
    moe = {"kind": "moe", "expert": {"ff": expert_ff},
           "router": {"experts": experts, "top": top, "groups": {"count": 4, "keep": 2}}}
    return {"architecture": "Felovik", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": 1e-5},
            "embedding": {"scale": 1.0}, "postln_alpha": 1.0,
            "layers": [{"type": "parallel", "mixer": mixer, "mlp": dense if i % dense_every == 0 else moe} for i in range(n_layers)]}


# The third architecture: a test-sized model and the layer sizes of a 2B-class model (random weights; no
# checkpoint of this design exists).
CATALOG += [
    ModelEntry("felovik-tiny", felovik_config(320, 96, 4, 2, 32, 4, 16, 16, 2, 160, 8, 48, 2, 4, max_positions=512),
               default_ctx=512, init_norm_jitter=True),
    ModelEntry("felovik-2b", felovik_config(32768, 2048, 16, 8, 128, 32, 64, 128, 8, 6144, 32, 1024, 4, 24)),
]



def sogavik_config(vocab, width, heads, kv_heads, dim, window, mem_heads, mem_dim, experts, expert_ff, top, side_dim, n_layers,
                   parallel_every=4, max_positions=40960):
    """A Sogavik configuration: windowed attention with a gate per head in most layers (its rotation's
    frequencies stretched eightfold beyond 4,096 positions), and in every ``parallel_every``-th layer (the third
    among them) a windowed attention of a quarter of the window beside a matrix memory; routed experts in every
    layer, and ``side_dim`` columns of the side table for each."""
    def attention(w, stretched):
        rot = {"base": 1000000.0, "dims": dim}
        if stretched:
            rot["scaling"] = {"factor": 8.0, "original": 4096, "fast": 24.0, "slow": 2.0}
        return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "mask": {"size": w}, "rot": rot}
    mlp = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top}}
    layers = []
    for i in range(n_layers):
        if i % parallel_every == min(2, parallel_every - 1):
            mixer = {"left": attention(max(window // 4, 1), False),
                     "right": {"heads": mem_heads, "dim": mem_dim, "vdim": mem_dim, "gate_cap": 10.0}}
            layers.append({"type": "parallel", "mixer": mixer, "mlp": mlp})
        else:
            layers.append({"type": "attention", "mixer": attention(window, True), "mlp": mlp})
    return {"architecture": "Sogavik", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "token_side": {"dim": side_dim},
            "max_positions": max_positions, "layers": layers}


# The fourth architecture: a test-sized model and the layer sizes of a 2B-class model (random weights; no
# checkpoint of this design exists).
CATALOG += [
    ModelEntry("sogavik-tiny", sogavik_config(320, 96, 4, 2, 32, 40, 2, 24, 8, 48, 2, 8, 4, max_positions=512),
               default_ctx=512, init_norm_jitter=True),
    ModelEntry("sogavik-2b", sogavik_config(32768, 2048, 16, 8, 128, 1024, 16, 128, 32, 1024, 4, 64, 24)),
]



def roravik_config(vocab, width, heads, kv_heads, dim, window, ret_heads, ret_dim, mix_heads, mix_dim, ff, experts, expert_ff, top,
                   n_layers, loop=None, conv=4, decay_rank=64):
    """A Roravik configuration: a pair of mixers (a windowed attention whose q, k and v pass a short convolution, with a
    soft cap and a sink per head, beside a recurrence with a decay per token and channel) in the even layers and a
    retention in the odd ones; a dense feed-forward and routed experts (two groups of which one is kept, and a shared
    expert of twice an expert's size) in turn.  ``loop``: ``(start, stop, times)`` or None."""
    rot = {"base": 10000.0, "dims": dim}
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": conv, "scale": dim ** -0.5, "softcap": 50.0,
            "mask": {"size": window}, "rot": rot}
    right = {"heads": mix_heads, "dim": mix_dim, "decay_rank": decay_rank}
    decay = [1.0 - 2.0 ** (-5 - 6 * h / max(ret_heads - 1, 1)) for h in range(ret_heads)]
    retention = {"heads": ret_heads, "dim": ret_dim, "vdim": ret_dim, "decay": decay, "rot": {"base": 1000000.0, "dims": ret_dim}}
    dense = {"kind": "dense", "ff": ff, "limit": 7.0}
    moe = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top, "groups": {"count": 2, "keep": 1}},
           "shared": {"ff": 2 * expert_ff}}
    layers = []
    for i in range(n_layers):
        mlp = dense if i % 2 == 0 else moe
        if i % 2 == 0:
            layers.append({"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 0.5, "right_scale": 0.5}, "mlp": mlp})
        else:
            layers.append({"type": "retention", "mixer": retention, "mlp": mlp})
    cfg = {"architecture": "Roravik", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "embedding": {"scale": width ** 0.5},
           "logit_softcap": 25.0, "layers": layers}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


# The fifth architecture: a test-sized model and the layer sizes of a 2B-class model (random weights; no
# checkpoint of this design exists).
CATALOG += [
    ModelEntry("roravik-tiny", roravik_config(352, 96, 4, 2, 32, 48, 2, 24, 2, 16, 160, 8, 48, 2, 4, loop=(0, 2, 2), decay_rank=8),
               default_ctx=512, init_norm_jitter=True),
    ModelEntry("roravik-2b", roravik_config(32768, 2048, 16, 8, 128, 1024, 16, 128, 32, 64, 6144, 32, 1024, 4, 24)),
]

_BY_NAME = {e.name: e for e in CATALOG}


def register_model(entry: ModelEntry) -> None:
    """Adds a named configuration (of any registered architecture) to the catalog."""
    if entry.name in _BY_NAME:
        raise ValueError(f"the catalog already has a model called {entry.name!r}")
    CATALOG.append(entry)
    _BY_NAME[entry.name] = entry


def catalog_names() -> List[str]:
    from .registry import load_plugins
    load_plugins()
    return [e.name for e in CATALOG]


def looks_like_path(name_or_path: str) -> bool:
    """A folder with config.json, or anything with a path separator, is a path
    (rocml/src/registry/mod.rs:123-127 has the same rule for files)."""
    return (os.sep in name_or_path or name_or_path.startswith(".")
            or os.path.isdir(name_or_path))


@dataclass(frozen=True)
class Resolved:
    path: Optional[str]          # model folder, if --model was one
    entry: Optional[ModelEntry]  # catalog entry, if --model was a name


def resolve(name_or_path: str) -> Resolved:
    from .registry import load_plugins
    load_plugins()
    if looks_like_path(name_or_path):
        if not os.path.isfile(os.path.join(name_or_path, "config.json")):
            raise UnknownModelError(f"{name_or_path!r} is not a model folder (no config.json in it)")
        return Resolved(path=name_or_path, entry=None)
    if name_or_path not in _BY_NAME:
        raise UnknownModelError(
            f"unknown model {name_or_path!r}; known names: {', '.join(catalog_names())}; "
            "or give a folder with config.json and model.safetensors")
    return Resolved(path=None, entry=_BY_NAME[name_or_path])
