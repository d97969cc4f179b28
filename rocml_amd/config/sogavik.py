"""Typed configuration of the Sogavik decoder, read from config.json.

A Sogavik model is a list of layers in which a sublayer reads the residual stream itself and a
layer norm (weight and bias) is applied to the sublayer's output before it is added:
``x += norm1(mixer(x))``, ``x += norm2(ff(x))``.  After the feed-forward every layer adds an input
that depends on the token's id: the layer's columns of the token's row of a side table gate a
small projection of the stream, and the result is added under a root-mean-square norm.  A layer's
mixer is either a windowed softmax attention (``attention``) or a pair of mixers on one input
(``parallel``): such an attention without an output gate (``left``) and a matrix memory
(``right``), each output normed over the width with a gain of its own, and averaged.  The
attention has biased q/k/v projections, norms q and k over a token's whole projection, rotates
the first ``rot.dims`` values of every head (optionally with slowed frequencies) and, in the
``attention`` layer, gates every head's output with one number.  The feed-forward is a mixture of
experts chosen by the largest router logits, weighted by the softmax over the chosen logits.
config.json gives every size layer by layer:

* ``architecture``: ``"Sogavik"``; ``vocab``, ``width``; ``norm.eps``; ``token_side.dim``;
* ``layers[i]``: ``type`` (``attention`` or ``parallel``), ``mixer`` and ``mlp``: null or
  ``{"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}``;
* an attention (``mixer`` of an ``attention`` layer, ``mixer.left`` of a ``parallel`` one):
  ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size``, ``rot`` (``base``, ``dims``,
  optionally ``scaling`` with ``factor``, ``original``, ``fast``, ``slow``);
* ``mixer.right``: ``heads``, ``dim``, ``vdim``, ``gate_cap``.

``max_positions`` may be given; without it sequences are bounded by the cache alone.

Constants the design fixes live here: the half in front of the two mixers' sum, the floor under
the matrix memory's denominator, the activation of the side input.
"""
from __future__ import annotations

import copy
import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

from ..errors import ConfigError, UnsupportedArchitectureError
from .spec import (AttentionSpec, BlockSpec, LayerNormSpec, MatrixMemorySpec, ModelSpec, NormSpec, ParallelMixerSpec,
                   RopeSpec, RopeStretch, RoutedExpertsSpec, TableSpec, TokenSideSpec, default_schedule)

ARCHITECTURE = "Sogavik"
BRANCH_WEIGHT = 0.5              # half the sum of the two mixers' normed outputs
MEMORY_FLOOR = 1e-6              # added to the matrix memory's denominator
SIDE_ACTIVATION = "gelu_tanh"
SIDE_TABLE = "token_side"
UNBOUNDED_POSITIONS = 1 << 30    # a model that names no limit


def _table(where: str, d: Dict, key: str) -> Dict:
    if not isinstance(d.get(key), dict):
        raise ConfigError(f"config.json lacks the table {where}{key}")
    return d[key]


def _int(where: str, d: Dict, key: str) -> int:
    if key not in d:
        raise ConfigError(f"config.json lacks {where}{key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json {where}{key!r} must be a positive integer, found {v!r}")
    return v


def _num(where: str, d: Dict, key: str) -> float:
    if key not in d:
        raise ConfigError(f"config.json lacks {where}{key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or v <= 0:
        raise ConfigError(f"config.json {where}{key!r} must be a positive number, found {v!r}")
    return float(v)


def _check_attention(where: str, m: Dict) -> None:
    for key in ("heads", "kv_heads", "dim", "vdim"):
        _int(where, m, key)
    _num(where, m, "scale")
    if m["heads"] % m["kv_heads"] != 0:
        raise ConfigError(f"config.json {where[:-1]}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv_heads")
    if m.get("mask") is not None:
        _int(where + "mask.", _table(where, m, "mask"), "size")
    if m.get("rot") is not None:
        rot = _table(where, m, "rot")
        dims = _int(where + "rot.", rot, "dims")
        base = _num(where + "rot.", rot, "base")
        if dims % 2 != 0 or dims > m["dim"] or base <= 1.0:
            raise ConfigError(f"config.json {where}rot: dims {dims} must be even and at most dim {m['dim']}, base above 1")
        if rot.get("scaling") is not None:
            sc = _table(where + "rot.", rot, "scaling")
            for key in ("factor", "original", "fast", "slow"):
                _num(where + "rot.scaling.", sc, key)


def _check_layer(i: int, layer) -> Dict:
    where = f"layers[{i}]."
    kind = layer.get("type") if isinstance(layer, dict) else None
    if kind not in ("attention", "parallel"):
        raise ConfigError(f"config.json {where}type is {kind!r}; known: attention, parallel")
    m = _table(where, layer, "mixer")
    if kind == "attention":
        _check_attention(where + "mixer.", m)
    else:
        _check_attention(where + "mixer.left.", _table(where + "mixer.", m, "left"))
        right = _table(where + "mixer.", m, "right")
        for key in ("heads", "dim", "vdim"):
            _int(where + "mixer.right.", right, key)
        _num(where + "mixer.right.", right, "gate_cap")
    mlp = layer.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
            raise ConfigError(f"config.json {where}mlp must be null or of kind 'moe', found {mlp!r}")
        _int(where + "mlp.expert.", _table(where + "mlp.", mlp, "expert"), "ff")
        r = _table(where + "mlp.", mlp, "router")
        experts, top = _int(where + "mlp.router.", r, "experts"), _int(where + "mlp.router.", r, "top")
        if top > experts:
            raise ConfigError(f"config.json {where}mlp.router: top {top} exceeds the {experts} experts")
    return copy.deepcopy(layer)


@dataclass(frozen=True)
class SogavikConfig:
    vocab: int
    width: int
    eps: float
    side_dim: Optional[int]                # None: the model has no side input
    layers: Tuple[Dict, ...]               # as config.json has them, validated
    max_positions: Optional[int] = None
    eos_token_id: Optional[Tuple[int, ...]] = None

    @classmethod
    def from_dict(cls, raw: Dict) -> "SogavikConfig":
        if raw.get("architecture") != ARCHITECTURE:
            raise UnsupportedArchitectureError(
                f"config.json names architecture {raw.get('architecture')!r}; this class reads {ARCHITECTURE!r}")
        vocab, width = _int("", raw, "vocab"), _int("", raw, "width")
        eps = _num("norm.", _table("", raw, "norm"), "eps")
        side_dim = None
        if raw.get("token_side") is not None:
            side_dim = _int("token_side.", _table("", raw, "token_side"), "dim")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json key 'layers' must be a list with at least one layer")
        checked: List[Dict] = [_check_layer(i, layer) for i, layer in enumerate(layers)]
        values = dict(vocab=vocab, width=width, eps=eps, side_dim=side_dim, layers=tuple(checked))
        if raw.get("max_positions") is not None:
            values["max_positions"] = _int("", raw, "max_positions")
        eos = raw.get("eos_token_id")
        if eos is not None:
            ids = list(eos) if isinstance(eos, (list, tuple)) else [eos]
            for t in ids:
                if isinstance(t, bool) or not isinstance(t, int) or not 0 <= t < vocab:
                    raise ConfigError(f"config.json key 'eos_token_id' must name token ids below vocab, found {eos!r}")
            values["eos_token_id"] = tuple(ids)
        return cls(**values)

    def to_dict(self) -> Dict:
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "layers": copy.deepcopy(list(self.layers))}
        if self.side_dim is not None:
            d["token_side"] = {"dim": self.side_dim}
        if self.max_positions is not None:
            d["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    def _attention(self, m: Dict, head_gate: bool) -> AttentionSpec:
        q_dim, kv_dim = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
        position = None
        rot = m.get("rot")
        if rot is not None:
            sc = rot.get("scaling")
            stretch = None if sc is None else RopeStretch(factor=float(sc["factor"]), original=float(sc["original"]),
                                                          fast=float(sc["fast"]), slow=float(sc["slow"]))
            position = RopeSpec(head_dim=m["dim"], rot_dim=rot["dims"], theta=float(rot["base"]), stretch=stretch)
        mask = m.get("mask")
        return AttentionSpec(hidden=self.width, n_heads=m["heads"], n_kv_heads=m["kv_heads"], head_dim=m["dim"],
                             v_head_dim=m["vdim"], scale=float(m["scale"]), window=None if mask is None else mask["size"],
                             # (the norm's size is the query projection's; the key's gain has the key projection's)
                             qk_norm=NormSpec(size=q_dim, eps=self.eps), qk_norm_span="projection", position=position,
                             bias=True, o_bias=False, gate=head_gate, gate_per_head=head_gate)

    def to_model_spec(self) -> ModelSpec:
        layer_norm = LayerNormSpec(size=self.width, eps=self.eps)
        blocks = []
        for i, layer in enumerate(self.layers):
            m = layer["mixer"]
            if layer["type"] == "attention":
                mixer = self._attention(m, head_gate=True)
            else:
                right = m["right"]
                memory = MatrixMemorySpec(hidden=self.width, n_heads=right["heads"], head_dim=right["dim"],
                                          v_head_dim=right["vdim"], gate_cap=float(right["gate_cap"]), eps=self.eps,
                                          floor=MEMORY_FLOOR)
                mixer = ParallelMixerSpec(hidden=self.width, weight=BRANCH_WEIGHT, eps=self.eps,
                                          branches=(("left", self._attention(m["left"], head_gate=False)), ("right", memory)))
            mlp = layer.get("mlp")
            ffn = None
            if mlp is not None:
                r = mlp["router"]
                ffn = RoutedExpertsSpec(hidden=self.width, n_experts=r["experts"], top=r["top"], intermediate=mlp["expert"]["ff"],
                                        activation="silu", weighting="softmax_chosen", router_bias=True)
            side = side_norm = None
            if self.side_dim is not None:
                side = TokenSideSpec(hidden=self.width, dim=self.side_dim, table=SIDE_TABLE, column0=i * self.side_dim,
                                     activation=SIDE_ACTIVATION)
                side_norm = NormSpec(size=self.width, eps=self.eps)
            blocks.append(BlockSpec(mixer=mixer, ffn=ffn, mixer_norm=layer_norm, ffn_norm=None if ffn is None else layer_norm,
                                    arrangement="sublayer_norm", side=side, side_norm=side_norm))
        tables = ()
        if self.side_dim is not None:
            tables = (TableSpec(name=SIDE_TABLE, rows=self.vocab, cols=len(blocks) * self.side_dim),)
        spec = ModelSpec(architecture=ARCHITECTURE, vocab=self.vocab, hidden=self.width, layers=tuple(blocks),
                         schedule=default_schedule(len(blocks)), final_norm=layer_norm, tie_lm_head=False,
                         max_positions=self.max_positions or UNBOUNDED_POSITIONS, eos_token_ids=self.eos_token_id or (),
                         tables=tables)
        spec.validate()
        return spec


def checkpoint_names(spec: ModelSpec) -> Dict[str, str]:
    """Internal parameter name -> tensor name in the checkpoint: ``embed``, ``side.embed``,
    ``l<i>.norm1|norm2`` (a bias is the name with ``.b``), ``l<i>.mix.q|k|v`` (with ``.b``),
    ``l<i>.mix.q.norm|k.norm|g|o`` (under ``mix.left.`` in a parallel layer, which has no ``g``),
    ``l<i>.mix.right.q|k|v|g|o|norm|i|i.b|f|f.b``, ``l<i>.mix.left.out|right.out``,
    ``l<i>.mlp.router|router.b``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.side.gate|proj|norm``,
    ``final.norm|norm.b``, ``head``."""
    names = {"embed.weight": "embed", "final_norm.weight": "final.norm", "final_norm.bias": "final.norm.b",
             "lm_head.weight": "head"}
    for t in spec.tables:
        names[f"tables.{t.name}"] = "side.embed"

    def attention(dst: str, src: str, gate: bool) -> None:
        for p in ("q", "k", "v"):
            names[dst + f"{p}_proj.weight"] = src + p
            names[dst + f"{p}_proj.bias"] = src + p + ".b"
        names[dst + "q_norm.weight"] = src + "q.norm"
        names[dst + "k_norm.weight"] = src + "k.norm"
        names[dst + "o_proj.weight"] = src + "o"
        if gate:
            names[dst + "g_proj.weight"] = src + "g"

    for i, block in enumerate(spec.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"], names[dst + "mixer_norm.bias"] = src + "norm1", src + "norm1.b"
        if block.mixer.kind == "parallel":
            attention(dst + "mixer.left.", src + "mix.left.", gate=False)
            for p in ("q", "k", "v", "g", "o", "i", "f"):
                names[dst + f"mixer.right.{p}_proj.weight"] = src + f"mix.right.{p}"
            names[dst + "mixer.right.i_proj.bias"] = src + "mix.right.i.b"
            names[dst + "mixer.right.f_proj.bias"] = src + "mix.right.f.b"
            names[dst + "mixer.right.norm.weight"] = src + "mix.right.norm"
            names[dst + "mixer.left.out_norm.weight"] = src + "mix.left.out"
            names[dst + "mixer.right.out_norm.weight"] = src + "mix.right.out"
        else:
            attention(dst + "mixer.", src + "mix.", gate=True)
        if block.ffn is not None:
            names[dst + "ffn_norm.weight"], names[dst + "ffn_norm.bias"] = src + "norm2", src + "norm2.b"
            names[dst + "ffn.router.weight"], names[dst + "ffn.router.bias"] = src + "mlp.router", src + "mlp.router.b"
            for e in range(block.ffn.n_experts):
                for p in ("gate", "up", "down"):
                    names[dst + f"ffn.experts.{e}.{p}_proj.weight"] = src + f"mlp.e{e}.{p}"
        if block.side is not None:
            names[dst + "side.gate_proj.weight"] = src + "side.gate"
            names[dst + "side.out_proj.weight"] = src + "side.proj"
            names[dst + "side_norm.weight"] = src + "side.norm"
    return names


def unused_tensors(spec: ModelSpec) -> Tuple[str, ...]:
    """Tensors a checkpoint may hold that the model does not read: the second norm of a layer
    without a feed-forward."""
    out = []
    for i, block in enumerate(spec.layers):
        if block.ffn is None:
            out += [f"l{i}.norm2", f"l{i}.norm2.b"]
    return tuple(out)
