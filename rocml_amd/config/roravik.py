"""Typed configuration of the Roravik decoder, read from config.json.

A Roravik layer has a norm before and one after each sublayer, ``x += norm1b(mixer(norm1(x)))`` and
``x += norm2b(ff(norm2(x)))``, all of them root-mean-square norms whose stored weight is the gain's
distance from one.  A layer's mixer is

* a **retention** (``type: retention``): linear attention with a fixed decay per head, rotated q and
  k, every head's output divided by its root mean square and gated by ``silu(W_g h)``; or
* a **pair of mixers on one input** (``type: parallel``): a windowed softmax attention whose q, k
  and v pass a short causal convolution, with a soft cap on the scores and a learned sink per head
  (``left``), and a recurrence whose decay depends on the token (``right``); the result is
  ``left_scale * left + right_scale * right``.

The feed-forward is dense (gate and up values held under a limit, ``g sigmoid(1.702 g) (u + 1)``), a
mixture of small experts (sigmoid scores, a correction added for the choice only, groups scored by
the sum of their two best, and a gated shared expert), or absent.  A stretch of layers may run
several times in a row with the same weights; before every pass but the first the embedding's output
is added to the stream.  The logits come from the embedding's own table and pass a soft cap.
config.json gives every size layer by layer:

* ``architecture``: ``"Roravik"``; ``vocab``, ``width``; ``norm.eps``; ``embedding.scale``;
  ``logit_softcap``; ``loop`` (``start``, ``stop``, ``times``) or absent; ``max_positions`` or absent;
* ``layers[i]``: ``type``; for ``retention`` ``mixer`` has ``heads``, ``dim``, ``vdim``, ``decay`` (a
  number per head) and ``rot`` (``base``, ``dims``); for ``parallel`` ``mixer.left`` has ``heads``,
  ``kv_heads``, ``dim``, ``vdim``, ``conv``, ``scale``, ``softcap``, ``mask.size`` and ``rot``,
  ``mixer.right`` has ``heads`` and ``dim``, and ``mixer.left_scale`` / ``right_scale`` weigh the two;
  ``mlp``: null, ``{"kind": "dense", "ff", "limit"}`` or ``{"kind": "moe", "expert": {"ff"}, "router":
  {"experts", "top", "groups": {"count", "keep"} or null}, "shared": {"ff"} or null}``.

The inner width of the decay's two small matrices is read from the checkpoint's tensor shapes by the
loader's name table; here it is the configuration's ``mixer.right.decay_rank`` when given and
otherwise filled in from the shapes (``with_shapes``).

Constants the design fixes live here: the 1.702 in the dense feed-forward's gate, the one added to
its up values, the 1e-20 under the experts' weights, the two best scores that make a group's score.
"""
from __future__ import annotations

import copy
import math
from dataclasses import dataclass, replace
from typing import Dict, List, Optional, Tuple

from ..errors import ConfigError, UnsupportedArchitectureError
from .spec import (AttentionSpec, BlockSpec, GatedMlpSpec, ModelSpec, NormSpec, ParallelMixerSpec, RetentionSpec, RopeSpec,
                   RoutedExpertsSpec, ScheduleEntry, TimeMixSpec)

ARCHITECTURE = "Roravik"
DENSE_ACTIVATION = "sigmoid_1702"
DENSE_UP_OFFSET = 1.0
EXPERT_SUM_EPS = 1e-20
GROUP_SCORE = "top2_sum"
DEFAULT_DECAY_RANK = 16          # used for random models when the configuration names none
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


def _num(where: str, d: Dict, key: str, positive: bool = True) -> float:
    if key not in d:
        raise ConfigError(f"config.json lacks {where}{key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or (positive and v <= 0):
        raise ConfigError(f"config.json {where}{key!r} must be a {'positive ' if positive else ''}number, found {v!r}")
    return float(v)


def _check_rot(where: str, m: Dict, dim: int) -> None:
    rot = _table(where, m, "rot")
    _num(where + "rot.", rot, "base")
    dims = _int(where + "rot.", rot, "dims")
    if dims % 2 != 0 or dims > dim:
        raise ConfigError(f"config.json {where}rot.dims must be even and at most the head size {dim}, found {dims}")


def _check_mlp(where: str, mlp) -> None:
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
        raise ConfigError(f"config.json {where}mlp must be null or of kind 'dense' or 'moe', found {mlp!r}")
    if mlp["kind"] == "dense":
        _int(where + "mlp.", mlp, "ff")
        _num(where + "mlp.", mlp, "limit")
        return
    _int(where + "mlp.expert.", _table(where + "mlp.", mlp, "expert"), "ff")
    r = _table(where + "mlp.", mlp, "router")
    experts, top = _int(where + "mlp.router.", r, "experts"), _int(where + "mlp.router.", r, "top")
    if top > experts:
        raise ConfigError(f"config.json {where}mlp.router: top {top} exceeds the {experts} experts")
    if r.get("groups") is not None:
        g = _table(where + "mlp.router.", r, "groups")
        count, keep = _int(where + "mlp.router.groups.", g, "count"), _int(where + "mlp.router.groups.", g, "keep")
        if experts % count != 0 or keep > count or top > keep * (experts // count):
            raise ConfigError(f"config.json {where}mlp.router.groups: {count} groups of which {keep} are kept do "
                              f"not fit {experts} experts and top {top}")
    if mlp.get("shared") is not None:
        _int(where + "mlp.shared.", _table(where + "mlp.", mlp, "shared"), "ff")


def _check_layer(i: int, layer) -> Dict:
    where = f"layers[{i}]."
    kind = layer.get("type") if isinstance(layer, dict) else None
    if kind not in ("retention", "parallel"):
        raise ConfigError(f"config.json {where}type is {kind!r}; known: retention, parallel")
    m = _table(where, layer, "mixer")
    if kind == "retention":
        w = where + "mixer."
        heads, dim = _int(w, m, "heads"), _int(w, m, "dim")
        _int(w, m, "vdim")
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or \
                any(isinstance(d, bool) or not isinstance(d, (int, float)) or not math.isfinite(d) for d in decay):
            raise ConfigError(f"config.json {w}decay must list one number per head ({heads})")
        _check_rot(w, m, dim)
    else:
        left, right = _table(where + "mixer.", m, "left"), _table(where + "mixer.", m, "right")
        w = where + "mixer.left."
        for key in ("heads", "kv_heads", "dim", "vdim", "conv"):
            _int(w, left, key)
        _num(w, left, "scale")
        _num(w, left, "softcap")
        _int(w + "mask.", _table(w, left, "mask"), "size")
        if left["heads"] % left["kv_heads"] != 0:
            raise ConfigError(f"config.json {w[:-1]}: {left['heads']} heads are not a multiple of {left['kv_heads']} kv_heads")
        _check_rot(w, left, left["dim"])
        for key in ("heads", "dim"):
            _int(where + "mixer.right.", right, key)
        if right.get("decay_rank") is not None:
            _int(where + "mixer.right.", right, "decay_rank")
        _num(where + "mixer.", m, "left_scale", positive=False)
        _num(where + "mixer.", m, "right_scale", positive=False)
    _check_mlp(where, layer.get("mlp"))
    return copy.deepcopy(layer)


@dataclass(frozen=True)
class RoravikConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    logit_softcap: float
    layers: Tuple[Dict, ...]               # as config.json has them, validated
    loop: Optional[Tuple[int, int, int]] = None      # (start, stop, times)
    max_positions: Optional[int] = None
    eos_token_id: Optional[Tuple[int, ...]] = None

    @classmethod
    def from_dict(cls, raw: Dict) -> "RoravikConfig":
        if raw.get("architecture") != ARCHITECTURE:
            raise UnsupportedArchitectureError(
                f"config.json names architecture {raw.get('architecture')!r}; this class reads {ARCHITECTURE!r}")
        vocab, width = _int("", raw, "vocab"), _int("", raw, "width")
        eps = _num("norm.", _table("", raw, "norm"), "eps")
        scale = _num("embedding.", _table("", raw, "embedding"), "scale")
        cap = _num("", raw, "logit_softcap")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json key 'layers' must be a list with at least one layer")
        checked: List[Dict] = [_check_layer(i, layer) for i, layer in enumerate(layers)]
        values = dict(vocab=vocab, width=width, eps=eps, embedding_scale=scale, logit_softcap=cap, layers=tuple(checked))
        if raw.get("loop") is not None:
            lp = _table("", raw, "loop")
            for key in ("start", "stop"):
                v = lp.get(key)
                if isinstance(v, bool) or not isinstance(v, int) or v < 0:
                    raise ConfigError(f"config.json loop.{key} must be a layer index, found {v!r}")
            times = _int("loop.", lp, "times")
            if not lp["start"] < lp["stop"] <= len(checked):
                raise ConfigError(f"config.json loop: layers {lp['start']} .. {lp['stop']} - 1 are no stretch of the "
                                  f"{len(checked)} layers")
            values["loop"] = (lp["start"], lp["stop"], times)
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
             "embedding": {"scale": self.embedding_scale}, "logit_softcap": self.logit_softcap,
             "layers": copy.deepcopy(list(self.layers))}
        if self.loop is not None:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.max_positions is not None:
            d["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    def with_shapes(self, shapes: Dict[str, Tuple[int, ...]]) -> "RoravikConfig":
        """The configuration with what only the checkpoint's tensor shapes say filled in: the inner
        width of every decay's two small matrices (``l<i>.mix.right.w1`` is ``[rank, width]``)."""
        layers = []
        for i, layer in enumerate(self.layers):
            layer = copy.deepcopy(layer)
            if layer["type"] == "parallel" and layer["mixer"]["right"].get("decay_rank") is None:
                shape = shapes.get(f"l{i}.mix.right.w1")
                if shape is not None and len(shape) == 2:
                    layer["mixer"]["right"]["decay_rank"] = int(shape[0])
            layers.append(layer)
        return replace(self, layers=tuple(layers))

    def schedule(self) -> Tuple[ScheduleEntry, ...]:
        n = len(self.layers)
        if self.loop is None:
            return tuple(ScheduleEntry(layer=i) for i in range(n))
        start, stop, times = self.loop
        entries = [ScheduleEntry(layer=i) for i in range(start)]
        for rep in range(times):
            entries += [ScheduleEntry(layer=i, add_embedding=rep > 0 and i == start) for i in range(start, stop)]
        return tuple(entries + [ScheduleEntry(layer=i) for i in range(stop, n)])

    def to_model_spec(self) -> ModelSpec:
        def norm() -> NormSpec:
            return NormSpec(size=self.width, eps=self.eps, unit_offset=True)
        blocks = []
        for layer in self.layers:
            m = layer["mixer"]
            if layer["type"] == "retention":
                rot = m["rot"]
                mixer = RetentionSpec(hidden=self.width, n_heads=m["heads"], head_dim=m["dim"], v_head_dim=m["vdim"],
                                      decay=tuple(float(d) for d in m["decay"]), eps=self.eps,
                                      position=RopeSpec(head_dim=m["dim"], rot_dim=rot["dims"], theta=float(rot["base"])))
            else:
                left, right = m["left"], m["right"]
                rot = left["rot"]
                attention = AttentionSpec(hidden=self.width, n_heads=left["heads"], n_kv_heads=left["kv_heads"],
                                          head_dim=left["dim"], v_head_dim=left["vdim"], scale=float(left["scale"]),
                                          window=left["mask"]["size"], qk_norm=None,
                                          position=RopeSpec(head_dim=left["dim"], rot_dim=rot["dims"], theta=float(rot["base"])),
                                          sink=True, sink_learned=True, softcap=float(left["softcap"]), conv=left["conv"])
                recurrence = TimeMixSpec(hidden=self.width, n_heads=right["heads"], head_dim=right["dim"],
                                         decay_rank=right.get("decay_rank") or DEFAULT_DECAY_RANK, eps=self.eps)
                mixer = ParallelMixerSpec(hidden=self.width, branches=(("left", attention), ("right", recurrence)),
                                          weight=1.0, eps=self.eps, normed=False,
                                          branch_weights=(float(m["left_scale"]), float(m["right_scale"])))
            mlp = layer.get("mlp")
            if mlp is None:
                ffn = None
            elif mlp["kind"] == "dense":
                ffn = GatedMlpSpec(hidden=self.width, intermediate=mlp["ff"], activation=DENSE_ACTIVATION,
                                   limit=float(mlp["limit"]), up_offset=DENSE_UP_OFFSET)
            else:
                r = mlp["router"]
                g = r.get("groups")
                shared = mlp.get("shared")
                ffn = RoutedExpertsSpec(hidden=self.width, n_experts=r["experts"], top=r["top"],
                                        intermediate=mlp["expert"]["ff"], activation="silu",
                                        groups=None if g is None else (g["count"], g["keep"]), sum_eps=EXPERT_SUM_EPS,
                                        weighting="sigmoid", correction=True, group_score=GROUP_SCORE,
                                        shared_intermediate=None if shared is None else shared["ff"],
                                        shared_gate=shared is not None)
            blocks.append(BlockSpec(mixer=mixer, ffn=ffn, mixer_norm=norm(), ffn_norm=None if ffn is None else norm(),
                                    arrangement="sandwich_norm", mixer_out_norm=norm(),
                                    ffn_out_norm=None if ffn is None else norm()))
        spec = ModelSpec(architecture=ARCHITECTURE, vocab=self.vocab, hidden=self.width, layers=tuple(blocks),
                         schedule=self.schedule(), final_norm=norm(), tie_lm_head=True,
                         max_positions=self.max_positions or UNBOUNDED_POSITIONS, embed_scale=self.embedding_scale,
                         eos_token_ids=self.eos_token_id or (), logit_softcap=self.logit_softcap)
        spec.validate()
        return spec


def checkpoint_names(spec: ModelSpec) -> Dict[str, str]:
    """Internal parameter name -> tensor name in the checkpoint: ``embed``, ``l<i>.norm1|norm1b|norm2|norm2b``,
    ``l<i>.mix.q|k|v|g|o`` (retention), ``l<i>.mix.left.q|k|v|o|sink`` and ``l<i>.mix.left.q.conv|k.conv|v.conv``,
    ``l<i>.mix.right.mu.r|k|v|g|w``, ``l<i>.mix.right.r|k|v|g|o|w1|w2|w0|u|norm``, ``l<i>.mlp.gate|up|down`` or
    ``l<i>.mlp.router|correction``, ``l<i>.mlp.e<j>.gate|up|down`` and ``l<i>.mlp.shared.gate|up|down|sg``,
    ``final.norm``."""
    names = {"embed.weight": "embed", "final_norm.weight": "final.norm"}
    for i, block in enumerate(spec.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"], names[dst + "mixer_out_norm.weight"] = src + "norm1", src + "norm1b"
        if block.mixer.kind == "retention":
            for p in ("q", "k", "v", "g", "o"):
                names[dst + f"mixer.{p}_proj.weight"] = src + f"mix.{p}"
        else:
            for p in ("q", "k", "v"):
                names[dst + f"mixer.left.{p}_proj.weight"] = src + f"mix.left.{p}"
                names[dst + f"mixer.left.{p}_conv.weight"] = src + f"mix.left.{p}.conv"
            names[dst + "mixer.left.o_proj.weight"] = src + "mix.left.o"
            names[dst + "mixer.left.sink"] = src + "mix.left.sink"
            for p in ("r", "k", "v", "g", "w"):
                names[dst + f"mixer.right.mu_{p}"] = src + f"mix.right.mu.{p}"
            for p in ("r", "k", "v", "g", "o"):
                names[dst + f"mixer.right.{p}_proj.weight"] = src + f"mix.right.{p}"
            for internal, stored in (("w1.weight", "w1"), ("w2.weight", "w2"), ("w0", "w0"), ("u", "u"), ("norm.weight", "norm")):
                names[dst + "mixer.right." + internal] = src + "mix.right." + stored
        if block.ffn is None:
            continue
        names[dst + "ffn_norm.weight"], names[dst + "ffn_out_norm.weight"] = src + "norm2", src + "norm2b"
        if block.ffn.kind == "routed_experts":
            names[dst + "ffn.router.weight"] = src + "mlp.router"
            names[dst + "ffn.correction"] = src + "mlp.correction"
            for e in range(block.ffn.n_experts):
                for p in ("gate", "up", "down"):
                    names[dst + f"ffn.experts.{e}.{p}_proj.weight"] = src + f"mlp.e{e}.{p}"
            if block.ffn.shared_intermediate is not None:
                for p in ("gate", "up", "down"):
                    names[dst + f"ffn.shared.{p}_proj.weight"] = src + f"mlp.shared.{p}"
                names[dst + "ffn.shared.gate.weight"] = src + "mlp.shared.sg"
        else:
            for p in ("gate", "up", "down"):
                names[dst + f"ffn.{p}_proj.weight"] = src + f"mlp.{p}"
    return names


def unused_tensors(spec: ModelSpec) -> Tuple[str, ...]:
    """Tensors a checkpoint may hold that the model does not read: the second norms of a layer
    without a feed-forward."""
    out = []
    for i, block in enumerate(spec.layers):
        if block.ffn is None:
            out += [f"l{i}.norm2", f"l{i}.norm2b"]
    return tuple(out)
