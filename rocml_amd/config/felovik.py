"""Typed configuration of the Felovik decoder, read from config.json.

A Felovik model is a list of layers whose norms follow the residual sums (``x <- norm(alpha x + sublayer(x))``;
a sublayer is fed the stream as it is).  A layer's mixer is a pair of mixers that run on one
input, a gated softmax attention without rotation (``left``) and a state-space recurrence with a
scalar decay per head (``right``), whose outputs are normed over the width, each with a gain of its
own, and averaged.  Its feed-forward is dense (gate and up values held under a limit) or a mixture
of small experts, or absent.  Positions enter through a learned table added to the scaled token
embedding, and through a stretch of the queries that grows with the logarithm of the position.
config.json gives every size layer by layer:

* ``architecture``: ``"Felovik"``; ``vocab``, ``width``, ``max_positions``; ``norm.eps``;
  ``embedding.scale``; ``postln_alpha``;
* ``layers[i]``: ``type`` (``parallel``), ``mixer.left`` (``heads``, ``kv_heads``, ``dim``, ``vdim``,
  ``scale``, ``q_temp`` with ``coef`` and ``every``, or null), ``mixer.right`` (``heads``, ``vdim``,
  ``state``, ``groups``, ``conv``, ``norm_groups``) and ``mlp``: null, ``{"kind": "dense", "ff",
  "limit"}`` or ``{"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "groups": {"count",
  "keep"} or null}}``.

Constants the design fixes live here: the 1.702 in the dense feed-forward's gate, the one added to
its up values, the half in front of the two mixers' sum, the 1e-20 under the experts' weights.
"""
from __future__ import annotations

import copy
import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

from ..errors import ConfigError, UnsupportedArchitectureError
from .spec import (AttentionSpec, BlockSpec, GatedMlpSpec, ModelSpec, NormSpec, ParallelMixerSpec, RoutedExpertsSpec,
                   StateSpaceSpec, TokenPositionTableSpec, default_schedule)

ARCHITECTURE = "Felovik"
BRANCH_WEIGHT = 0.5           # half the sum of the two mixers' normed outputs
DENSE_ACTIVATION = "sigmoid_1702"
DENSE_UP_OFFSET = 1.0
EXPERT_SUM_EPS = 1e-20


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


def _check_layer(i: int, layer) -> Dict:
    where = f"layers[{i}]."
    if not isinstance(layer, dict) or layer.get("type") != "parallel":
        kind = layer.get("type") if isinstance(layer, dict) else None
        raise ConfigError(f"config.json {where}type is {kind!r}; known: parallel")
    m = _table(where, layer, "mixer")
    left, right = _table(where + "mixer.", m, "left"), _table(where + "mixer.", m, "right")
    for key in ("heads", "kv_heads", "dim", "vdim"):
        _int(where + "mixer.left.", left, key)
    _num(where + "mixer.left.", left, "scale")
    if left["heads"] % left["kv_heads"] != 0:
        raise ConfigError(f"config.json {where}mixer.left: {left['heads']} heads are not a multiple of {left['kv_heads']} kv_heads")
    if left.get("q_temp") is not None:
        qt = _table(where + "mixer.left.", left, "q_temp")
        _num(where + "mixer.left.q_temp.", qt, "coef", positive=False)
        _int(where + "mixer.left.q_temp.", qt, "every")
    for key in ("heads", "vdim", "state", "groups", "conv", "norm_groups"):
        _int(where + "mixer.right.", right, key)
    if right["heads"] % right["groups"] != 0:
        raise ConfigError(f"config.json {where}mixer.right: {right['heads']} heads do not fall into {right['groups']} groups")
    if (right["heads"] * right["vdim"]) % right["norm_groups"] != 0:
        raise ConfigError(f"config.json {where}mixer.right: heads * vdim does not fall into {right['norm_groups']} norm_groups")
    mlp = layer.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
            raise ConfigError(f"config.json {where}mlp must be null or of kind 'dense' or 'moe', found {mlp!r}")
        if mlp["kind"] == "dense":
            _int(where + "mlp.", mlp, "ff")
            if mlp.get("limit") is not None:
                _num(where + "mlp.", mlp, "limit")
        else:
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
    return copy.deepcopy(layer)


@dataclass(frozen=True)
class FelovikConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    embedding_scale: float
    postln_alpha: float
    layers: Tuple[Dict, ...]               # as config.json has them, validated
    eos_token_id: Optional[Tuple[int, ...]] = None

    @classmethod
    def from_dict(cls, raw: Dict) -> "FelovikConfig":
        if raw.get("architecture") != ARCHITECTURE:
            raise UnsupportedArchitectureError(
                f"config.json names architecture {raw.get('architecture')!r}; this class reads {ARCHITECTURE!r}")
        vocab, width = _int("", raw, "vocab"), _int("", raw, "width")
        max_positions = _int("", raw, "max_positions")
        eps = _num("norm.", _table("", raw, "norm"), "eps")
        scale = _num("embedding.", _table("", raw, "embedding"), "scale")
        alpha = _num("", raw, "postln_alpha")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json key 'layers' must be a list with at least one layer")
        checked: List[Dict] = [_check_layer(i, layer) for i, layer in enumerate(layers)]
        values = dict(vocab=vocab, width=width, max_positions=max_positions, eps=eps, embedding_scale=scale,
                      postln_alpha=alpha, layers=tuple(checked))
        eos = raw.get("eos_token_id")
        if eos is not None:
            ids = list(eos) if isinstance(eos, (list, tuple)) else [eos]
            for t in ids:
                if isinstance(t, bool) or not isinstance(t, int) or not 0 <= t < vocab:
                    raise ConfigError(f"config.json key 'eos_token_id' must name token ids below vocab, found {eos!r}")
            values["eos_token_id"] = tuple(ids)
        return cls(**values)

    def to_dict(self) -> Dict:
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
             "norm": {"eps": self.eps}, "embedding": {"scale": self.embedding_scale}, "postln_alpha": self.postln_alpha,
             "layers": copy.deepcopy(list(self.layers))}
        if self.eos_token_id is not None:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    def to_model_spec(self) -> ModelSpec:
        hidden_norm = NormSpec(size=self.width, eps=self.eps)
        blocks = []
        for layer in self.layers:
            left, right = layer["mixer"]["left"], layer["mixer"]["right"]
            qt = left.get("q_temp")
            attention = AttentionSpec(hidden=self.width, n_heads=left["heads"], n_kv_heads=left["kv_heads"],
                                      head_dim=left["dim"], v_head_dim=left["vdim"], scale=float(left["scale"]),
                                      qk_norm=NormSpec(size=left["dim"], eps=self.eps, learned=False), position=None,
                                      q_temp=None if qt is None else (float(qt["coef"]), int(qt["every"])), gate=True)
            recurrence = StateSpaceSpec(hidden=self.width, n_heads=right["heads"], head_dim=right["vdim"],
                                        state=right["state"], groups=right["groups"], conv=right["conv"],
                                        norm_groups=right["norm_groups"], eps=self.eps)
            mixer = ParallelMixerSpec(hidden=self.width, branches=(("left", attention), ("right", recurrence)),
                                      weight=BRANCH_WEIGHT, eps=self.eps)
            mlp = layer.get("mlp")
            if mlp is None:
                ffn = None
            elif mlp["kind"] == "dense":
                ffn = GatedMlpSpec(hidden=self.width, intermediate=mlp["ff"], activation=DENSE_ACTIVATION,
                                   limit=None if mlp.get("limit") is None else float(mlp["limit"]), up_offset=DENSE_UP_OFFSET)
            else:
                r = mlp["router"]
                g = r.get("groups")
                ffn = RoutedExpertsSpec(hidden=self.width, n_experts=r["experts"], top=r["top"],
                                        intermediate=mlp["expert"]["ff"], activation="silu",
                                        groups=None if g is None else (g["count"], g["keep"]), sum_eps=EXPERT_SUM_EPS)
            blocks.append(BlockSpec(mixer=mixer, ffn=ffn, mixer_norm=hidden_norm, ffn_norm=None if ffn is None else hidden_norm,
                                    arrangement="post_norm", residual_scale=self.postln_alpha))
        spec = ModelSpec(architecture=ARCHITECTURE, vocab=self.vocab, hidden=self.width, layers=tuple(blocks),
                         schedule=default_schedule(len(blocks)), final_norm=hidden_norm, tie_lm_head=False,
                         max_positions=self.max_positions, eos_token_ids=self.eos_token_id or (),
                         embedding=TokenPositionTableSpec(vocab=self.vocab, hidden=self.width,
                                                          max_positions=self.max_positions, scale=self.embedding_scale))
        spec.validate()
        return spec


def checkpoint_names(spec: ModelSpec) -> Dict[str, str]:
    """Internal parameter name -> tensor name in the checkpoint: ``embed``, ``pos``, ``l<i>.norm1|norm2``,
    ``l<i>.mix.left.q|k|v|g|o|out``, ``l<i>.mix.right.in|conv|conv.b|dt_bias|A_log|D|norm|o|out``,
    ``l<i>.mlp.gate|up|down`` or ``l<i>.mlp.router`` and ``l<i>.mlp.e<j>.gate|up|down``, ``final.norm``, ``head``."""
    names = {"embed.weight": "embed", "embed.positions": "pos", "final_norm.weight": "final.norm", "lm_head.weight": "head"}
    for i, block in enumerate(spec.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "norm1"
        for p in ("q", "k", "v", "g", "o"):
            names[dst + f"mixer.left.{p}_proj.weight"] = src + f"mix.left.{p}"
        names[dst + "mixer.left.out_norm.weight"] = src + "mix.left.out"
        for internal, stored in (("in_proj.weight", "in"), ("conv.weight", "conv"), ("conv.bias", "conv.b"), ("dt_bias", "dt_bias"),
                                 ("A_log", "A_log"), ("D", "D"), ("norm.weight", "norm"), ("out_proj.weight", "o"),
                                 ("out_norm.weight", "out")):
            names[dst + "mixer.right." + internal] = src + "mix.right." + stored
        if block.ffn is None:
            continue
        names[dst + "ffn_norm.weight"] = src + "norm2"
        if block.ffn.kind == "routed_experts":
            names[dst + "ffn.router.weight"] = src + "mlp.router"
            for e in range(block.ffn.n_experts):
                for p in ("gate", "up", "down"):
                    names[dst + f"ffn.experts.{e}.{p}_proj.weight"] = src + f"mlp.e{e}.{p}"
        else:
            for p in ("gate", "up", "down"):
                names[dst + f"ffn.{p}_proj.weight"] = src + f"mlp.{p}"
    return names


def unused_tensors(spec: ModelSpec) -> Tuple[str, ...]:
    """Tensors a checkpoint may hold that the model does not read: the second norm of a layer
    without a feed-forward."""
    return tuple(f"l{i}.norm2" for i, block in enumerate(spec.layers) if block.ffn is None)
