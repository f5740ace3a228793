"""Typed configuration of the Dokulix decoder, read from config.json.

A Dokulix model is a list of pre-norm layers, each with one of two mixers and an optional
gated feed-forward, a stretch of layers that runs several times in a row with the same weights,
and norms whose stored weight lies around zero.  config.json gives every size layer by layer:

* ``architecture``: ``"Dokulix"``; ``vocab``, ``width``; ``norm.eps``;
* ``layers[i]``: ``type`` (``attention`` or ``latent_attention``), ``mixer`` (its sizes and
  constants) and ``mlp`` (``{"kind": "dense", "ff": n}`` or null);
* ``loop`` (optional): ``start``, ``stop``, ``times``: layers ``start .. stop-1`` run ``times``
  times, each pass with cache lines of its own, and row ``t`` of the tensor ``loop.step`` is
  added to the residual stream before the first layer of pass ``t``.

Constants the design fixes live here: the distance slopes ``2^(-8 (h+1) / H)`` of the biased
attention, its sink, the rectifier of the feed-forward, the rotation's pairing.
"""
from __future__ import annotations

import copy
import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

from ..errors import ConfigError, UnsupportedArchitectureError
from .spec import (AttentionSpec, BlockSpec, GatedMlpSpec, LatentAttentionSpec, ModelSpec, NormSpec, RopeSpec,
                   ScheduleEntry)

ARCHITECTURE = "Dokulix"
DEFAULT_MAX_POSITIONS = 1 << 20      # the design has no bound of its own; config.json may give "max_positions"

_MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale", "mask"),
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "mask", "rot"),
}


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


def distance_slopes(n_heads: int) -> Tuple[float, ...]:
    """Slope of head ``h``: ``2^(-8 (h + 1) / H)``."""
    return tuple(2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads))


@dataclass(frozen=True)
class DokulixConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[Dict, ...]               # as config.json has them, validated
    loop: Optional[Tuple[int, int, int]]   # (start, stop, times)
    max_positions: int = DEFAULT_MAX_POSITIONS
    eos_token_id: Optional[Tuple[int, ...]] = None

    # ---- reading ---------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict) -> "DokulixConfig":
        if raw.get("architecture") != ARCHITECTURE:
            raise UnsupportedArchitectureError(
                f"config.json names architecture {raw.get('architecture')!r}; this class reads {ARCHITECTURE!r}")
        vocab, width = _int("", raw, "vocab"), _int("", raw, "width")
        if not isinstance(raw.get("norm"), dict):
            raise ConfigError("config.json lacks the table 'norm'")
        eps = _num("norm.", raw["norm"], "eps")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json key 'layers' must be a list with at least one layer")
        checked: List[Dict] = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind not in _MIXER_KEYS:
                raise ConfigError(f"config.json {where}type is {kind!r}; known: {', '.join(sorted(_MIXER_KEYS))}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json lacks the table {where}mixer")
            for key in _MIXER_KEYS[kind]:
                if key in ("scale",):
                    _num(where + "mixer.", m, key)
                elif key == "mask":
                    if not isinstance(m.get("mask"), dict):
                        raise ConfigError(f"config.json lacks the table {where}mixer.mask")
                    _int(where + "mixer.mask.", m["mask"], "size")
                elif key == "rot":
                    if not isinstance(m.get("rot"), dict):
                        raise ConfigError(f"config.json lacks the table {where}mixer.rot")
                    _num(where + "mixer.rot.", m["rot"], "base")
                    dims = _int(where + "mixer.rot.", m["rot"], "dims")
                    if dims % 2 != 0 or dims > _int(where + "mixer.", m, "rot_dim"):
                        raise ConfigError(f"config.json {where}mixer.rot.dims must be even and at most rot_dim "
                                          "(pairs i, i + dims/2 of the rotated part)")
                else:
                    _int(where + "mixer.", m, key)
            if kind == "attention" and m["heads"] % m["kv_heads"] != 0:
                raise ConfigError(f"config.json {where}mixer: {m['heads']} heads are not a multiple of "
                                  f"{m['kv_heads']} kv_heads")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json {where}mlp must be null or of kind 'dense', found {mlp!r}")
                _int(where + "mlp.", mlp, "ff")
            checked.append(copy.deepcopy(layer))
        loop = None
        if raw.get("loop") is not None:
            lp = raw["loop"]
            if not isinstance(lp, dict):
                raise ConfigError("config.json key 'loop' must be a table")
            start = lp.get("start")
            if isinstance(start, bool) or not isinstance(start, int) or start < 0:
                raise ConfigError(f"config.json loop.start must be a layer index, found {start!r}")
            stop, times = _int("loop.", lp, "stop"), _int("loop.", lp, "times")
            if not start < stop <= len(checked):
                raise ConfigError(f"config.json loop: layers {start} .. {stop - 1} are not a stretch of the "
                                  f"{len(checked)} layers")
            loop = (start, stop, times)
        values = dict(vocab=vocab, width=width, eps=eps, layers=tuple(checked), loop=loop)
        if "max_positions" in raw:
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
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    # ---- derived ---------------------------------------------------------
    def run_order(self) -> List[Tuple[int, Optional[int]]]:
        """``(layer, pass)`` in the order the layers run; ``pass`` is the number of the loop's pass
        on the first layer of each pass and None elsewhere."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        start, stop, times = self.loop
        order: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(start)]
        for t in range(times):
            order += [(i, t if i == start else None) for i in range(start, stop)]
        order += [(i, None) for i in range(stop, n)]
        return order

    def to_model_spec(self) -> ModelSpec:
        hidden_norm = NormSpec(size=self.width, eps=self.eps, unit_offset=True)
        blocks = []
        for layer in self.layers:
            m = layer["mixer"]
            if layer["type"] == "attention":
                head_norm = NormSpec(size=m["dim"], eps=self.eps)
                mixer = AttentionSpec(hidden=self.width, n_heads=m["heads"], n_kv_heads=m["kv_heads"],
                                      head_dim=m["dim"], v_head_dim=m["vdim"], scale=float(m["scale"]),
                                      qk_norm=head_norm, position=None, bias=True, chunk=m["mask"]["size"],
                                      distance_slopes=distance_slopes(m["heads"]), sink=True)
            else:
                rope = RopeSpec(head_dim=m["rot_dim"], rot_dim=m["rot"]["dims"], theta=float(m["rot"]["base"]))
                mixer = LatentAttentionSpec(hidden=self.width, n_heads=m["heads"], head_dim=m["dim"],
                                            rot_dim=m["rot_dim"], v_head_dim=m["vdim"], q_rank=m["q_rank"],
                                            kv_rank=m["kv_rank"], scale=float(m["scale"]),
                                            q_norm=NormSpec(size=m["q_rank"], eps=self.eps),
                                            kv_norm=NormSpec(size=m["kv_rank"], eps=self.eps),
                                            position=rope, window=m["mask"]["size"], gate=True)
            mlp = layer.get("mlp")
            ffn = None if mlp is None else GatedMlpSpec(hidden=self.width, intermediate=mlp["ff"], activation="relu")
            blocks.append(BlockSpec(mixer=mixer, ffn=ffn, mixer_norm=hidden_norm,
                                    ffn_norm=None if ffn is None else hidden_norm))
        schedule = tuple(ScheduleEntry(layer=i, offset_row=t) for i, t in self.run_order())
        spec = ModelSpec(architecture=ARCHITECTURE, vocab=self.vocab, hidden=self.width, layers=tuple(blocks),
                         schedule=schedule, final_norm=hidden_norm, tie_lm_head=False,
                         max_positions=self.max_positions, eos_token_ids=self.eos_token_id or (),
                         pass_offsets=0 if self.loop is None else self.loop[2])
        spec.validate()
        return spec


def checkpoint_names(spec: ModelSpec) -> Dict[str, str]:
    """Internal parameter name -> tensor name in the checkpoint: ``embed``, ``loop.step``,
    ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.gate|up|down``, ``final.norm``, ``head``."""
    names = {"embed.weight": "embed", "final_norm.weight": "final.norm", "lm_head.weight": "head"}
    if spec.pass_offsets:
        names["pass_offset.weight"] = "loop.step"
    for i, block in enumerate(spec.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "norm1"
        if block.mixer.kind == "attention":
            for p in ("q", "k", "v", "o"):
                names[dst + f"mixer.{p}_proj.weight"] = src + f"mix.{p}"
                names[dst + f"mixer.{p}_proj.bias"] = src + f"mix.{p}.b"
            names[dst + "mixer.q_norm.weight"] = src + "mix.q.norm"
            names[dst + "mixer.k_norm.weight"] = src + "mix.k.norm"
        else:
            for p in ("dq", "uq", "dkv", "uk", "uv", "g"):
                names[dst + f"mixer.{p}.weight"] = src + f"mix.{p}"
            names[dst + "mixer.dq_norm.weight"] = src + "mix.dq.norm"
            names[dst + "mixer.dkv_norm.weight"] = src + "mix.dkv.norm"
            names[dst + "mixer.o_proj.weight"] = src + "mix.o"
        if block.ffn is not None:
            names[dst + "ffn_norm.weight"] = src + "norm2"
            for p in ("gate", "up", "down"):
                names[dst + f"ffn.{p}_proj.weight"] = src + f"mlp.{p}"
    return names


def unused_tensors(spec: ModelSpec) -> Tuple[str, ...]:
    """Tensors a checkpoint may hold that the model does not read: the second norm of a layer
    without a feed-forward, the loop's vectors of a model without a loop."""
    names = [f"l{i}.norm2" for i, block in enumerate(spec.layers) if block.ffn is None]
    if not spec.pass_offsets:
        names.append("loop.step")
    return tuple(names)
