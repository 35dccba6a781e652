"""Typed configuration of Zifunex, read from its own config.json keys.

A Zifunex folder names its design in ``architecture`` and gives every size and
constant that may differ between models: ``vocab``, ``width``, ``streams``,
``norm.eps``, ``embedding.bigram`` (``buckets``, ``mul_prev``, ``mul_cur``),
``layers`` (each with ``type``, ``mixer`` and ``mlp``) and ``loop`` (``start``,
``stop``, ``times``).  Nothing has a default: a key that is missing is an
error, so that a model never runs on a guess.  One size is not in the file,
the inner size of a ``gla`` mixer's decay projections; it is read from the
tensors (a configuration written for a random model names it as ``rank``).
"""

from __future__ import annotations

import copy
import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import InvalidInput, Unsupported

ARCHITECTURE = "Zifunex"


def _get(raw: Dict[str, Any], key: str, where: str):
    if not isinstance(raw, dict) or key not in raw:
        raise InvalidInput(f"config.json {where} has no {key!r}")
    return raw[key]


def _int(raw, key, where, least=1) -> int:
    value = _get(raw, key, where)
    if isinstance(value, bool) or not isinstance(value, int) or value < least:
        raise InvalidInput(f"config.json {where}.{key} must be an integer of at least {least}; got {value!r}")
    return value


def _number(raw, key, where) -> float:
    value = _get(raw, key, where)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(float(value)) or float(value) <= 0.0:
        raise InvalidInput(f"config.json {where}.{key} must be a finite positive number; got {value!r}")
    return float(value)


@dataclass
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    rot_dims: int
    rot_base: float
    scale: float
    softcap: float

    @classmethod
    def from_dict(cls, raw, where):
        rot = _get(raw, "rot", where)
        out = cls(_int(raw, "heads", where), _int(raw, "kv_heads", where), _int(raw, "dim", where), _int(raw, "vdim", where),
                  _int(rot, "dims", where + ".rot", least=2), _number(rot, "base", where + ".rot"), _number(raw, "scale", where),
                  _number(raw, "softcap", where))
        if out.heads % out.kv_heads:
            raise InvalidInput(f"config.json {where}: {out.heads} heads do not divide into {out.kv_heads} kv_heads")
        if out.rot_dims % 2 or out.rot_dims > out.dim:
            raise InvalidInput(f"config.json {where}.rot.dims must be even and at most dim ({out.dim}); got {out.rot_dims}")
        return out


@dataclass
class ScanSizes:
    inner: int
    state: int
    dt_rank: int
    conv: int

    @classmethod
    def from_dict(cls, raw, where):
        return cls(_int(raw, "inner", where), _int(raw, "state", where), _int(raw, "dt_rank", where), _int(raw, "conv", where))


@dataclass
class GlaSizes:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: Optional[int]

    @classmethod
    def from_dict(cls, raw, where):
        rank = _int(raw, "rank", where) if isinstance(raw, dict) and "rank" in raw else None
        return cls(_int(raw, "heads", where), _int(raw, "dim", where), _int(raw, "vdim", where), _number(raw, "tau", where), rank)


@dataclass
class LayerSizes:
    type: str  # "parallel" or "gla"
    left: Optional[AttentionSizes] = None
    right: Optional[ScanSizes] = None
    gla: Optional[GlaSizes] = None
    ff: Optional[int] = None  # None: the layer has no feed-forward


@dataclass
class ZifunexConfig:
    vocab: int
    width: int
    streams: int
    eps: float
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: List[LayerSizes]
    loop_start: int
    loop_stop: int
    loop_times: int
    raw: Dict[str, Any] = field(default_factory=dict)
    architecture: str = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ZifunexConfig":
        bigram = _get(_get(raw, "embedding", "file"), "bigram", "embedding")
        layers = _get(raw, "layers", "file")
        if not isinstance(layers, list) or not layers:
            raise InvalidInput("config.json layers must be a list with at least one layer")
        out_layers = []
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            kind = _get(layer, "type", where)
            mixer = _get(layer, "mixer", where)
            mlp = _get(layer, "mlp", where)
            ff = None
            if mlp is not None:
                if _get(mlp, "kind", where + ".mlp") != "dense":
                    raise Unsupported(f"config.json {where}.mlp.kind {mlp['kind']!r}; this design has dense feed-forwards")
                ff = _int(mlp, "ff", where + ".mlp")
            if kind == "parallel":
                out_layers.append(LayerSizes(kind, left=AttentionSizes.from_dict(_get(mixer, "left", where + ".mixer"), where + ".mixer.left"),
                                             right=ScanSizes.from_dict(_get(mixer, "right", where + ".mixer"), where + ".mixer.right"), ff=ff))
            elif kind == "gla":
                out_layers.append(LayerSizes(kind, gla=GlaSizes.from_dict(mixer, where + ".mixer"), ff=ff))
            else:
                raise Unsupported(f"config.json {where}.type {kind!r}; this design has the mixers 'parallel' and 'gla'")
        loop = raw.get("loop")
        start, stop, times = 0, 0, 1
        if loop is not None:
            start, stop = _int(loop, "start", "loop", least=0), _int(loop, "stop", "loop", least=0)
            times = _int(loop, "times", "loop", least=1)
            if not start <= stop <= len(out_layers):
                raise InvalidInput(f"config.json loop covers layers {start} to {stop - 1}, but there are {len(out_layers)}")
        return cls(
            vocab=_int(raw, "vocab", "file"), width=_int(raw, "width", "file"), streams=_int(raw, "streams", "file"),
            eps=_number(_get(raw, "norm", "file"), "eps", "norm"), buckets=_int(bigram, "buckets", "embedding.bigram"),
            mul_prev=_int(bigram, "mul_prev", "embedding.bigram", least=0), mul_cur=_int(bigram, "mul_cur", "embedding.bigram", least=0),
            layers=out_layers, loop_start=start, loop_stop=stop, loop_times=times, raw=copy.deepcopy(raw))

    def layer_runs(self) -> List[int]:
        """The layers in the order they run: the looped stretch as often as the loop says, with the same weights."""
        inside = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + inside * self.loop_times + list(range(self.loop_stop, len(self.layers)))

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
