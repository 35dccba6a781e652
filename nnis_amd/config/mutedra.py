"""Typed configuration of Mutedra, read from its own config.json keys.

A Mutedra folder names its design in ``architecture`` and gives every size and
constant that may differ between models: ``vocab``, ``width``, ``norm.eps``,
``embedding.scale``, ``logit_softcap``, ``layers`` (each with ``type``, the
mixer's sizes in ``mixer`` and ``mlp`` -- ``{"kind": "dense", "ff": n}`` or
null) and ``loop`` (``start``, ``stop``, ``times``).  No size has a default: a
size that is missing is an error, so that a model never runs on a guess.  A
mechanism that the file does not mention at all does not exist in that model:
without ``loop`` no layer runs twice and no pass begins, without
``embedding.scale`` or ``logit_softcap`` rows and logits stay as they are,
an ``attention`` mixer without ``mask`` sees every earlier key and without
``bias_max`` has no bias by distance.  One
size is not in the file, the number of rows of an ``attention`` mixer's table
of distance biases; it is read from the tensor (a configuration written for a
random model names it as ``bias_buckets``).
"""

from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import InvalidInput, Unsupported
from .zifunex import _get, _int, _number

ARCHITECTURE = "Mutedra"
MIXERS = ("attention", "latent_attention", "latent_attention_2")


@dataclass
class WindowedSizes:
    """Mixer ``attention``: grouped heads, a sliding window that keeps the first tokens, a bias by distance."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int  # 0: no window, every earlier key is seen
    keep_first: int
    bias_max: int  # 0: no bias by distance
    bias_buckets: Optional[int]

    @classmethod
    def from_dict(cls, raw, where):
        mask = raw.get("mask") if isinstance(raw, dict) else None
        biased = isinstance(raw, dict) and raw.get("bias_max") is not None
        out = cls(_int(raw, "heads", where), _int(raw, "kv_heads", where), _int(raw, "dim", where), _int(raw, "vdim", where),
                  _number(raw, "scale", where), _int(mask, "size", where + ".mask") if mask is not None else 0,
                  _int(mask, "keep_first", where + ".mask", least=0) if mask is not None else 0,
                  _int(raw, "bias_max", where, least=2) if biased else 0,
                  _int(raw, "bias_buckets", where, least=2) if "bias_buckets" in raw else None)
        if out.heads % out.kv_heads:
            raise InvalidInput(f"config.json {where}: {out.heads} heads do not divide into {out.kv_heads} kv_heads")
        return out


@dataclass
class LatentSizes:
    """Mixers ``latent_attention`` (no positions, plain softmax) and ``latent_attention_2`` (a rotated part, a sink
    and a gate per head)."""

    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_dim: int = 0
    rot_base: float = 0.0

    @classmethod
    def from_dict(cls, raw, where, rotated: bool):
        out = cls(_int(raw, "heads", where), _int(raw, "dim", where), _int(raw, "vdim", where), _int(raw, "q_rank", where),
                  _int(raw, "kv_rank", where), _number(raw, "scale", where))
        if rotated:
            rot = _get(raw, "rot", where)
            out.rot_dim, out.rot_base = _int(raw, "rot_dim", where, least=2), _number(rot, "base", where + ".rot")
            if out.rot_dim % 2:
                raise InvalidInput(f"config.json {where}.rot_dim must be even; got {out.rot_dim}")
            if _int(rot, "dims", where + ".rot", least=2) != out.rot_dim:
                raise Unsupported(f"config.json {where}: rot.dims {rot['dims']} differs from rot_dim {out.rot_dim}; this design "
                                  "rotates the whole rotated part")
        return out


@dataclass
class LayerSizes:
    type: str
    windowed: Optional[WindowedSizes] = None
    latent: Optional[LatentSizes] = None
    ff: Optional[int] = None  # None: the layer has no feed-forward


@dataclass
class MutedraConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    logit_softcap: float
    layers: List[LayerSizes]
    loop_start: int
    loop_stop: int
    loop_times: int
    raw: Dict[str, Any] = field(default_factory=dict)
    architecture: str = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "MutedraConfig":
        layers = _get(raw, "layers", "file")
        if not isinstance(layers, list) or not layers:
            raise InvalidInput("config.json layers must be a list with at least one layer")
        out_layers = []
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            kind, mixer, mlp = _get(layer, "type", where), _get(layer, "mixer", where), _get(layer, "mlp", where)
            ff = None
            if mlp is not None:
                if _get(mlp, "kind", where + ".mlp") != "dense":
                    raise Unsupported(f"config.json {where}.mlp.kind {mlp['kind']!r}; this design has dense feed-forwards")
                ff = _int(mlp, "ff", where + ".mlp")
            if kind == "attention":
                out_layers.append(LayerSizes(kind, windowed=WindowedSizes.from_dict(mixer, where + ".mixer"), ff=ff))
            elif kind in ("latent_attention", "latent_attention_2"):
                out_layers.append(LayerSizes(kind, latent=LatentSizes.from_dict(mixer, where + ".mixer", kind.endswith("_2")), ff=ff))
            else:
                raise Unsupported(f"config.json {where}.type {kind!r}; this design has the mixers {', '.join(MIXERS)}")
        loop = raw.get("loop")
        start, stop, times = 0, 0, 1
        if loop is not None:
            start, stop = _int(loop, "start", "loop", least=0), _int(loop, "stop", "loop", least=0)
            times = _int(loop, "times", "loop", least=1)
            if not start <= stop <= len(out_layers):
                raise InvalidInput(f"config.json loop covers layers {start} to {stop - 1}, but there are {len(out_layers)}")
        embedding = raw.get("embedding") or {}
        return cls(
            vocab=_int(raw, "vocab", "file"), width=_int(raw, "width", "file"), eps=_number(_get(raw, "norm", "file"), "eps", "norm"),
            embedding_scale=_number(embedding, "scale", "embedding") if embedding.get("scale") is not None else 1.0,
            logit_softcap=_number(raw, "logit_softcap", "file") if raw.get("logit_softcap") is not None else 0.0, layers=out_layers, loop_start=start, loop_stop=stop,
            loop_times=times, raw=copy.deepcopy(raw))

    def layer_runs(self):
        """[(layer, pass)] in the order the layers run: the looped stretch as often as the loop says, with the same
        weights; ``pass`` is the number of the pass that the run begins, None for every other run."""
        runs = [(index, None) for index in range(self.loop_start)]
        for number in range(self.loop_times):
            runs += [(index, number if index == self.loop_start else None) for index in range(self.loop_start, self.loop_stop)]
        return runs + [(index, None) for index in range(self.loop_stop, len(self.layers))]

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
