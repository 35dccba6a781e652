"""Zifunex as a model description.  A decoder over several residual streams
(hyper-connections) whose embedding adds a hashed table of token pairs; a
layer is either an attention and a selective scan side by side (``parallel``)
or gated linear attention (``gla``), with a GELU-gated feed-forward or none; a
stretch of the layers runs several times with the same weights, every run with
a cache or state of its own; layer norms with bias throughout.  Tensor names
are the checkpoint's: layer i's start with ``l<i>.``.
"""

from __future__ import annotations

from ..config.zifunex import ZifunexConfig
from .spec import ModelSpec, ScheduleEntry


def _norm(cfg: ZifunexConfig, name: str, take=None):
    return {"kind": "layer", "width": cfg.width, "eps": cfg.eps, "weight": name, "bias": name + ".b", "streams": cfg.streams,
            "take": take}


def _attention(cfg: ZifunexConfig, prefix: str, sizes, position: str):
    return {
        "kind": "causal_attention", "width": cfg.width, "heads": sizes.heads, "kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
        "value_dim": sizes.vdim, "scale": sizes.scale, "softcap": sizes.softcap, "position": position,
        "q": prefix + "q", "k": prefix + "k", "v": prefix + "v", "o": prefix + "o",
        "q_bias": prefix + "q.b", "k_bias": prefix + "k.b", "v_bias": prefix + "v.b", "o_bias": prefix + "o.b",
    }


def _scan(cfg: ZifunexConfig, prefix: str, sizes):
    return {
        "kind": "selective_scan", "width": cfg.width, "channels": sizes.inner, "states": sizes.state, "dt_rank": sizes.dt_rank,
        "taps": sizes.conv, "w_in": prefix + "in", "conv": prefix + "conv", "conv_bias": prefix + "conv.b", "w_x": prefix + "x",
        "w_dt": prefix + "dt", "dt_bias": prefix + "dt.b", "a_log": prefix + "A_log", "d": prefix + "D", "w_out": prefix + "o",
    }


def _gla(cfg: ZifunexConfig, prefix: str, sizes):
    return {
        "kind": "gated_linear_attention", "width": cfg.width, "heads": sizes.heads, "key_dim": sizes.dim, "value_dim": sizes.vdim,
        "tau": sizes.tau, "eps": cfg.eps, "decay_rank": sizes.rank, "q": prefix + "q", "k": prefix + "k", "v": prefix + "v",
        "g": prefix + "g", "o": prefix + "o", "norm": prefix + "norm", "a1": prefix + "a1", "a2": prefix + "a2",
        "a2_bias": prefix + "a2.b",
    }


def zifunex_spec(cfg: ZifunexConfig) -> ModelSpec:
    positions, layers = {}, []
    for index, layer in enumerate(cfg.layers):
        prefix = f"l{index}."
        if layer.type == "parallel":
            # rotations that agree in size and base share their tables
            position = f"rope_{layer.left.rot_dims}_{layer.left.rot_base!r}"
            positions.setdefault(position, {"kind": "rotary_half", "rot_dim": layer.left.rot_dims, "theta": layer.left.rot_base,
                                            "max_positions": None, "angles": "float64"})
            mixer = {
                "kind": "side_by_side", "width": cfg.width, "eps": cfg.eps,
                "branches": [_attention(cfg, prefix + "mix.left.", layer.left, position), _scan(cfg, prefix + "mix.right.", layer.right)],
                "weights": [prefix + "mix.left.out", prefix + "mix.right.out"],
            }
        else:
            mixer = _gla(cfg, prefix + "mix.", layer.gla)
        block = {
            "kind": "hyper_connections", "width": cfg.width, "streams": cfg.streams,
            "norm1": _norm(cfg, prefix + "norm1", take=prefix + "hc1.in"), "mixer": mixer,
            "connect1": {"mix": prefix + "hc1.mix", "gain": prefix + "hc1.out"},
        }
        if layer.ff is not None:
            block["norm2"] = _norm(cfg, prefix + "norm2", take=prefix + "hc2.in")
            block["feed_forward"] = {"kind": "gated", "width": cfg.width, "inner": layer.ff, "activation": "gelu_tanh",
                                     "gate": prefix + "mlp.gate", "up": prefix + "mlp.up", "down": prefix + "mlp.down"}
            block["connect2"] = {"mix": prefix + "hc2.mix", "gain": prefix + "hc2.out"}
        layers.append(block)
    spec = ModelSpec(
        architecture=cfg.architecture,
        width=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=None,  # the design names no last position
        stored_dtype="bfloat16",
        embedding={"kind": "table_pairs", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "embed", "pairs": "bigram",
                   "buckets": cfg.buckets, "mul_prev": cfg.mul_prev, "mul_cur": cfg.mul_cur, "copies": cfg.streams},
        positions=positions,
        layers=layers,
        schedule=[ScheduleEntry(layer=index) for index in cfg.layer_runs()],  # every run keeps a cache or state of its own
        final_norm=_norm(cfg, "final.norm"),  # reads the plain sum of the streams
        head={"kind": "linear", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "head", "tied_to": None},
        stop_token_ids=(),
        config_json=cfg.to_dict(),
    )
    spec.validate()
    return spec
