"""Mutedra as a model description.  A decoder whose layers norm every
sublayer on the way in and on the way out with a norm that keeps no
statistics, tanh(alpha x) w + b; whose mixers are attention in a sliding
window that keeps the first tokens visible, with a learned bias by distance
and a sink of score zero (``attention``), or attention over a cached latent,
plain (``latent_attention``) or with a rotated key part, a learned sink and a
gate per head (``latent_attention_2``); whose feed-forward is gated by ReLU;
whose embedding is scaled and whose logits are bent by a cap.  A stretch of
the layers runs several times with the same weights, every run with a cache of
its own; each pass begins by adding a vector of its own to the stream, and
every pass but the first the embedding's output before that.  Tensor names are
the checkpoint's: layer i's start with ``l<i>.``.
"""

from __future__ import annotations

from ..config.mutedra import MutedraConfig
from .spec import ModelSpec, ScheduleEntry


def _norm(cfg: MutedraConfig, name: str):
    return {"kind": "dynamic_tanh", "width": cfg.width, "weight": name, "bias": name + ".b", "alpha": name + ".alpha"}


def _windowed(cfg: MutedraConfig, prefix: str, sizes):
    out = {
        "kind": "causal_attention", "width": cfg.width, "heads": sizes.heads, "kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
        "value_dim": sizes.vdim, "scale": sizes.scale, "sink": "zero",
        "q": prefix + "q", "k": prefix + "k", "v": prefix + "v", "o": prefix + "o",
    }
    if sizes.window:
        out.update(window=sizes.window, keep_first=sizes.keep_first)
    if sizes.bias_max:
        out.update(distance_bias=prefix + "rel", bias_reach=sizes.bias_max, bias_buckets=sizes.bias_buckets)
    return out


def _latent(cfg: MutedraConfig, prefix: str, sizes, position):
    out = {
        "kind": "latent_attention", "width": cfg.width, "heads": sizes.heads, "key_dim": sizes.dim, "value_dim": sizes.vdim,
        "q_rank": sizes.q_rank, "kv_rank": sizes.kv_rank, "scale": sizes.scale, "eps": cfg.eps,
        "dq": prefix + "dq", "dq_norm": prefix + "dq.norm", "uq": prefix + "uq", "dkv": prefix + "dkv",
        "dkv_norm": prefix + "dkv.norm", "uk": prefix + "uk", "uv": prefix + "uv", "o": prefix + "o",
    }
    if position is not None:
        out.update(rot_dim=sizes.rot_dim, position=position, sink=prefix + "sink", gate=prefix + "g")
    return out


def mutedra_spec(cfg: MutedraConfig) -> ModelSpec:
    positions, layers = {}, []
    for index, layer in enumerate(cfg.layers):
        prefix = f"l{index}."
        if layer.type == "attention":
            mixer = _windowed(cfg, prefix + "mix.", layer.windowed)
        elif layer.type == "latent_attention":
            mixer = _latent(cfg, prefix + "mix.", layer.latent, None)
        else:
            # rotations that agree in size and base share their tables
            position = f"pairs_{layer.latent.rot_dim}_{layer.latent.rot_base!r}"
            positions.setdefault(position, {"kind": "rotary_pairs", "rot_dim": layer.latent.rot_dim, "theta": layer.latent.rot_base,
                                            "max_positions": None, "angles": "float64"})
            mixer = _latent(cfg, prefix + "mix.", layer.latent, position)
        block = {"kind": "pre_post_norm", "width": cfg.width, "norm1": _norm(cfg, prefix + "norm1"),
                 "post1": _norm(cfg, prefix + "norm1b"), "mixer": mixer}
        if layer.ff is not None:
            block.update(norm2=_norm(cfg, prefix + "norm2"), post2=_norm(cfg, prefix + "norm2b"),
                         feed_forward={"kind": "gated", "width": cfg.width, "inner": layer.ff, "activation": "relu",
                                       "gate": prefix + "mlp.gate", "up": prefix + "mlp.up", "down": prefix + "mlp.down"})
        layers.append(block)
    schedule = [
        ScheduleEntry(layer=index, enter=None if number is None else {
            "kind": "restart", "width": cfg.width, "table": "loop.step", "rows": cfg.loop_times, "row": number,
            "add_embedding": number > 0})
        for index, number in cfg.layer_runs()]  # every run keeps a cache of its own
    spec = ModelSpec(
        architecture=cfg.architecture,
        width=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=None,  # the design names no last position
        stored_dtype="bfloat16",
        embedding={"kind": "table", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "embed", "scale": cfg.embedding_scale},
        positions=positions,
        layers=layers,
        schedule=schedule,
        final_norm=_norm(cfg, "final.norm"),
        head={"kind": "linear", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "head", "tied_to": None,
              "softcap": cfg.logit_softcap or None},
        stop_token_ids=(),
        config_json=cfg.to_dict(),
    )
    spec.validate()
    return spec
