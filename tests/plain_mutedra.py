"""Mutedra, plainly: one function a mechanism over whole sequences in 64-bit,
written from the design's equations and sharing nothing with the library.

Notation.  x: the residual stream [tokens, width].  A norm is N(x) = tanh(a x)
* w + b with one number a.  A layer is x <- x + N1b(mixer(N1(x))), then x <- x +
N2b(ff(N2(x))) if it has a feed-forward.  ``rnd`` rounds where an engine that
keeps activations in bfloat16 rounds them (the identity by default).
"""

import json
import math
import os

import torch
from safetensors.torch import load_file


def identity(x):
    return x


def bf16_round(x):
    return x.to(torch.bfloat16).to(x.dtype)


def tanh_norm(x, w, b, a):
    return torch.tanh(a * x) * w + b


def bias_row(distance, rows, reach):
    """Which row of a table of ``rows`` rows a key ``distance`` back reads."""
    half = rows // 2
    if distance < half:
        return distance
    step = math.log(distance / half) / math.log(reach / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(step)))


def windowed_attention(h, w, sizes, rnd=identity):
    """h [tokens, width].  w: q, k, v, o, rel.  Query i sees key j <= i if i - j < window or j < keep_first; the score is
    q . k * scale + rel[row(i - j), head]; the weights are exp(s) / (1 + sum exp(s))."""
    n = h.shape[0]
    heads, groups, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    mask = sizes.get("mask")  # (without one every earlier key is seen; without bias_max there is no bias)
    window, keep = (mask["size"], mask["keep_first"]) if mask else (n, 0)
    q = rnd(h @ w["q"].T).view(n, heads, dim)
    k = rnd(h @ w["k"].T).view(n, groups, dim)
    v = rnd(h @ w["v"].T).view(n, groups, vdim)
    biased = sizes.get("bias_max") is not None
    rows = torch.tensor([bias_row(d, w["rel"].shape[0], sizes["bias_max"]) if biased else 0 for d in range(n)])
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    seen = (j <= i) & ((i - j < window) | (j < keep))
    out = torch.zeros(n, heads, vdim, dtype=torch.float64)
    for head in range(heads):
        group = head // (heads // groups)
        s = (q[:, head] @ k[:, group].T) * sizes["scale"]
        if biased:
            s = s + w["rel"][rows[(i - j).clamp(min=0)], head]
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        top = s.max(dim=1, keepdim=True).values.clamp(min=0.0)  # the sink's score is 0
        e = torch.exp(s - top)
        p = e / (torch.exp(-top) + e.sum(dim=1, keepdim=True))
        out[:, head] = p @ v[:, group]
    return rnd(out.reshape(n, heads * vdim)) @ w["o"].T


def turn_pairs(x, positions, base):
    """x [..., tokens, d] with d even: channel 2i turns with channel 2i + 1 by the angle position * base^(-2i / d)."""
    d = x.shape[-1]
    angle = positions.double()[:, None] * base ** (-2.0 * torch.arange(d // 2, dtype=torch.float64) / d)[None, :]
    c, s = torch.cos(angle), torch.sin(angle)
    u, v = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


def root_mean_square_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def latent_attention(h, w, sizes, eps, rnd=identity):
    """h [tokens, width].  w: dq, dq.norm, uq, dkv, dkv.norm, uk, uv, o and, with a rotated part, sink and g.  Keys and
    values of every head are made of the latent here, as the equations have it; causal."""
    n = h.shape[0]
    heads, dim, vdim, rank = sizes["heads"], sizes["dim"], sizes["vdim"], sizes["kv_rank"]
    rot = sizes.get("rot_dim", 0)
    cq = rnd(root_mean_square_norm(h @ w["dq"].T, w["dq.norm"], eps))
    q = rnd(cq @ w["uq"].T).view(n, heads, dim + rot)
    down = h @ w["dkv"].T
    c = rnd(root_mean_square_norm(down[:, :rank], w["dkv.norm"], eps))
    k = rnd(c @ w["uk"].T).view(n, heads, dim)
    v = rnd(c @ w["uv"].T).view(n, heads, vdim)
    positions = torch.arange(n)
    causal = positions[None, :] <= positions[:, None]
    if rot:
        k_turned = rnd(turn_pairs(down[:, rank:], positions, sizes["rot"]["base"]))
    out = torch.zeros(n, heads, vdim, dtype=torch.float64)
    for head in range(heads):
        s = q[:, head, :dim] @ k[:, head].T
        if rot:
            s = s + rnd(turn_pairs(q[:, head, dim:], positions, sizes["rot"]["base"])) @ k_turned.T
        s = torch.where(causal, s * sizes["scale"], torch.full_like(s, -math.inf))
        if rot:
            top = torch.maximum(s.max(dim=1, keepdim=True).values, w["sink"][head])
            e = torch.exp(s - top)
            p = e / (e.sum(dim=1, keepdim=True) + torch.exp(w["sink"][head] - top))
        else:
            p = torch.softmax(s, dim=1)
        out[:, head] = p @ v[:, head]
    if rot:
        out = out * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return rnd(out.reshape(n, heads * vdim)) @ w["o"].T


def relu_gated(h, w, rnd=identity):
    return rnd(torch.relu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


class PlainMutedra:
    def __init__(self, folder):
        with open(os.path.join(folder, "config.json")) as handle:
            self.config = json.load(handle)
        self.w = {name: t.double() for name, t in load_file(os.path.join(folder, "model.safetensors")).items()}

    def _part(self, prefix):
        return {name[len(prefix):]: t for name, t in self.w.items() if name.startswith(prefix)}

    def _norm(self, x, name):
        return tanh_norm(x, self.w[name], self.w[name + ".b"], self.w[name + ".alpha"])

    def runs(self):
        """[(layer, number of the pass that begins there or None)]"""
        count = len(self.config["layers"])
        loop = self.config.get("loop") or {"start": 0, "stop": 0, "times": 1}
        out = [(i, None) for i in range(loop["start"])]
        for number in range(loop["times"]):
            out += [(i, number if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
        return out + [(i, None) for i in range(loop["stop"], count)]

    def logits(self, ids, rnd=identity, stream_after=None):
        cfg = self.config
        x = self.w["embed"][torch.tensor(list(ids))] * (cfg.get("embedding") or {}).get("scale", 1.0)
        embedded = x.clone()
        for index, number in self.runs():
            if number is not None:
                if number > 0:
                    x = x + embedded
                x = x + self.w["loop.step"][number]
            layer, prefix = cfg["layers"][index], f"l{index}."
            h = rnd(self._norm(x, prefix + "norm1"))
            if layer["type"] == "attention":
                y = windowed_attention(h, self._part(prefix + "mix."), layer["mixer"], rnd)
            else:
                y = latent_attention(h, self._part(prefix + "mix."), layer["mixer"], cfg["norm"]["eps"], rnd)
            x = x + self._norm(rnd(y), prefix + "norm1b")
            if layer["mlp"] is not None:
                y = relu_gated(rnd(self._norm(x, prefix + "norm2")), self._part(prefix + "mlp."), rnd)
                x = x + self._norm(rnd(y), prefix + "norm2b")
            if stream_after is not None:
                stream_after.append(x.clone())
        z = rnd(self._norm(x, "final.norm")) @ self.w["head"].T
        cap = cfg.get("logit_softcap")
        return z if cap is None else cap * torch.tanh(z / cap)

    def greedy(self, ids, count):
        ids, out = list(ids), []
        for _ in range(count):
            out.append(int(self.logits(ids)[-1].argmax()))
            ids.append(out[-1])
        return out
