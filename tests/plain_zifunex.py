"""A plain, slow Zifunex: every mechanism of the design as one function over a
whole sequence, written from its equations with ordinary tensor operations.
It shares no code with the library; the tests compare the library with it.

Notation: T tokens, W model width, H query heads, G key/value heads, d the
query/key size of a head, e its value size, C channels of the scan, N its
states, s residual streams.  A linear weight is [out, in] and applied as
x @ W^T.
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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def layer_norm(x, weight, bias, eps):
    mean = x.mean(dim=-1, keepdim=True)
    variance = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(variance + eps) * weight + bias


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x ** 2).mean(dim=-1, keepdim=True) + eps) * weight


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for each token: hashed from the token before it
    and itself; the first token of a sequence takes the table's last row."""
    rows = [buckets]
    for before, now in zip(tokens[:-1], tokens[1:]):
        rows.append((before * mul_prev + now * mul_cur) % buckets)
    return rows


def rotate_half(x, positions, dims, base):
    """x: [T, heads, size]; channel i < dims/2 is paired with channel i + dims/2."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = torch.tensor(positions, dtype=x.dtype)[:, None] * freq[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def capped_attention(h, p, m, rnd=identity):
    """Causal attention with biased projections, grouped heads, rotation of
    part of each head, scores bent by a tanh cap, values of their own size."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(h @ p["q"].T + p["q.b"]).view(T, H, d)
    k = rnd(h @ p["k"].T + p["k.b"]).view(T, G, d)
    v = rnd(h @ p["v"].T + p["v.b"]).view(T, G, e)
    positions = list(range(T))
    q = rnd(rotate_half(q, positions, m["rot"]["dims"], m["rot"]["base"]))
    k = rnd(rotate_half(k, positions, m["rot"]["dims"], m["rot"]["base"]))
    out = torch.zeros(T, H, e, dtype=h.dtype)
    visible = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for head in range(H):
        group = head // (H // G)
        score = (q[:, head] @ k[:, group].T) * m["scale"]
        score = m["softcap"] * torch.tanh(score / m["softcap"])
        score = score.masked_fill(~visible, float("-inf"))
        out[:, head] = torch.softmax(score, dim=-1) @ v[:, group]
    return rnd(rnd(out.reshape(T, H * e)) @ p["o"].T + p["o.b"])


def selective_scan(h, p, m, rnd=identity):
    """Mamba: gated input, short causal convolution, input-dependent step
    sizes and read/write vectors, a diagonal recurrence per channel."""
    T = h.shape[0]
    C, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = rnd(h @ p["in"].T)
    x, z = xz[:, :C], xz[:, C:]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=h.dtype), x], dim=0)
    conv = torch.zeros(T, C, dtype=h.dtype)
    for j in range(taps):  # the last column multiplies the current token
        conv = conv + padded[j:j + T] * p["conv"][:, j]
    x = rnd(silu(conv + p["conv.b"]))
    dbc = x @ p["x"].T
    dt, B, Cm = dbc[:, :R], dbc[:, R:R + N], dbc[:, R + N:]
    dt = torch.nn.functional.softplus(dt @ p["dt"].T + p["dt.b"], threshold=1e9)
    A = -torch.exp(p["A_log"])
    S = torch.zeros(C, N, dtype=h.dtype)
    y = torch.zeros(T, C, dtype=h.dtype)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ Cm[t] + p["D"] * x[t]
    return rnd(rnd(y * silu(z)) @ p["o"].T)


def gated_linear_attention(h, p, m, eps, rnd=identity):
    """A matrix state per head that decays per key channel and takes the outer
    product of key and value; read by the query, normed, gated, projected."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = (rnd(h @ p["q"].T) * d ** -0.5).view(T, H, d)
    k = rnd(h @ p["k"].T).view(T, H, d)
    v = rnd(h @ p["v"].T).view(T, H, e)
    z = (rnd(h @ p["a1"].T) @ p["a2"].T + p["a2.b"]).view(T, H, d)
    alpha = torch.sigmoid(z) ** (1.0 / m["tau"])
    S = torch.zeros(H, d, e, dtype=h.dtype)
    o = torch.zeros(T, H, e, dtype=h.dtype)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    o = rms_norm(o, p["norm"], eps).reshape(T, H * e)
    gate = silu(rnd(h @ p["g"].T))
    return rnd(rnd(o * gate) @ p["o"].T)


def side_by_side(h, p, m, eps, rnd=identity):
    """Attention and scan read the same input; each output is normed over the
    model width with its own weight; the result is half their sum."""
    left = capped_attention(h, {k[5:]: v for k, v in p.items() if k.startswith("left.")}, m["left"], rnd)
    right = selective_scan(h, {k[6:]: v for k, v in p.items() if k.startswith("right.")}, m["right"], rnd)
    return 0.5 * (rms_norm(left, p["left.out"], eps) + rms_norm(right, p["right.out"], eps))


def gated_feed_forward(h, p, rnd=identity):
    return rnd(rnd(gelu_tanh(rnd(h @ p["gate"].T)) * rnd(h @ p["up"].T)) @ p["down"].T)


def hyper_sublayer(streams, p, sublayer):
    """streams: [s, T, W].  The sublayer reads a weighted sum of the streams;
    every stream becomes a mix of the old ones plus a share of the output."""
    u = torch.einsum("s,stw->tw", p["in"], streams)
    y = sublayer(u)
    return torch.einsum("sr,stw->rtw", p["mix"], streams) + p["out"][:, None, None] * y[None]


class PlainZifunex:
    def __init__(self, folder, dtype=torch.float64):
        with open(os.path.join(folder, "config.json")) as handle:
            self.config = json.load(handle)
        self.dtype = dtype
        self.w = {name: (t if t.dtype in (torch.int32, torch.int64) else t.to(dtype))
                  for name, t in load_file(os.path.join(folder, "model.safetensors")).items()}

    def part(self, prefix):
        return {name[len(prefix):]: t for name, t in self.w.items() if name.startswith(prefix)}

    def layer_runs(self):
        """Indices of the layers in the order they run: a stretch of them is repeated."""
        count = len(self.config["layers"])
        loop = self.config.get("loop") or {"start": 0, "stop": 0, "times": 1}
        inside = list(range(loop["start"], loop["stop"]))
        return list(range(loop["start"])) + inside * loop["times"] + list(range(loop["stop"], count))

    def embed(self, tokens):
        x = self.w["embed"][torch.tensor(tokens)]
        b = self.config["embedding"].get("bigram")
        if b:
            x = x + self.w["bigram"][torch.tensor(bigram_rows(list(tokens), b["buckets"], b["mul_prev"], b["mul_cur"]))]
        return x

    def run_layer(self, index, streams, rnd=identity):
        layer = self.config["layers"][index]
        eps = self.config["norm"]["eps"]
        mix = self.part(f"l{index}.mix.")

        def mixer(u):
            h = rnd(layer_norm(u, self.w[f"l{index}.norm1"], self.w[f"l{index}.norm1.b"], eps))
            if layer["type"] == "parallel":
                return side_by_side(h, mix, layer["mixer"], eps, rnd)
            if layer["type"] == "gla":
                return gated_linear_attention(h, mix, layer["mixer"], eps, rnd)
            raise ValueError(layer["type"])

        streams = hyper_sublayer(streams, self.part(f"l{index}.hc1."), mixer)
        if layer["mlp"] is not None:
            def feed_forward(u):
                h = rnd(layer_norm(u, self.w[f"l{index}.norm2"], self.w[f"l{index}.norm2.b"], eps))
                return gated_feed_forward(h, self.part(f"l{index}.mlp."), rnd)

            streams = hyper_sublayer(streams, self.part(f"l{index}.hc2."), feed_forward)
        return streams

    def logits(self, tokens, rnd=identity, layers_out=None):
        """[T, vocab]; ``layers_out``: a list that receives the sum of the streams after every layer run."""
        x = self.embed(tokens)
        streams = x[None].repeat(self.config["streams"], 1, 1)
        for index in self.layer_runs():
            streams = self.run_layer(index, streams, rnd)
            if layers_out is not None:
                layers_out.append(streams.sum(dim=0))
        x = streams.sum(dim=0)
        x = rnd(layer_norm(x, self.w["final.norm"], self.w["final.norm.b"], self.config["norm"]["eps"]))
        return (x @ self.w["head"].T).float()

    def greedy(self, prompt, new_tokens):
        ids, out = list(prompt), []
        for _ in range(new_tokens):
            token = int(torch.argmax(self.logits(ids)[-1]))
            out.append(token)
            ids.append(token)
        return out
