"""Mutedra on the GPU against the plain implementation (``plain_mutedra``):
each mechanism alone, then whole models through the engine -- prompts whole, in
portions and token by token, unequal batches, slots and pages used again, keys
far away, at page borders and at the edges of a window and of the kept first
tokens, long decoding, greedy generation through the library's entry point.
32-bit is held to rounding; bfloat16 to the error of the plain model run with
its activations rounded where the engine rounds them.
"""

import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import nnis_amd
import plain_mutedra as M
from gpu_helpers import cache_for, context, runtime
from mutedra_configs import MUTEDRA_CONFIGS, latent, layer, mutedra, windowed

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def _relative(got, want):
    got, want = torch.as_tensor(np.asarray(got)).double(), torch.as_tensor(np.asarray(want)).double()
    return float((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_min(1e-30))


def _close(got, want, dtype, what="", bf16=3e-2):
    error = _relative(got.detach().float().cpu() if isinstance(got, torch.Tensor) else got, want)
    bound = 3e-5 if dtype == "float32" else bf16
    assert error <= bound, f"{what}: relative error {error:.3g} (bound {bound:.3g})"


def _weights(part, dtype, seed, scale=None):
    """Random tensors for a part, by its own declarations: (for the plain functions in 64-bit, for the part)."""
    from nnis_amd.weights.random_init import _INIT_RULES

    generator = torch.Generator().manual_seed(seed)
    stored = {}
    for t in part.tensors():
        value = _INIT_RULES[t.init](t, generator, torch.bfloat16)
        if scale and t.name in scale:
            value = (value.float() * scale[t.name]).to(torch.bfloat16)
        stored[t.name] = value
    wide = torch.float32 if dtype == "float32" else torch.bfloat16
    return {n: v.double() for n, v in stored.items()}, {n: v.to(wide).cuda() for n, v in stored.items()}


def _run_in_steps(mixer, cache, rt, xs, cuts):
    """Runs sequences through a mixer, all of them in every step; ``cuts[i]`` lists where sequence i's portions end."""
    slots = [cache.acquire() for _ in xs]
    done = [0] * len(xs)
    outs = [[] for _ in xs]
    cuts = [list(c) for c in cuts]
    while any(cuts):
        batch = [i for i in range(len(xs)) if cuts[i]]
        ends = [cuts[i].pop(0) for i in batch]
        ctx = context(cache, [(slots[i], end - done[i]) for i, end in zip(batch, ends)])
        x = torch.cat([xs[i][done[i]:end] for i, end in zip(batch, ends)]).to(rt.dtype).cuda()
        y = mixer.forward(x, ctx, cache.view(0), rt)
        row = 0
        for i, end in zip(batch, ends):
            outs[i].append(y[row:row + end - done[i]].float().cpu())
            row += end - done[i]
            done[i] = end
    for slot in slots:
        cache.release(slot)
    return [torch.cat(o) for o in outs]


# ---------------------------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
def test_the_residual_step_around_a_tanh_norm(y_dtype):
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(2)
    tokens, width = 37, 50
    x = torch.randn(tokens, width, generator=generator)
    y = (3.0 * torch.randn(tokens, width, generator=generator)).to(y_dtype)
    rows_add = torch.randn(tokens, width, generator=generator)
    w = [torch.randn(width, generator=generator).to(torch.bfloat16) for _ in range(5)]
    post, following = (0.4, w[0].cuda(), w[1].cuda()), (1.7, w[2].cuda(), w[3].cuda())
    want_x = x.double() + M.tanh_norm(y.double(), w[0].double(), w[1].double(), 0.4) + rows_add.double() + w[4].double()
    want_h = M.tanh_norm(want_x, w[2].double(), w[3].double(), 1.7)
    # everything at once, into a stream of its own (the input stays as it was)
    x_dev, x_out, h = x.cuda(), torch.empty(tokens, width, device="cuda"), torch.empty(tokens, width, device="cuda")
    ops.tanh_norm_step(x_dev, x_out=x_out, y=y.cuda(), post=post, rows_add=rows_add.cuda(), vec_add=w[4].cuda(), following=following, h=h)
    assert torch.equal(x_dev.cpu(), x)
    assert _relative(x_out.cpu(), want_x) < 1e-6 and _relative(h.cpu(), want_h) < 1e-6
    # in place, output in bfloat16, nothing but the sum and the norms
    h16 = torch.empty(tokens, width, device="cuda", dtype=torch.bfloat16)
    ops.tanh_norm_step(x_dev, x_out=x_dev, y=y.cuda(), post=post, following=following, h=h16)
    want_x = x.double() + M.tanh_norm(y.double(), w[0].double(), w[1].double(), 0.4)
    assert _relative(x_dev.cpu(), want_x) < 1e-6
    assert _relative(h16.float().cpu(), M.tanh_norm(want_x, w[2].double(), w[3].double(), 1.7)) < 4e-3
    # a list of rows, a plain sum (no norm on the way in), the stream left alone
    rows = torch.tensor([36, 0, 5, 5], dtype=torch.int32).cuda()
    before = x_dev.clone()
    h = torch.empty(4, width, device="cuda")
    ops.tanh_norm_step(x_dev, y=y.cuda(), following=following, h=h, rows=rows)
    want = M.tanh_norm(before.cpu().double() + y.double(), w[2].double(), w[3].double(), 1.7)[[36, 0, 5, 5]]
    assert torch.equal(x_dev, before) and _relative(h.cpu(), want) < 1e-6
    # the norm of rows that are no stream
    h = torch.empty(tokens, width, device="cuda")
    ops.tanh_norm_step(None, y=y.cuda(), following=post, h=h)
    assert _relative(h.cpu(), M.tanh_norm(y.double(), w[0].double(), w[1].double(), 0.4)) < 1e-6


@pytest.mark.parametrize("rows, width, inner", [(1, 64, 96), (8, 256, 384), (16, 100, 72), (200, 256, 640), (2048, 512, 1024), (300, 36, 40)])
def test_the_way_out_inside_the_projection(rows, width, inner):
    """The projection that ends a sublayer with the norm on the way out, the sum into the stream and the next norm in its
    own kernel (few tokens and many, widths that fill no tile) against the three steps one after the other."""
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(rows + width)
    x = torch.randn(rows, inner, generator=generator).to(torch.bfloat16)
    weight = (torch.randn(width, inner, generator=generator) / inner ** 0.5).to(torch.bfloat16)
    stream = torch.randn(rows, width, generator=generator)
    vectors = [torch.randn(width, generator=generator).to(torch.bfloat16) for _ in range(4)]
    post, following = (1.3, vectors[0].cuda(), vectors[1].cuda()), (0.6, vectors[2].cuda(), vectors[3].cuda())
    packed = ops.pack_weight(weight.cuda())
    resid, normed = stream.clone().cuda(), torch.empty(rows, width, device="cuda", dtype=torch.bfloat16)
    ss = torch.empty(ops.gemm_residual_parts(rows, width), rows, device="cuda")
    ops.gemm_residual_tanh(x.cuda(), packed, resid, post, following, normed, ss)
    y = x.double() @ weight.double().T
    want = stream.double() + M.tanh_norm(y, vectors[0].double(), vectors[1].double(), 1.3)
    assert _relative(resid.cpu(), want) < 1e-5
    assert _relative(normed.float().cpu(), M.tanh_norm(want, vectors[2].double(), vectors[3].double(), 0.6)) < 4e-3


@pytest.mark.parametrize("activation", ["relu", "gelu_tanh", "silu"])
@pytest.mark.parametrize("rows, width, inner", [(1, 64, 96), (8, 256, 384), (40, 128, 200), (200, 256, 640), (2048, 512, 1024), (300, 40, 36)])
def test_the_gate_inside_the_projection(activation, rows, width, inner):
    """Gate and up projection with the gating in the product's epilogue, on plain rows, against the products in 64-bit."""
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(rows + inner)
    x = torch.randn(rows, width, generator=generator).to(torch.bfloat16)
    weight = (3.0 * torch.randn(2 * inner, width, generator=generator) / width ** 0.5).to(torch.bfloat16)
    got = ops.gated_linear(x.cuda(), ops.pack_weight(weight.cuda()), torch.empty(rows, inner, device="cuda", dtype=torch.bfloat16), activation)
    gate, up = x.double() @ weight[:inner].double().T, x.double() @ weight[inner:].double().T
    act = {"relu": torch.relu, "silu": torch.nn.functional.silu,
           "gelu_tanh": lambda g: 0.5 * g * (1 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))}[activation]
    assert _relative(got.float().cpu(), act(gate) * up) < 4e-3


def test_embedding_scale_logit_cap_and_relu_gate():
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(3)
    table = torch.randn(20, 24, generator=generator).to(torch.bfloat16)
    ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32)
    out = ops.embed(ids.cuda(), table.cuda(), torch.empty(4, 24, device="cuda"), 7.5)
    assert torch.equal(out.cpu(), table.float()[ids.long()] * 7.5)
    logits = 40.0 * torch.randn(5, 33, generator=generator)
    got = ops.tanh_cap(logits.clone().cuda(), 12.0)
    assert _relative(got.cpu(), 12.0 * torch.tanh(logits.double() / 12.0)) < 1e-6 and float(got.abs().max()) <= 12.0
    for dtype in (torch.float32, torch.bfloat16):
        gate_up = torch.randn(6, 2 * 40, generator=generator).to(dtype)
        got = ops.gated_act(gate_up.cuda(), torch.empty(6, 40, device="cuda", dtype=dtype), "relu")
        want = torch.relu(gate_up[:, :40].double()) * gate_up[:, 40:].double()
        assert _relative(got.float().cpu(), want) < (1e-6 if dtype == torch.float32 else 4e-3)


def _windowed_part(sizes, width, buckets):
    from nnis_amd.parts import build_part

    return build_part("mixer", dict(kind="causal_attention", width=width, heads=sizes["heads"], kv_heads=sizes["kv_heads"],
                                    head_dim=sizes["dim"], value_dim=sizes["vdim"], scale=sizes["scale"], window=sizes["mask"]["size"],
                                    keep_first=sizes["mask"]["keep_first"], distance_bias="rel", bias_reach=sizes["bias_max"],
                                    bias_buckets=buckets, sink="zero", q="q", k="k", v="v", o="o"))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, window, keep, reach, buckets, width", [
    (4, 2, 32, 16, 37, 5, 50, 12, 64), (3, 1, 16, 48, 70, 0, 90, 8, 48), (6, 6, 32, 16, 8, 3, 20, 6, 96), (2, 1, 16, 48, 64, 64, 33, 10, 40),
    (2, 2, 32, 16, 130, 1, 64, 32, 56)])
def test_windowed_attention_alone(dtype, heads, kv_heads, dim, vdim, window, keep, reach, buckets, width):
    """Grouped heads, values of their own size, a window with kept first tokens, a bias by distance large enough to
    decide which keys count, and the sink.  Whole prompts; then portions down to two tokens and single tokens across
    the borders of pages (64, 128) and of the window."""
    rt = runtime(dtype)
    sizes = windowed(heads, kv_heads, dim, vdim, window, keep, reach, buckets, scale=0.3)
    mixer = _windowed_part(sizes, width, buckets)
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"q": 20.0, "k": 20.0, "rel": 100.0})
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    generator = torch.Generator().manual_seed(5)
    lengths = [200, 3, 67]
    xs = [torch.randn(n, width, generator=generator).to(torch.bfloat16).double() for n in lengths]
    rnd = M.identity if dtype == "float32" else M.bf16_round
    want = [M.windowed_attention(x, plain_w, sizes, rnd) for x in xs]
    assert float(plain_w["rel"].abs().mean()) > 1.0
    for cuts in ([[200], [3], [67]], [[61, 63, 64, 66, 128, 130, 131, 200], [1, 2, 3], [2, 4, 64, 65, 66, 67]],
                 [[150] + list(range(151, 201)), [3], [60] + list(range(61, 68))]):
        got = _run_in_steps(mixer, cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"windowed attention {cuts[0][:2]} length {n}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window, keep", [(37, 5), (64, 3), (70, 64), (9, 0)])
def test_the_edges_of_the_window_and_of_the_kept_tokens_decide(dtype, window, keep):
    """One head whose queries read the input's first eight channels and whose keys read the next eight.  The last
    token's query channels match the key channels of one earlier token and of no other, so that token takes all the
    weight if the last token sees it, and the sink and the near keys share it if not: the output tells which.  The
    marked token stands just inside and just outside the window, and on the last kept place and the first one not
    kept; the last token comes in a prompt, in a portion, and alone."""
    rt = runtime(dtype)
    width = dim = 32
    sizes = windowed(1, 1, dim, 16, window, keep, 40, 8, scale=1.0)
    mixer = _windowed_part(sizes, width, 8)
    plain_w, part_w = _weights(mixer, dtype, 11)
    reads = {"q": torch.zeros(dim, width, dtype=torch.float64), "k": torch.zeros(dim, width, dtype=torch.float64)}
    reads["q"][:8, :8] = torch.eye(8, dtype=torch.float64)
    reads["k"][:8, 8:16] = torch.eye(8, dtype=torch.float64)
    for name in ("q", "k"):
        plain_w[name] = reads[name]
        part_w[name] = reads[name].to(part_w[name].dtype).cuda()
    plain_w["rel"].zero_()
    part_w["rel"].zero_()
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    n = 180
    generator = torch.Generator().manual_seed(1)
    places = [n - window, n - window - 1] + ([keep - 1, keep] if keep else [])  # just inside, just outside; kept, not kept
    seen_outputs = []
    for place in places:
        x = (0.05 * torch.randn(n, width, generator=generator)).to(torch.bfloat16).double()
        x[place, 8:16] = 2.0
        x[n - 1, :8] = 2.0  # a score of 32 with the marked token, against scores near 0
        want = M.windowed_attention(x, plain_w, sizes)
        inside = (n - 1 - place < window) or place < keep
        value = (x[place] @ plain_w["v"].T) @ plain_w["o"].T
        assert (_relative(want[n - 1], value) < 1e-3) == inside, (place, inside)  # seen, the marked token's value is the output
        for cuts in ([n], [n - 3, n], [n - 1, n], [100] + list(range(101, n + 1))):
            got = _run_in_steps(mixer, cache, rt, [x], [cuts])[0]
            _close(got[n - 1], want[n - 1], dtype, f"mark at {place} (window {window}, kept {keep}), cuts {cuts[:2]}", bf16=2e-2)
            _close(got, want, dtype, f"mark at {place}, all tokens, cuts {cuts[:2]}", bf16=2e-2)
        seen_outputs.append(inside)
    assert seen_outputs[:2] == [True, False] and (not keep or seen_outputs[2:] == [True, False])


def _latent_part(sizes, width, eps, rotated):
    from nnis_amd.parts import build_part

    positions = {}
    extra = {}
    if rotated:
        rope = build_part("position", {"kind": "rotary_pairs", "rot_dim": sizes["rot_dim"], "theta": sizes["rot"]["base"],
                                       "max_positions": None, "angles": "float64"})
        positions, extra = {"r": rope}, dict(rot_dim=sizes["rot_dim"], position="r", sink="sink", gate="g")
    mixer = build_part("mixer", dict(kind="latent_attention", width=width, heads=sizes["heads"], key_dim=sizes["dim"], value_dim=sizes["vdim"],
                                     q_rank=sizes["q_rank"], kv_rank=sizes["kv_rank"], scale=sizes["scale"], eps=eps, dq="dq", dq_norm="dq.norm",
                                     uq="uq", dkv="dkv", dkv_norm="dkv.norm", uk="uk", uv="uv", o="o", **extra), positions=positions)
    return mixer, positions


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, vdim, q_rank, kv_rank, rot, width", [
    (3, 16, 24, 40, 32, 16, 64), (2, 24, 8, 16, 48, 0, 48), (2, 32, 32, 24, 64, 32, 96), (5, 8, 40, 48, 40, 0, 40), (4, 24, 16, 32, 24, 8, 56),
    (2, 16, 24, 32, 272, 16, 48)])  # (the last: a latent wider than the matrix-core kernels carry runs on the row kernel)
def test_latent_attention_alone(dtype, heads, dim, vdim, q_rank, kv_rank, rot, width):
    """Attention over the cached latent against the equations, which make every head's keys and values of the latent:
    plain, and with the rotated part, the sink and the gates.  The up projections are large enough for the attention
    to be sharp, the sinks large enough to take a good part of the weight."""
    rt = runtime(dtype)
    sizes = latent(heads, dim, vdim, q_rank, kv_rank, scale=0.3, rot_dim=rot or None, base=500.0)
    mixer, positions = _latent_part(sizes, width, 1e-5, bool(rot))
    plain_w, part_w = _weights(mixer, dtype, 7, scale={"uq": 12.0, "uk": 12.0, "sink": 100.0, "g": 30.0, "dkv": 3.0})
    for rope in positions.values():
        rope.bind({}, rt)
        rope.reach(1024)
    mixer.check(rt)  # (as a model's load does: a latent wider than 256 channels is accepted for the row kernel here)
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=2048, max_positions=1024)
    generator = torch.Generator().manual_seed(5)
    lengths = [150, 3, 67]
    xs = [torch.randn(n, width, generator=generator).to(torch.bfloat16).double() for n in lengths]
    rnd = M.identity if dtype == "float32" else M.bf16_round
    want = [M.latent_attention(x, plain_w, sizes, 1e-5, rnd) for x in xs]
    for cuts in ([[150], [3], [67]], [[61, 63, 64, 66, 128, 130, 131, 150], [1, 2, 3], [2, 4, 64, 65, 66, 67]],
                 [[100] + list(range(101, 151)), [3], [60] + list(range(61, 68))]):
        got = _run_in_steps(mixer, cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"latent attention {cuts[0][:2]} length {n}", bf16=4e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rot", [0, 32])
def test_a_far_latent_counts(dtype, rot):
    """The queries read the input with its two halves swapped where the keys read it as it is, and the input of one
    token far back is the last token's with the halves swapped: sharp attention gives that token most of the weight (and
    none to the last token's own key), so a page lost or a run of keys skipped changes the output by its own size.
    Places 0, 1, 63, 64 and 500 of 700."""
    rt = runtime(dtype)
    width = 64
    sizes = latent(2, 64, 16, 64, 64, scale=1.0, rot_dim=rot or None, base=1e6)
    mixer, positions = _latent_part(sizes, width, 1e-5, bool(rot))
    plain_w, part_w = _weights(mixer, dtype, 13, scale={"uq": 40.0, "uk": 40.0, "dq": 10.0, "dkv": 10.0})
    for rope in positions.values():
        rope.bind({}, rt)
        rope.reach(1024)
    # both heads' queries and keys read the latents alike, so that a query and a key of matching inputs make a large score
    swap = torch.cat([torch.arange(32, 64), torch.arange(0, 32)])
    for w, to in ((plain_w, lambda t: t), (part_w, lambda t: t.to(part_w["uq"].dtype).cuda())):
        w["dq"] = to(w["dkv"][:64].cpu()[:, swap].clone())
        shared = w["uk"].cpu().clone()
        uq = w["uq"].cpu().clone().view(2, 64 + rot, 64)
        uq[:, :64] = shared.view(2, 64, 64)
        uq[:, 64:] = 0.0
        w["uq"] = to(uq.reshape(2 * (64 + rot), 64))
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=2048, max_positions=1024)
    n = 700
    generator = torch.Generator().manual_seed(1)
    for far in (0, 1, 63, 64, 500):
        x = torch.randn(n, width, generator=generator).to(torch.bfloat16).double()
        x[far] = x[n - 1][swap]
        want = M.latent_attention(x, plain_w, sizes, 1e-5)
        without = x.clone()
        without[far] = 0.0
        assert _relative(M.latent_attention(without, plain_w, sizes, 1e-5)[n - 1], want[n - 1]) > 0.3  # the far token decides
        for cuts in ([n], [n - 1, n], [650] + list(range(651, n + 1))):
            got = _run_in_steps(mixer, cache, rt, [x], [cuts])[0]
            _close(got[n - 1], want[n - 1], dtype, f"far key at {far}, cuts {cuts[:2]}", bf16=5e-2)


# ---------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------

def _sharpen(folder):
    """A random model's weights are too small for its mixers to matter: their outputs, a few hundredths, would pass the
    norm on the way out as little more than its bias, and the logits would be the embedding's.  Queries and keys are
    scaled up so that attention is sharp (a key left out or one too many shows); values, output and feed-forward
    projections so that every sublayer's output is of order one where its norm bends it; bias tables, sinks, gates and
    the passes' vectors so that every one of them matters; the head so that the cap bends the logits."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for key in tensors:
        if key.endswith((".mix.q", ".mix.k", ".mix.uq", ".mix.uk")):
            factor = 12.0
        elif key.endswith((".mix.v", ".mix.o", ".mix.uv", ".mlp.gate", ".mlp.up", ".mlp.down")):
            factor = 7.0
        elif key.endswith((".mix.rel", ".mix.sink")):
            factor = 80.0
        elif key.endswith(".mix.g") or key in ("loop.step", "head"):
            factor = 25.0
        elif key.endswith(".b") or key == "embed":
            factor = 10.0
        else:
            continue
        tensors[key] = (tensors[key].float() * factor).to(torch.bfloat16)
    save_file(tensors, path)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (config, seed) in MUTEDRA_CONFIGS.items():
        folder = str(tmp_path_factory.mktemp(f"mutedra_{name}"))
        nnis_amd.write_random_model(folder, config, seed)
        _sharpen(folder)
        out[name] = folder
    return out


def _ids(count, vocab, seed):
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=generator).tolist()


class Yardstick:
    """What the engine may differ from the plain 64-bit logits by, as root mean square relative to the logits' own: in
    32-bit, rounding; in bfloat16, three times what rounding the plain model's activations to bfloat16 does on the same
    tokens (a single position: four times the worst position's)."""

    def __init__(self, plain):
        self.plain, self.known = plain, {}
        self.least = (0.0, 0.0)
        self.least = self.twin(_ids(64, plain.config["vocab"], 999))[1:]

    def twin(self, ids):
        key = tuple(ids)
        if key not in self.known:
            want, twin = self.plain.logits(ids), self.plain.logits(ids, M.bf16_round)
            rows = [_relative(twin[i], want[i]) for i in range(len(ids))]
            self.known[key] = (want, _relative(twin, want), max(rows))
            assert 1e-4 < self.known[key][1] < 0.3, self.known[key][1]
        return self.known[key]

    def check(self, got, ids, dtype, what, rows=None):
        want, overall, worst = self.twin(ids)
        single = isinstance(rows, int)
        want = want if rows is None else want[rows]
        error = _relative(got, want)
        bound = 5e-5 if dtype == "float32" else (4.0 * max(worst, self.least[1]) if single else 3.0 * max(overall, self.least[0]))
        assert error <= bound, f"{what}: relative error {error:.3g} (bound {bound:.3g})"


def _collect(engine, slot, ids, cuts):
    from nnis_amd.engine.batch import StepEntry

    rows, done = [], 0
    for end in cuts:
        rows.append(engine.step([StepEntry(slot, ids[done:end], list(range(end - done)))]).cpu())
        done = end
    return torch.cat(rows)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_stream_after_every_layer_run(folders, dtype):
    """The residual stream behind every run of a layer (a looped layer counts each time), read off the engine's own
    blocks as the model runs, against the plain model's."""
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.parts.lazy import PostNormed, PreparedRows

    plain = M.PlainMutedra(folders["A"])
    engine = nnis_amd.load_engine(folders["A"], dtype=dtype, max_tokens=256)
    ids = _ids(40, MUTEDRA_CONFIGS["A"][0]["vocab"], 8)
    want = []
    plain.logits(ids, stream_after=want)
    seen = []
    for block in engine.model.layers:
        def watched(stream, ctx, view, rt, following=None, inner=block.forward):
            out = inner(stream, ctx, view, rt, following=following)
            if isinstance(out, PreparedRows):
                seen.append(out.x.clone())
            else:
                x, pending = out
                owed = pending.materialize(rt) if isinstance(pending, PostNormed) else pending
                seen.append(x + owed.float() if owed is not None else x.clone())
            return out
        block.forward = watched
    slot = engine.start_sequence()
    engine.step([StepEntry(slot, ids, [0])])
    assert len(seen) == len(want) == 7
    for run, (got, expected) in enumerate(zip(seen, want)):
        assert _relative(got.cpu(), expected) < (1e-5 if dtype == "float32" else 3e-2), f"layer run {run}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MUTEDRA_CONFIGS))
def test_prompts_whole_in_portions_and_token_by_token(folders, name, dtype):
    config = MUTEDRA_CONFIGS[name][0]
    plain = M.PlainMutedra(folders[name])
    engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=1024)
    ids = _ids(150, config["vocab"], 1)
    yard = Yardstick(plain)
    for cuts in ([150], [2, 4, 5, 63, 64, 66, 128, 129, 150], [100] + list(range(101, 151)), list(range(1, 41))):
        slot = engine.start_sequence()
        got = _collect(engine, slot, ids, cuts)
        engine.end_sequence(slot)
        yard.check(got, ids, dtype, f"{name} cuts {cuts[:3]}..", rows=slice(0, cuts[-1]))
        for place in (0, 1, 2, cuts[-1] - 1):  # every position by itself, the first tokens among them
            yard.check(got[place], ids, dtype, f"{name} cuts {cuts[:3]}.. position {place}", rows=place)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_unequal_batches_equal_each_request_alone(folders, name, dtype):
    """Requests of different lengths start together, are decoded together and end one after the other; their slots
    and pages go to requests that start later.  Every logit equals the plain model's on that request alone."""
    from nnis_amd.engine.batch import StepEntry

    config = MUTEDRA_CONFIGS[name][0]
    plain = M.PlainMutedra(folders[name])
    engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=64 * 9, max_slots=4)
    yard = Yardstick(plain)
    for batch_seed, lengths in ((0, [1, 70, 130, 9]), (1, [65, 3, 128]), (2, [2, 2, 200, 64])):
        requests = [_ids(n + decode, config["vocab"], 100 * batch_seed + i) for i, (n, decode) in enumerate(zip(lengths, (12, 5, 9, 1)))]
        slots = [engine.start_sequence() for _ in requests]
        at = list(lengths)
        logits = engine.step([StepEntry(s, r[:n], list(range(n))) for s, r, n in zip(slots, requests, lengths)]).cpu()
        row = 0
        for i, n in enumerate(lengths):
            yard.check(logits[row:row + n], requests[i], dtype, f"{name} batch {batch_seed} prompt {i}", rows=slice(0, n))
            row += n
        live = list(range(len(requests)))
        while live:
            live = [i for i in live if at[i] < len(requests[i]) or engine.end_sequence(slots[i])]
            if not live:
                break
            logits = engine.step([StepEntry(slots[i], [requests[i][at[i]]], [0]) for i in live]).cpu()
            for row, i in enumerate(live):
                yard.check(logits[row], requests[i], dtype, f"{name} batch {batch_seed} request {i} position {at[i]}", rows=at[i])
                at[i] += 1
        assert engine.free_slots() == 4 and engine.free_pages() == 9


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_across_windows_and_pages(folders, dtype):
    """330 tokens one by one behind a prompt of 3: the windows of 64 and 70 tokens pass over decoded tokens, the kept
    first tokens fall out of the window, four page borders are crossed."""
    for name in ("B", "C"):
        config = MUTEDRA_CONFIGS[name][0]
        plain = M.PlainMutedra(folders[name])
        engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=512)
        ids = _ids(330, config["vocab"], 4)
        slot = engine.start_sequence()
        got = _collect(engine, slot, ids, [3] + list(range(4, 331)))
        yard = Yardstick(plain)
        yard.check(got, ids, dtype, f"{name} long decoding")
        yard.check(got[-1], ids, dtype, f"{name} long decoding, the last token", rows=len(ids) - 1)


@pytest.mark.parametrize("name", sorted(MUTEDRA_CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name):
    """``nnis_amd.generate``: the library's scheduler, batches and selection on the device.  In 32-bit the tokens are
    the plain model's, unless two logits are closer than rounding."""
    config = MUTEDRA_CONFIGS[name][0]
    plain = M.PlainMutedra(folders[name])
    prompts = [_ids(n, config["vocab"], 50 + n) for n in (1, 19, 70)]
    got = nnis_amd.generate(folders[name], prompts, max_new_tokens=10, dtype="float32", stop_token_ids=[])
    for prompt, tokens in zip(prompts, got):
        assert len(tokens) == 10
        logits = plain.logits(prompt + tokens)[len(prompt) - 1:-1]
        for row, token in zip(logits, tokens):
            assert float(row[token]) >= float(row.max()) - 1e-4 * float(row.abs().max()), "a generated token is not the plain model's best"
    got16 = nnis_amd.generate(folders[name], prompts, max_new_tokens=6, dtype="bfloat16", stop_token_ids=[])
    assert [len(t) for t in got16] == [6, 6, 6]


def test_the_command_line_runs_the_model(folders):
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "nnis"), "generate", "--model", folders["A"], "--prompt-ids", "5,17,3",
                           "--max-new-tokens", "4", "--dtype", "float32"], capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    plain = M.PlainMutedra(folders["A"])
    assert [int(t) for t in done.stdout.strip().splitlines()[-1].split(",")] == plain.greedy([5, 17, 3], 4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_model_without_the_optional_mechanisms(tmp_path, dtype):
    """No loop, no embedding scale, no cap of the logits, an attention without window and bias (the sink stays)."""
    import copy

    config = copy.deepcopy(MUTEDRA_CONFIGS["A"][0])
    del config["loop"], config["logit_softcap"], config["embedding"]["scale"]
    del config["layers"][1]["mixer"]["mask"], config["layers"][1]["mixer"]["bias_max"], config["layers"][1]["mixer"]["bias_buckets"]
    folder = str(tmp_path / "bare")
    nnis_amd.write_random_model(folder, config, 41)
    _sharpen(folder)
    plain = M.PlainMutedra(folder)
    engine = nnis_amd.load_engine(folder, dtype=dtype, max_tokens=512)
    ids = _ids(100, config["vocab"], 6)
    slot = engine.start_sequence()
    got = _collect(engine, slot, ids, [70] + list(range(71, 101)))
    Yardstick(plain).check(got, ids, dtype, "a model without the optional mechanisms")


SIZES = {"attention": [(32, 16), (16, 48)], "latent": [(32, 16), (48, 0), (64, 32), (40, 0), (24, 8)]}  # modules that are built beforehand


def test_other_sizes_drawn_from_a_seed(tmp_path):
    """Configurations whose every size is drawn at random, in 32-bit against the plain model: prompt, a portion, single tokens."""
    import random

    for seed in range(6):
        r = random.Random(seed)
        layers = []
        for _ in range(r.randint(1, 4)):
            ff = r.choice([None, r.randint(8, 90)])
            if r.random() < 0.4:
                dim, vdim = r.choice(SIZES["attention"])
                buckets = 2 * r.randint(1, 9)
                layers.append(layer("attention", windowed(r.randint(1, 3) * (k := r.randint(1, 2)), k, dim, vdim, window=r.randint(1, 90),
                                                          keep_first=r.choice([0, 1, r.randint(2, 70)]), bias_max=buckets // 2 + r.randint(1, 80),
                                                          buckets=buckets, scale=r.uniform(0.05, 0.5)), ff))
            else:
                rank, rot = r.choice(SIZES["latent"])
                kind = "latent_attention_2" if rot else "latent_attention"
                layers.append(layer(kind, latent(r.randint(1, 5), r.randint(1, 40), r.randint(1, 40), r.randint(1, 50), rank,
                                                 scale=r.uniform(0.05, 0.5), rot_dim=rot or None, base=r.choice([50.0, 1e4, 1e6])), ff))
        start = r.randint(0, len(layers))
        config = mutedra(vocab=r.randint(20, 400), width=4 * r.randint(3, 30), layers=layers,
                         loop=(start, r.randint(start, len(layers)), r.randint(1, 3)), scale=r.choice([1.0, r.uniform(0.5, 20.0)]),
                         softcap=r.uniform(5.0, 60.0), eps=r.choice([1e-5, 1e-6, 1e-3]))
        folder = str(tmp_path / f"m{seed}")
        nnis_amd.write_random_model(folder, config, seed)
        _sharpen(folder)
        plain = M.PlainMutedra(folder)
        engine = nnis_amd.load_engine(folder, dtype="float32", max_tokens=256)
        ids = _ids(80, config["vocab"], seed)
        want = plain.logits(ids)
        slot = engine.start_sequence()
        got = _collect(engine, slot, ids, [66, 70] + list(range(71, 81)))
        assert _relative(got, want) < 5e-5, f"seed {seed}: {config}"
