"""Mutedra on the CPU: its configuration reader, its model description, the
cache it asks for, the table of distance biases, and the plain implementation's
own mechanisms against special cases."""

import copy
import math

import pytest
import torch

import nnis_amd
import plain_mutedra as M
from mutedra_configs import MUT_A, MUT_B, MUT_C, MUTEDRA_CONFIGS
from nnis_amd.config.registry import spec_from_config
from nnis_amd.errors import InvalidInput, Unsupported
from nnis_amd.models.decoder import DecoderModel
from nnis_amd.parts.attention import distance_bucket
from nnis_amd.parts.base import KVRequest


def test_the_architecture_is_chosen_by_its_name():
    cfg, spec = spec_from_config(MUT_A)
    assert spec.architecture == "Mutedra" and spec.width == 96 and spec.vocab_size == 300 and spec.max_positions is None
    assert "Mutedra" in nnis_amd.config.registered_architectures()
    with pytest.raises(Unsupported):
        spec_from_config(dict(MUT_A, architecture="Mutedra2"))


@pytest.mark.parametrize("config, runs", [
    (MUT_A, [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None)]),
    (MUT_B, [(0, 0), (1, None)]),
    (MUT_C, [(0, 0), (1, None), (0, 1), (1, None), (2, None), (3, None)])])
def test_passes_and_their_entries(config, runs):
    cfg, spec = spec_from_config(config)
    assert cfg.layer_runs() == runs
    assert [entry.layer for entry in spec.schedule] == [layer for layer, _ in runs]
    assert all(entry.reads_cache_of is None for entry in spec.schedule)  # every run keeps a cache of its own
    for entry, (_, number) in zip(spec.schedule, runs):
        if number is None:
            assert entry.enter is None
        else:
            assert entry.enter["row"] == number and entry.enter["add_embedding"] == (number > 0)
            assert entry.enter["rows"] == config["loop"]["times"]
    assert M.PlainMutedra.runs(type("stub", (), {"config": config})()) == runs


def test_missing_and_wrong_keys_are_refused():
    for path in (["vocab"], ["norm", "eps"], ["loop", "times"],
                 ["layers", 0, "mixer", "kv_rank"], ["layers", 0, "mixer", "rot"], ["layers", 0, "mixer", "rot_dim"],
                 ["layers", 1, "mixer", "mask", "keep_first"], ["layers", 1, "mixer", "scale"],
                 ["layers", 1, "mlp"], ["layers", 2, "mlp", "ff"], ["layers", 2, "mixer", "q_rank"]):
        raw = copy.deepcopy(MUT_A)
        at = raw
        for key in path[:-1]:
            at = at[key]
        del at[path[-1]]
        with pytest.raises(InvalidInput):
            spec_from_config(raw)
    for change, error in ((lambda raw: raw["layers"][0].update(type="conv"), Unsupported),
                          (lambda raw: raw["loop"].update(stop=7), InvalidInput),
                          (lambda raw: raw["layers"][1]["mixer"].update(kv_heads=3), InvalidInput),
                          (lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=8), Unsupported),
                          (lambda raw: raw["layers"][2]["mlp"].update(kind="routed"), Unsupported)):
        raw = copy.deepcopy(MUT_A)
        change(raw)
        with pytest.raises(error):
            spec_from_config(raw)


def test_a_mechanism_that_the_file_does_not_mention_does_not_exist():
    raw = copy.deepcopy(MUT_A)
    del raw["loop"], raw["logit_softcap"], raw["embedding"]["scale"]
    del raw["layers"][1]["mixer"]["mask"], raw["layers"][1]["mixer"]["bias_max"]
    cfg, spec = spec_from_config(raw)
    assert cfg.layer_runs() == [(0, None), (1, None), (2, None)] and all(entry.enter is None for entry in spec.schedule)
    assert spec.embedding["scale"] == 1.0 and spec.head["softcap"] is None
    mixer = spec.layers[1]["mixer"]
    assert "window" not in mixer and "distance_bias" not in mixer and mixer["sink"] == "zero"
    model = DecoderModel(spec)
    names = {t.name for t in model.tensors()}
    assert "loop.step" not in names and "l1.mix.rel" not in names
    assert model.cache_requests()[0][1][1] == KVRequest(2, 32, None, 16)


def test_tensors_and_cache_requests():
    _, spec = spec_from_config(MUT_A)
    model = DecoderModel(spec)
    shapes = {t.name: t.shape for t in model.tensors()}
    assert shapes["loop.step"] == (3, 96) and shapes["l1.mix.rel"] == (12, 4) and shapes["l0.mix.sink"] == (3,)
    assert shapes["l0.mix.dkv"] == (32 + 16, 96) and shapes["l0.mix.uq"] == (3 * (16 + 16), 40) and shapes["l0.mix.g"] == (3, 96)
    assert shapes["l0.norm1.alpha"] == () and shapes["final.norm.b"] == (96,) and "l1.mlp.gate" not in shapes
    assert "l2.mix.sink" not in shapes and "l2.mix.g" not in shapes
    requests, shared = model.cache_requests()
    assert not shared and len(requests) == 7
    by_layer = {spec.schedule[index].layer: request for index, request in requests}
    # the latent is the one key/value head: keys [latent | rotated part], values the latent
    assert by_layer[0] == KVRequest(1, 48, None, 32) and by_layer[2] == KVRequest(1, 48, None, None)
    assert by_layer[1] == KVRequest(2, 32, 37, 16)


@pytest.mark.parametrize("rows, reach", [(12, 50), (8, 90), (6, 20), (10, 33), (16, 120), (32, 128), (2, 5)])
def test_the_bias_table_by_distance(rows, reach):
    half = rows // 2
    got = [distance_bucket(n, rows, reach) for n in range(3 * reach)]
    assert got == [M.bias_row(n, rows, reach) for n in range(3 * reach)]
    assert got[:half] == list(range(half)) and got[half] == half  # the distance itself, then the first of the wider steps
    assert all(a <= b for a, b in zip(got, got[1:])) and max(got) == rows - 1
    assert all(row == rows - 1 for row in got[reach:])  # the last row is met at `reach` and holds beyond


def test_plain_mechanisms_in_special_cases():
    generator = torch.Generator().manual_seed(0)
    x = torch.randn(9, 10, generator=generator, dtype=torch.float64)
    # a norm with alpha -> 0 is linear in x: tanh(a x) ~ a x
    w, b = torch.randn(10, generator=generator, dtype=torch.float64), torch.randn(10, generator=generator, dtype=torch.float64)
    assert torch.allclose(M.tanh_norm(x, w, b, 1e-6), 1e-6 * x * w + b, atol=1e-15)
    # a turn by position 0 changes nothing; a turn keeps every pair's length; turns add up
    turned = M.turn_pairs(x, torch.arange(9), 100.0)
    assert torch.equal(turned[0], x[0])
    assert torch.allclose(turned[:, 0::2] ** 2 + turned[:, 1::2] ** 2, x[:, 0::2] ** 2 + x[:, 1::2] ** 2)
    assert torch.allclose(M.turn_pairs(M.turn_pairs(x, torch.full((9,), 3), 100.0), torch.full((9,), 4), 100.0),
                          M.turn_pairs(x, torch.full((9,), 7), 100.0))
    # windowed attention with a window over everything, no bias and a sink that the scores dwarf is ordinary causal attention
    sizes = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 5, "scale": 0.5, "bias_max": 9, "mask": {"size": 100, "keep_first": 0}}
    weights = {"q": torch.randn(8, 10, generator=generator, dtype=torch.float64), "k": torch.randn(4, 10, generator=generator, dtype=torch.float64),
               "v": torch.randn(5, 10, generator=generator, dtype=torch.float64), "o": torch.eye(10, dtype=torch.float64),
               "rel": torch.zeros(4, 2, dtype=torch.float64)}
    got = M.windowed_attention(x, weights, sizes)
    q, k, v = (x @ weights["q"].T).view(9, 2, 4), x @ weights["k"].T, x @ weights["v"].T
    for head in range(2):
        s = (q[:, head] @ k.T) * 0.5
        s = s.masked_fill(torch.triu(torch.ones(9, 9, dtype=torch.bool), 1), -math.inf)
        e = torch.exp(s)
        want = (e / (1.0 + e.sum(1, keepdim=True))) @ v
        assert torch.allclose(got[:, 5 * head:5 * head + 5], want)
    # a window of one token and no kept tokens: each token sees itself only
    sizes["mask"] = {"size": 1, "keep_first": 0}
    got = M.windowed_attention(x, weights, sizes)
    s = ((q[:, 0] * k).sum(1) * 0.5).exp()
    assert torch.allclose(got[:, :5], (s / (1 + s))[:, None] * v)


def test_random_models_are_written_and_described(tmp_path):
    for name, (config, seed) in MUTEDRA_CONFIGS.items():
        folder = str(tmp_path / name)
        nnis_amd.write_random_model(folder, config, seed)
        plain = M.PlainMutedra(folder)
        logits = plain.logits([1, 2, 3, 4, 5])
        assert logits.shape == (5, config["vocab"]) and bool(torch.isfinite(logits).all())
        assert float(logits.abs().max()) <= config["logit_softcap"]
        # causal: a later token changes no earlier logit
        assert torch.equal(plain.logits([1, 2, 3, 4, 5, 6])[:5], logits)
