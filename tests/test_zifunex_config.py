"""Zifunex on the CPU: its configuration reader, its model description, the
cache it asks for, and the plain implementation's own mechanisms."""

import copy
import math

import pytest
import torch

import nnis_amd
import plain_zifunex as Z
from nnis_amd.config.registry import spec_from_config
from nnis_amd.errors import InvalidInput, Unsupported
from nnis_amd.models.decoder import DecoderModel
from zifunex_configs import ZIF_A, ZIF_B, ZIF_C, ZIFUNEX_CONFIGS


def test_the_architecture_is_chosen_by_its_name():
    cfg, spec = spec_from_config(ZIF_A)
    assert spec.architecture == "Zifunex" and spec.width == 96 and spec.vocab_size == 300 and spec.max_positions is None
    assert "Zifunex" in nnis_amd.config.registered_architectures()
    with pytest.raises(Unsupported):
        spec_from_config(dict(ZIF_A, architecture="Zifunex2"))


@pytest.mark.parametrize("config, runs", [(ZIF_A, [0, 1, 0, 1, 2]), (ZIF_B, [0, 1]), (ZIF_C, [0, 1, 2, 1, 2, 1, 2, 3])])
def test_a_looped_stretch_runs_several_times_with_the_same_weights(config, runs):
    cfg, spec = spec_from_config(config)
    assert cfg.layer_runs() == runs
    assert [entry.layer for entry in spec.schedule] == runs
    assert all(entry.reads_cache_of is None for entry in spec.schedule)  # every run keeps a cache or state of its own


def test_missing_and_wrong_keys_are_refused():
    for path in (["vocab"], ["norm", "eps"], ["embedding", "bigram", "buckets"], ["layers", 0, "mixer", "tau"],
                 ["layers", 1, "mixer", "left", "softcap"], ["layers", 1, "mixer", "right", "conv"], ["layers", 2, "mlp", "ff"],
                 ["layers", 1, "mlp"], ["streams"]):
        raw = copy.deepcopy(ZIF_A)
        at = raw
        for key in path[:-1]:
            at = at[key]
        del at[path[-1]]
        with pytest.raises(InvalidInput):
            spec_from_config(raw)
    raw = copy.deepcopy(ZIF_A)
    raw["layers"][0]["type"] = "conv"
    with pytest.raises(Unsupported):
        spec_from_config(raw)
    raw = copy.deepcopy(ZIF_A)
    raw["loop"]["stop"] = 7
    with pytest.raises(InvalidInput):
        spec_from_config(raw)
    raw = copy.deepcopy(ZIF_A)
    raw["layers"][1]["mixer"]["left"]["kv_heads"] = 3
    with pytest.raises(InvalidInput):
        spec_from_config(raw)
    raw = copy.deepcopy(ZIF_A)
    raw["layers"][1]["mixer"]["left"]["rot"]["dims"] = 34
    with pytest.raises(InvalidInput):
        spec_from_config(raw)


def test_tensors_follow_the_configuration():
    _, spec = spec_from_config(ZIF_A)
    shapes = {t.name: tuple(t.shape) for t in DecoderModel(spec).tensors()}
    assert shapes["embed"] == (300, 96) and shapes["bigram"] == (212, 96) and shapes["head"] == (300, 96)
    assert shapes["l0.mix.q"] == (48, 96) and shapes["l0.mix.v"] == (72, 96) and shapes["l0.mix.a1"] == (8, 96) and shapes["l0.mix.a2"] == (48, 8)
    assert shapes["l0.mix.norm"] == (24,) and shapes["l0.hc1.mix"] == (2, 2) and shapes["l0.hc2.in"] == (2,)
    assert shapes["l1.mix.left.q"] == (128, 96) and shapes["l1.mix.left.k"] == (64, 96) and shapes["l1.mix.left.v"] == (32, 96)
    assert shapes["l1.mix.left.o"] == (96, 64) and shapes["l1.mix.left.o.b"] == (96,) and shapes["l1.mix.left.v.b"] == (32,)
    assert shapes["l1.mix.right.in"] == (160, 96) and shapes["l1.mix.right.x"] == (5 + 24, 80) and shapes["l1.mix.right.dt"] == (80, 5)
    assert shapes["l1.mix.right.conv"] == (80, 3) and shapes["l1.mix.right.A_log"] == (80, 12) and shapes["l1.mix.left.out"] == (96,)
    assert "l1.norm2" not in shapes and "l1.hc2.mix" not in shapes and "l1.mlp.gate" not in shapes  # no feed-forward there
    assert shapes["l2.mlp.down"] == (96, 160) and shapes["final.norm.b"] == (96,)
    # without the inner size of the decays' projections in the file, that size is left to the tensors
    raw = copy.deepcopy(ZIF_A)
    del raw["layers"][0]["mixer"]["rank"]
    shapes = {t.name: tuple(t.shape) for t in DecoderModel(spec_from_config(raw)[1]).tensors()}
    assert shapes["l0.mix.a1"] == (None, 96) and shapes["l0.mix.a2"] == (48, None)


def test_the_cache_gives_every_run_what_its_mixers_ask_for():
    from nnis_amd.cache import SequenceCache
    from nnis_amd.cache.cache import KVView, StateView

    _, spec = spec_from_config(ZIF_A)
    model = DecoderModel(spec)
    requests, shared = model.cache_requests()
    assert not shared and [index for index, _ in requests] == ["embedding", 0, 1, 2, 3, 4]
    cache = SequenceCache(requests, shared, 256, 256, torch.float32, "cpu")
    assert isinstance(cache.view("embedding"), StateView) and cache.view("embedding").state.dtype == torch.int32
    assert isinstance(cache.view(0), StateView) and cache.view(0).state.shape[1:] == (3, 16, 24)
    assert cache.view(0).state is not cache.view(2).state  # the second pass over the same layer has a state of its own
    left, right = cache.view(1)
    assert isinstance(left, KVView) and left.v_pages.shape[-5] == 1 and left.k_pages.shape[-3] == 4  # values of 16, keys of 32 channels
    assert right[0].state.shape[1:] == (80, 12) and right[1].state.shape[1:] == (2, 80)
    assert cache.view(1)[0].k_pages is not cache.view(3)[0].k_pages
    assert len(cache.kv_groups) == 2  # the two kinds of attention layers keep pages of their own shapes
    # a slot that is taken again starts from zero state
    slot = cache.acquire()
    cache.view(0).state[slot].fill_(3.0)
    right[1].state[slot].fill_(2.0)
    cache.view("embedding").state[slot] = 17
    cache.release(slot)
    assert cache.acquire() == slot
    assert float(cache.view(0).state[slot].abs().sum()) == 0 and float(right[1].state[slot].abs().sum()) == 0
    assert int(cache.view("embedding").state[slot]) == 0
    with pytest.raises(InvalidInput):
        cache.grow({slot: 5}) or cache.truncate(slot, 2)  # state has consumed the tokens


@pytest.mark.parametrize("name", sorted(ZIFUNEX_CONFIGS))
def test_a_random_model_is_written_and_read_by_the_plain_implementation(tmp_path, name):
    config, seed = ZIFUNEX_CONFIGS[name]
    nnis_amd.write_random_model(str(tmp_path), config, seed)
    plain = Z.PlainZifunex(str(tmp_path))
    ids = [5, 9, 9, 200, 1, 0, 7, 7, 7, 33, 150]
    layers = []
    logits = plain.logits(ids, layers_out=layers)
    assert logits.shape == (len(ids), config["vocab"]) and bool(torch.isfinite(logits).all())
    assert len(layers) == len(plain.layer_runs())
    # causal: a position's logits do not depend on what follows it
    again = plain.logits(ids[:6])
    assert float((again - logits[:6]).abs().max()) < 1e-9
    assert float(logits.std()) > 1e-3


def test_plain_mechanisms():
    assert Z.bigram_rows([4, 9, 9, 0], 97, 3, 5) == [97, (4 * 3 + 9 * 5) % 97, (9 * 3 + 9 * 5) % 97, (9 * 3) % 97]
    x = torch.randn(5, 3, 12, dtype=torch.float64)
    y = Z.rotate_half(x, [0, 1, 2, 3, 100], 8, 100.0)
    assert torch.allclose(y[0], x[0]) and torch.allclose(y[..., 8:], x[..., 8:])  # position 0 and the channels beyond the rotation
    assert torch.allclose(y[..., :8].norm(dim=-1), x[..., :8].norm(dim=-1))
    a = 1.0 * 100.0 ** (-2.0 * 1 / 8)  # channel 1 pairs with channel 5
    assert math.isclose(float(y[1, 0, 1]), float(x[1, 0, 1] * math.cos(a) - x[1, 0, 5] * math.sin(a)), rel_tol=1e-12)
    assert math.isclose(float(y[1, 0, 5]), float(x[1, 0, 5] * math.cos(a) + x[1, 0, 1] * math.sin(a)), rel_tol=1e-12)
    z = torch.linspace(-4, 4, 9, dtype=torch.float64)
    assert torch.allclose(Z.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    u = torch.randn(4, 6, dtype=torch.float64)
    w, b = torch.randn(6, dtype=torch.float64), torch.randn(6, dtype=torch.float64)
    assert torch.allclose(Z.layer_norm(u, w, b, 1e-5), torch.nn.functional.layer_norm(u, (6,), w, b, 1e-5))
    # streams: with the identity as mix and a zero gain nothing changes
    streams = torch.randn(3, 4, 6, dtype=torch.float64)
    p = {"in": torch.ones(3, dtype=torch.float64), "mix": torch.eye(3, dtype=torch.float64), "out": torch.zeros(3, dtype=torch.float64)}
    assert torch.equal(Z.hyper_sublayer(streams, p, lambda u: u), streams)
    # mix is indexed [from, to]
    p["mix"] = torch.zeros(3, 3, dtype=torch.float64)
    p["mix"][0, 2] = 1.0
    out = Z.hyper_sublayer(streams, p, lambda u: u)
    assert torch.equal(out[2], streams[0]) and float(out[0].abs().sum()) == 0
