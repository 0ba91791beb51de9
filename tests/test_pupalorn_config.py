"""The Pupalorn configuration reader and plan, on the CPU: what the file's keys become, what is refused,
and that the plain implementation's frequency table equals the engine's."""
import copy

import numpy as np
import pytest
import torch

import plain_pupalorn as plain
from imparo_amd.config import ConfigError, plan_from_config
from imparo_amd.config.errors import BadValue, Inconsistent, MissingKey
from imparo_amd.engine.model import declared_tensors
from imparo_amd.parts.position import scale_by_wavelength
from pupalorn_models import CONFIGS, random_weights


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_plan_declares_the_tensors_the_model_has(name):
    cfg, seed = CONFIGS[name]
    typed, plan = plan_from_config(cfg)
    assert typed.unread_keys == []
    declared = declared_tensors(plan)
    have = random_weights(cfg, seed)
    assert set(declared) == set(have)
    for k, (decl, _) in declared.items():
        assert tuple(decl.shape) == tuple(have[k].shape), k


def test_plan_of_a():
    typed, plan = plan_from_config(CONFIGS["A"][0])
    assert [c.cache_of for c in plan.order] == [None, None, 0, 1]
    assert [l.arrangement for l in plan.layers] == ["sandwich"] * 4
    assert "ffn" not in plan.layers[1].parts and "ffn_post" not in plan.layers[1].parts
    m0, m2, m3 = plan.layers[0].mixer, plan.layers[2].mixer, plan.layers[3].mixer
    assert (m0["window"], m0["keep_window"]) == (24, 40)        # layer 2 looks further back into layer 0's cache
    assert (m2["window"], m2["keep_window"], m2["shared_kv"]) == (40, 40, True)
    assert plan.layers[1].mixer["keep_window"] is None and m3["window"] == 9 and m3["keep_window"] is None
    assert plan.layers[0].mixer_post["multiplier"] == 0.5 and plan.embedding["scale"] == 1.7
    assert plan.layers[0].ffn["identity"] == 2 and plan.layers[3].ffn["top"] == 4
    _, plan_b = plan_from_config(CONFIGS["B"][0])
    assert plan_b.embedding["scale"] == 1.0 and plan_b.layers[0].mixer_post["multiplier"] == 1.0
    assert plan_b.layers[1].mixer["position"] is None


def _broken(change):
    cfg = copy.deepcopy(CONFIGS["A"][0])
    change(cfg)
    return cfg


@pytest.mark.parametrize("change,error", [
    (lambda c: c.pop("norm"), MissingKey),
    (lambda c: c["layers"][0]["mixer"].pop("vdim"), MissingKey),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), BadValue),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "dense"), BadValue),
    (lambda c: c["layers"][0]["mixer"].__setitem__("heads", 3), Inconsistent),
    (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 2), Inconsistent),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 2), Inconsistent),       # layer 2 has no keys itself
    (lambda c: c["layers"][2]["mixer"].__setitem__("dim", 32), Inconsistent),          # differs from its source's
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 18), Inconsistent),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 7), Inconsistent),
    (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), BadValue),
])
def test_refused(change, error):
    with pytest.raises(error):
        plan_from_config(_broken(change))
    assert issubclass(error, ConfigError)


@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, (4.0, 1.0, 4.0, 200)), (16, 100.0, (4.0, 1.0, 8.0, 64)),
                                               (64, 10000.0, (8.0, 1.0, 4.0, 512)), (128, 500000.0, (32.0, 1.0, 4.0, 8192))])
def test_frequency_scaling_has_three_bands(dims, base, scaling):
    keys = dict(zip(("factor", "low", "high", "original"), scaling))
    want = plain.inverse_frequencies(dims, base, keys).numpy()
    raw = plain.inverse_frequencies(dims, base, None).numpy()
    got = scale_by_wavelength(raw, **keys)
    np.testing.assert_allclose(got, want, rtol=1e-14)
    kept, divided = np.isclose(got, raw, rtol=1e-12), np.isclose(got, raw / scaling[0], rtol=1e-12)
    assert kept.any() and divided.any() and (~kept & ~divided).any(), "a band is not met by this case"
    assert np.all(np.diff(got) < 0)


def test_random_weights_mode_writes_a_loadable_model(tmp_path):
    """The seeded random-weights mode writes what the plan declares, and the by-name loader takes it back;
    a file with a tensor that a layer on borrowed keys must not have is refused by name."""
    from imparo_amd import WeightsError, write_random_model
    from imparo_amd.weights import load_weights
    from imparo_amd.weights.safetensors_io import save_file
    cfg = CONFIGS["A"][0]
    d = write_random_model(cfg, 5, str(tmp_path / "m"))
    _, plan = plan_from_config(cfg)
    declared = {k: decl for k, (decl, _) in declared_tensors(plan).items()}
    tensors = load_weights(d, declared)
    tensors.pop("__file__").close()
    assert set(tensors) == set(declared)
    assert float(tensors["l0.norm1"].float().abs().max()) < 0.2        # kept as the distance from one
    assert abs(float(tensors["l0.ls1"].float().mean()) - 1.0) < 0.1
    extra = dict(tensors)
    extra["l2.mix.k"] = tensors["l0.mix.k"].clone()
    save_file({k: v.contiguous() for k, v in extra.items()}, str(tmp_path / "m" / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_weights(d, declared)
    assert e.value.unexpected == ["l2.mix.k"]
