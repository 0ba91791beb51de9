"""Tumadra's configuration reader and plan, and the plain implementation's own pieces (no GPU)."""
import copy

import pytest
import torch

import plain_tumadra as plain
from tumadra_models import CONFIG_A, CONFIG_B, CONFIG_C, CONFIG_D, n_layer_runs, random_weights


def test_plan_follows_the_file():
    from imparo_amd.config import plan_from_config
    from imparo_amd.engine.model import declared_tensors
    for config in (CONFIG_A, CONFIG_B, CONFIG_C, CONFIG_D):
        cfg, plan = plan_from_config(config)
        assert plan.architecture == "Tumadra" and not cfg.unread_keys
        assert [c.layer for c in plan.order] == plain.run_order(config)
        assert len(plan.order) == n_layer_runs(config)
        declared = {k: tuple(d.shape) for k, (d, _) in declared_tensors(plan).items()}
        assert declared == {k: tuple(v.shape) for k, v in random_weights(config, 0).items()}
        for layer, entry in zip(plan.layers, config["layers"]):
            assert ("ffn" in layer.parts) == (entry["mlp"] is not None)
            assert layer.spec("mixer_norm")["groups"] == config["norm"]["groups"]
    assert [c.layer for c in plan_from_config(CONFIG_A)[1].order] == [0, 1, 0, 1, 0, 1, 2, 3]


def test_each_pass_of_a_loop_has_its_own_state():
    from imparo_amd.config import plan_from_config
    _, plan = plan_from_config(CONFIG_A)
    assert all(c.cache_of is None for c in plan.order)


def test_refusals():
    from imparo_amd.config import BadValue, Inconsistent, MissingKey, UnknownArchitecture, plan_from_config
    def changed(**kw):
        c = copy.deepcopy(CONFIG_A)
        c.update(kw)
        return c
    with pytest.raises(UnknownArchitecture):
        plan_from_config(changed(architecture="Tumadro"))
    with pytest.raises(MissingKey):
        plan_from_config({k: v for k, v in CONFIG_A.items() if k != "norm"})
    with pytest.raises(Inconsistent):
        plan_from_config(changed(norm=dict(eps=1e-5, groups=5)))
    with pytest.raises(Inconsistent):
        plan_from_config(changed(loop=dict(start=2, stop=9, times=2)))
    bad = copy.deepcopy(CONFIG_A)
    bad["layers"][0]["type"] = "mamba7"
    with pytest.raises(BadValue):
        plan_from_config(bad)
    bad = copy.deepcopy(CONFIG_A)
    bad["layers"][1]["mlp"]["kind"] = "routed"
    with pytest.raises(BadValue):
        plan_from_config(bad)
    bad = copy.deepcopy(CONFIG_A)
    del bad["layers"][1]["mixer"]["vdim"]
    with pytest.raises(MissingKey):
        plan_from_config(bad)
    extra = changed(something_new=3)
    assert plan_from_config(extra)[0].unread_keys == ["something_new"]


def test_paged_state_with_a_fixed_part_groups_and_resets():
    """A site that keeps pages and a fixed-size row: equal specs share a group, and the manager counts it
    among the sites whose slots are cleared."""
    from imparo_amd.cache.pages import (PAGE, CacheManager, FixedArray, FixedSpec, PagedArray, PagedSpec, fixed_part,
                                        with_fixed_arrays)
    kv = PagedSpec((PagedArray("k", (2, PAGE, 8)), PagedArray("v", (1, PAGE, 12))))
    extra = (FixedArray("shift_prev", (16,)),)
    both = with_fixed_arrays(kv, extra)
    assert isinstance(both, PagedSpec) and fixed_part(both).all_arrays() == extra and both != kv
    only = with_fixed_arrays(None, extra)
    assert isinstance(only, FixedSpec)
    scan = with_fixed_arrays(FixedSpec(arrays=(FixedArray("scan", (4, 2)),)), extra)
    assert [a.name for a in scan.all_arrays()] == ["scan", "shift_prev"]
    m = CacheManager([both, scan, with_fixed_arrays(kv, extra), None], 8, 4, 2)
    assert len(m.groups) == 1 and m.groups[0].sites == [0, 2] and m.fixed_sites == [0, 1, 2]


# ---- the plain implementation's pieces against library routines and by hand
def test_plain_group_norm_and_shift():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(5, 12, generator=g), torch.rand(12, generator=g)
    one = plain.group_norm(x, w, 1, 1e-5)
    assert torch.allclose(one, x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w)
    three = plain.group_norm(x, w, 3, 1e-5)
    for k in range(3):
        part = x[:, 4 * k:4 * k + 4]
        assert torch.allclose(three[:, 4 * k:4 * k + 4], part / torch.sqrt((part * part).mean(-1, keepdim=True) + 1e-5) * w[4 * k:4 * k + 4])
    mix = torch.rand(12, generator=g)
    s = plain.token_shift(x, mix)
    assert torch.allclose(s[0], x[0] * (1 - mix)) and torch.allclose(s[3], x[3] * (1 - mix) + x[2] * mix)
    assert torch.equal(plain.token_shift(x, torch.zeros(12)), x)


def test_plain_sinusoid_and_temperature():
    s = plain.sinusoid(torch.arange(7), 10)
    assert torch.allclose(s[:, 0], torch.sin(torch.arange(7.0))) and torch.allclose(s[:, 1], torch.cos(torch.arange(7.0)))
    assert torch.allclose(s[3, 4], torch.sin(torch.tensor(3.0 * 10000.0 ** (-4 / 10))))
    t = plain.query_temperature(torch.arange(20), 0.5, 8)
    assert float(t[6]) == 1.0 and abs(float(t[7]) - (1 + 0.5 * torch.log(torch.tensor(2.0)))) < 1e-6
    assert abs(float(t[15]) - (1 + 0.5 * torch.log(torch.tensor(3.0)))) < 1e-6


def test_plain_differential_core_is_two_softmaxes():
    g = torch.Generator().manual_seed(1)
    q, k, v = torch.randn(6, 2, 2, 4, generator=g), torch.randn(6, 1, 2, 4, generator=g), torch.randn(6, 1, 5, generator=g)
    out = plain.differential_core(q, k, v, torch.arange(6), 0.5, 0.8, 0.25, 1e-6).reshape(6, 2, 5)
    mask = torch.tril(torch.ones(6, 6, dtype=torch.bool))
    for h in range(2):
        a = [torch.nn.functional.scaled_dot_product_attention(q[None, :, h, m], k[None, :, 0, m], v[None, :, 0], attn_mask=mask,
                                                              scale=0.5)[0] for m in range(2)]
        o = a[0] - 0.8 * a[1]
        assert torch.allclose(out[:, h], o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6) * 0.75, atol=1e-5)


def test_plain_scan_and_conv_continue():
    """The recurrence cut in two gives what the whole gives; the conv equals the library's with left padding."""
    g = torch.Generator().manual_seed(2)
    T, C, N = 9, 6, 3
    dt, x = torch.rand(T, C, generator=g) * 0.3, torch.randn(T, C, generator=g)
    B, Cm = torch.randn(T, N, generator=g), torch.randn(T, N, generator=g)
    A, D = -torch.rand(C, N, generator=g) * 4, torch.randn(C, generator=g)
    whole = plain.scan(dt, x, B, Cm, A, D)
    S = torch.zeros(C, N)
    parts = torch.cat([plain.scan(dt[:4], x[:4], B[:4], Cm[:4], A, D, S), plain.scan(dt[4:], x[4:], B[4:], Cm[4:], A, D, S)])
    assert torch.allclose(whole, parts, atol=1e-6)
    w, b = torch.randn(C, 4, generator=g), torch.randn(C, generator=g)
    lib = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), w[:, None, :], b, groups=C)[0].T
    assert torch.allclose(plain.causal_conv(x, w, b), lib, atol=1e-6)
