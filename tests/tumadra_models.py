"""Small Tumadra configurations with random weights, for tests. The weights are drawn so that every
mechanism matters: projections of unit gain, token-shift mixes across (0, 1), step sizes of a few
hundredths to a few tenths, decays over a range, activation coefficients of order one."""
import json
import math
import os

import torch


def attention(heads, kv_heads, dim, vdim, diff=0.4, scale=None, q_temp=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, diff=diff,
             scale=scale if scale is not None else 1.0 / math.sqrt(dim))
    if q_temp is not None:
        m["q_temp"] = dict(coef=q_temp[0], every=q_temp[1])
    return m


def layer(kind, mixer, ff):
    return dict(type=kind, mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff))


# A: a loop over two layers three times, kv heads shared by two heads, dt_rank below 8, a layer without feed-forward
CONFIG_A = dict(
    architecture="Tumadra", vocab=200, width=64, norm=dict(eps=1e-6, groups=2),
    loop=dict(start=0, stop=2, times=3),
    layers=[
        layer("mamba1", dict(inner=96, state=8, dt_rank=4, conv=4), 80),
        layer("attention", attention(4, 2, 16, 32, diff=0.3, q_temp=(0.5, 8)), 72),
        layer("attention", attention(2, 2, 32, 16, diff=0.7, scale=0.2), None),
        layer("mamba1", dict(inner=64, state=16, dt_rank=8, conv=2), 96),
    ])

# B: no loop, one norm group, a state count that is no power of two, a hidden width that is no multiple of 8
CONFIG_B = dict(
    architecture="Tumadra", vocab=300, width=96, norm=dict(eps=1e-5, groups=1),
    layers=[
        layer("attention", attention(3, 1, 24, 40, diff=0.5, q_temp=(0.25, 5)), 100),
        layer("mamba1", dict(inner=160, state=20, dt_rank=6, conv=3), 100),
        layer("attention", attention(6, 3, 8, 16, diff=0.2), 44),
    ])

# C: the smallest of everything: one head, one state, one tap, a loop that runs once, groups of four values, a
# temperature that moves at every position (mild: a steep one spreads the scores so far that bfloat16's
# rounding of q and k alone moves the weights by several percent, which is conditioning and no fault)
CONFIG_C = dict(
    architecture="Tumadra", vocab=64, width=32, norm=dict(eps=1e-4, groups=8),
    loop=dict(start=1, stop=2, times=1),
    layers=[
        layer("attention", attention(1, 1, 8, 8, diff=0.0, q_temp=(0.2, 1)), None),
        layer("mamba1", dict(inner=32, state=1, dt_rank=1, conv=1), 16),
    ])

# D: sizes that are no multiples of 8 (width, inner, dim, the step rank, the hidden width): under bfloat16 the
# projections over such inner sizes run in float32
CONFIG_D = dict(
    architecture="Tumadra", vocab=70, width=36, norm=dict(eps=1e-5, groups=3),
    loop=dict(start=0, stop=1, times=2),
    layers=[
        layer("mamba1", dict(inner=20, state=3, dt_rank=2, conv=2), 50),
        layer("attention", attention(2, 1, 12, 20, diff=0.25, q_temp=(0.3, 16)), 28),
    ])

CONFIGS = {"A": (CONFIG_A, 11), "B": (CONFIG_B, 12), "C": (CONFIG_C, 13), "D": (CONFIG_D, 14)}


def n_layer_runs(config):
    loop = config.get("loop")
    extra = (loop["stop"] - loop["start"]) * (loop["times"] - 1) if loop else 0
    return len(config["layers"]) + extra


def random_weights(config, seed, gain=1.0):
    g = torch.Generator().manual_seed(seed)
    E, V = config["width"], config["vocab"]
    randn = lambda *shape: torch.randn(*shape, generator=g)
    rand = lambda *shape: torch.rand(*shape, generator=g)
    matrix = lambda out, inn: randn(out, inn) * (gain / math.sqrt(inn))
    t = {"embed": randn(V, E), "final.norm": 1.0 + 0.2 * (rand(E) - 0.5), "head": randn(V, E) / math.sqrt(E)}
    for i, l in enumerate(config["layers"]):
        p, m = f"l{i}", l["mixer"]
        t[f"{p}.norm1"] = 1.0 + 0.2 * (rand(E) - 0.5)
        t[f"{p}.shift"] = rand(E)
        if l["type"] == "attention":
            H, G, D, Vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[f"{p}.mix.q"], t[f"{p}.mix.q.b"] = matrix(H * 2 * D, E) * 2.0, 0.2 * randn(H * 2 * D)
            t[f"{p}.mix.k"], t[f"{p}.mix.k.b"] = matrix(G * 2 * D, E) * 2.0, 0.2 * randn(G * 2 * D)
            t[f"{p}.mix.v"], t[f"{p}.mix.v.b"] = matrix(G * Vd, E), 0.2 * randn(G * Vd)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                t[f"{p}.mix.{name}"] = 0.3 * randn(D)
            t[f"{p}.mix.g"] = matrix(H * Vd, E)
            t[f"{p}.mix.o"] = matrix(E, H * Vd)
        else:
            C, N, R, L = m["inner"], m["state"], m["dt_rank"], m["conv"]
            t[f"{p}.mix.in"] = matrix(2 * C, E)
            t[f"{p}.mix.conv"], t[f"{p}.mix.conv.b"] = randn(C, L) / math.sqrt(L), 0.1 * randn(C)
            t[f"{p}.mix.x"] = matrix(R + 2 * N, C)
            t[f"{p}.mix.dt"] = matrix(C, R)
            t[f"{p}.mix.dt.b"] = -3.0 + 2.0 * rand(C)            # softplus: steps of 0.05 to 0.3
            t[f"{p}.mix.A_log"] = torch.log(1.0 + 7.0 * rand(C, N))
            t[f"{p}.mix.D"] = 1.0 + 0.2 * randn(C)
            t[f"{p}.mix.o"] = matrix(E, C)
        if l["mlp"] is not None:
            F = l["mlp"]["ff"]
            t[f"{p}.norm2"] = 1.0 + 0.2 * (rand(E) - 0.5)
            t[f"{p}.mlp.up"], t[f"{p}.mlp.down"] = matrix(F, E), matrix(E, F)
            t[f"{p}.mlp.act"] = torch.tensor([1.0, 0.5, -0.3, 0.1]) + 0.2 * randn(4)
    return t


def write_model(config, seed, out_dir, gain=1.0, overrides=None):
    """Writes config.json and model.safetensors (bfloat16) and returns the folder."""
    from imparo_amd.weights.safetensors_io import save_file
    tensors = random_weights(config, seed, gain)
    tensors.update(overrides or {})
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(out_dir, "model.safetensors"))
    return out_dir
