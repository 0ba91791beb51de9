"""Small Pupalorn configurations with random weights, for tests. The weights are drawn so that every
mechanism matters: projections of unit gain, norm weights kept as their distance from one, layer scales of order one,
a router whose scores spread and a correction large enough to change some choices."""
import json
import math
import os

import torch


def attention(heads, kv_heads, dim, vdim, window=None, rot=None, scaling=None, kv_from=None, scale=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else 1.0 / math.sqrt(dim))
    if window is not None:
        m["mask"] = dict(size=window)
    if rot is not None:
        m["rot"] = dict(dims=rot[0], base=rot[1])
        if scaling is not None:
            m["rot"]["scaling"] = dict(factor=scaling[0], low=scaling[1], high=scaling[2], original=scaling[3])
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(ff, experts, identity, top):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, identity=identity, top=top))


def layer(mixer, mlp):
    return dict(type="attention", mixer=mixer, mlp=mlp)


_ROT_A = ((8, 10000.0), (4.0, 1.0, 4.0, 200))
# A: values wider and narrower than keys, two layers that read earlier layers' keys (one with a wider window than
# the layer it reads from), a layer without feed-forward, a layer without window, one chosen expert, more
# pass-through experts than real ones
CONFIG_A = dict(
    architecture="Pupalorn", vocab=200, width=64, norm=dict(eps=1e-6), residual_mult=0.5, embedding=dict(scale=1.7),
    layers=[
        layer(attention(4, 2, 16, 32, window=24, rot=_ROT_A[0], scaling=_ROT_A[1]), moe(40, 4, 2, 2)),
        layer(attention(2, 2, 32, 16, rot=(32, 500.0)), None),
        layer(attention(4, 2, 16, 32, window=40, rot=_ROT_A[0], scaling=_ROT_A[1], kv_from=0), moe(24, 3, 0, 1)),
        layer(attention(2, 2, 32, 16, window=9, rot=(32, 500.0), kv_from=1), moe(16, 2, 3, 4)),
    ])

# B: keys and values of one size, a frequency scaling whose blended band is hit, a window of one (a token sees
# itself only), no rotation in one layer, a hidden width that is no multiple of 8, no multiplier, no embedding scale
CONFIG_B = dict(
    architecture="Pupalorn", vocab=300, width=96, norm=dict(eps=1e-5),
    layers=[
        layer(attention(6, 3, 16, 16, window=33, rot=(16, 100.0), scaling=(4.0, 1.0, 8.0, 64)), moe(20, 8, 1, 3)),
        layer(attention(3, 1, 24, 40, window=1), moe(44, 5, 0, 2)),
        layer(attention(6, 3, 16, 16, window=33, rot=(16, 100.0), scaling=(4.0, 1.0, 8.0, 64), kv_from=0), None),
    ])

# C: sizes that are no multiples of 8 (width, key size), one expert, one head group
CONFIG_C = dict(
    architecture="Pupalorn", vocab=70, width=36, norm=dict(eps=1e-4), residual_mult=1.3, embedding=dict(scale=0.25),
    layers=[
        layer(attention(2, 1, 12, 20, window=5, rot=(4, 50.0)), moe(10, 1, 0, 1)),
        layer(attention(2, 1, 12, 20, window=70, rot=(4, 50.0), kv_from=0), moe(12, 2, 2, 2)),
    ])

# E: heads x value size no multiple of 8 under a width that is one (the attention rows end in zeros, the output
# projection in columns of zero weight)
CONFIG_E = dict(
    architecture="Pupalorn", vocab=90, width=48, norm=dict(eps=1e-5), residual_mult=0.4,
    layers=[
        layer(attention(3, 1, 16, 20, window=11, rot=(8, 100.0)), moe(16, 2, 1, 2)),
        layer(attention(3, 3, 8, 4, rot=(8, 100.0)), None),
        layer(attention(3, 1, 16, 20, window=30, rot=(8, 100.0), kv_from=0), moe(8, 3, 0, 1)),
    ])

# D: heads of 64 rotated in half, sixteen experts of which four are used, a long window
CONFIG_D = dict(
    architecture="Pupalorn", vocab=500, width=128, norm=dict(eps=1e-5), residual_mult=0.7, embedding=dict(scale=2.0),
    layers=[
        layer(attention(4, 2, 64, 64, window=100, rot=(32, 10000.0)), moe(64, 16, 2, 4)),
        layer(attention(4, 2, 64, 64, window=130, rot=(32, 10000.0), kv_from=0), moe(64, 16, 2, 4)),
        layer(attention(2, 1, 128, 128, rot=(128, 10000.0), scaling=(8.0, 1.0, 4.0, 256)), moe(32, 6, 0, 2)),
    ])

CONFIGS = {"A": (CONFIG_A, 21), "B": (CONFIG_B, 22), "C": (CONFIG_C, 23), "D": (CONFIG_D, 24), "E": (CONFIG_E, 25)}


def random_weights(config, seed, gain=1.0):
    g = torch.Generator().manual_seed(seed)
    E, V = config["width"], config["vocab"]
    randn = lambda *shape: torch.randn(*shape, generator=g)
    rand = lambda *shape: torch.rand(*shape, generator=g)
    matrix = lambda out, inn: randn(out, inn) * (gain / math.sqrt(inn))
    around_zero = lambda n: 0.4 * (rand(n) - 0.5)
    t = {"embed": randn(V, E), "final.norm": around_zero(E), "head": randn(V, E) / math.sqrt(E)}
    for i, l in enumerate(config["layers"]):
        p, m = f"l{i}", l["mixer"]
        H, G, D, Vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t[f"{p}.norm1"], t[f"{p}.norm1b"], t[f"{p}.ls1"] = around_zero(E), around_zero(E), 0.5 + rand(E)
        t[f"{p}.mix.q"], t[f"{p}.mix.q.norm"] = matrix(H * D, E), 1.5 + 0.5 * rand(D)
        if m.get("kv_from") is None:
            t[f"{p}.mix.k"], t[f"{p}.mix.k.norm"] = matrix(G * D, E), 1.5 + 0.5 * rand(D)
            t[f"{p}.mix.v"] = matrix(G * Vd, E)
        t[f"{p}.mix.o"] = matrix(E, H * Vd)
        if l["mlp"] is not None:
            F, r = l["mlp"]["expert"]["ff"], l["mlp"]["router"]
            R = r["experts"] + r.get("identity", 0)
            t[f"{p}.norm2"], t[f"{p}.norm2b"], t[f"{p}.ls2"] = around_zero(E), around_zero(E), 0.5 + rand(E)
            t[f"{p}.mlp.router"], t[f"{p}.mlp.correction"] = matrix(R, E) * 1.5, 0.1 * randn(R)
            for e in range(r["experts"]):
                t[f"{p}.mlp.e{e}.up"], t[f"{p}.mlp.e{e}.down"] = matrix(F, E), matrix(E, F)
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
