"""Pupalorn configurations drawn at random with fixed seeds (sizes, head counts, key and value sizes, rotated
dimensions, frequency scaling, windows, which layers read whose keys, layers without feed-forward, experts of
both kinds, constants), each stepped through a random mixed schedule on a pool at the schedule's peak against
the plain implementation. float32 runs the model as drawn, under the float32 bound. bfloat16 runs the same
model with a router that cannot be moved by rounding (a zero router matrix and a correction that sets the
experts well apart: every token chooses the same experts, all scores are equal) and a residual multiplier
of at most one half, under the plain bfloat16 bound with no row excepted: with the drawn router a near-tie between two choice scores may go the other way
under bfloat16's rounding of the router's input, which is no fault and would have to be excepted."""
import math
import random

import pytest
import torch

import plain_pupalorn as plain
from conftest import prompt_tokens
from gpu_helpers import make_engine, mixed_schedule, peak_pages
from pupalorn_models import attention, layer, moe, write_model
from pupalorn_models import random_weights
from tolerances import bound, check_logits

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = random.Random(seed)
    width = rng.choice([32, 48, 64, 96, 128, 160, 256])
    n_layers = rng.randint(1, 5)
    shapes = {}
    layers = []
    for i in range(n_layers):
        src = None
        owners = [j for j in range(i) if layers[j]["mixer"].get("kv_from") is None]
        if owners and rng.random() < 0.45:
            src = rng.choice(owners)
        if src is None:
            kv = rng.choice([1, 2, 3, 4])
            heads = kv * rng.choice([1, 1, 2, 3])
            dim = rng.choice([8, 16, 32, 64, 128]) if rng.random() < 0.8 else rng.choice([24, 40, 80])
            vdim = dim if rng.random() < 0.5 else rng.choice([4, 8, 12, 16, 20, 32, 64])
            rot = None
            if rng.random() < 0.85:
                dims = rng.choice([dim, dim // 2, dim // 4 * 2]) or 2
                rot = (dims - dims % 2, rng.choice([100.0, 10000.0, 1e6]))
            scaling = None
            if rot is not None and rot[0] > 0 and rng.random() < 0.6:
                scaling = (rng.choice([2.0, 8.0, 32.0]), 1.0, rng.choice([2.0, 4.0]), rng.choice([16, 64, 512]))
            shapes[i] = (heads, kv, dim, vdim, rot, scaling)
        heads, kv, dim, vdim, rot, scaling = shapes[i if src is None else src]
        if rot is not None and rot[0] == 0:
            rot = None
        window = None if rng.random() < 0.25 else rng.choice([1, 2, 7, 16, 33, 64, 100])
        mixer = attention(heads, kv, dim, vdim, window=window, rot=rot, scaling=scaling, kv_from=src,
                          # mild scores: the test models' head norms make |q||k| about 3 dim, and scores spread much
                          # wider than that turn bfloat16's rounding of q and k into weight shifts of several percent
                          # whichever kernel runs (the wave kernel and the matrix-core kernels miss alike then):
                          # conditioning, no fault
                          scale=rng.choice([1.0, 0.5, 1.0 / 3.0]) / math.sqrt(dim))
        mlp = None
        if rng.random() < 0.85:
            experts, identity = rng.choice([1, 2, 3, 8, 12]), rng.choice([0, 0, 1, 4])
            mlp = moe(rng.choice([8, 20, 32, 64]), experts, identity, rng.randint(1, min(4, experts + identity)))
        layers.append(layer(mixer, mlp))
    cfg = dict(architecture="Pupalorn", vocab=rng.choice([50, 97, 300, 500]), width=width,
               norm=dict(eps=rng.choice([1e-6, 1e-5, 1e-3])), layers=layers)
    if rng.random() < 0.7:
        cfg["residual_mult"] = rng.choice([0.25, 0.5, 1.5])
    if rng.random() < 0.7:
        cfg["embedding"] = dict(scale=rng.choice([0.5, 1.0, 3.0]))
    return cfg


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration_through_a_mixed_schedule(seed, tmp_path):
    from imparo_amd.engine import StepEntry
    cfg = draw_config(1000 + seed)
    dirs = {"float32": write_model(cfg, seed, str(tmp_path / "m"))}
    steady = {}
    for name, t in random_weights(cfg, seed).items():
        if name.endswith(".mlp.router"):
            steady[name] = torch.zeros_like(t)
            steady[name[:-len("router")] + "correction"] = 0.25 * torch.randperm(t.shape[0], generator=torch.Generator().manual_seed(seed)).float()
    # ... and with a multiplier of at most one half: every sublayer's result is normed to the stream's own size
    # before it is added, so with a multiplier of 1 or more each of the 2 x layers sublayers brings its own
    # bfloat16 rounding (half a percent of itself) into the stream undiminished, which the budget of
    # tolerances.py, stated for models whose layers add little to the stream, does not cover
    cfg16 = dict(cfg, residual_mult=min(cfg.get("residual_mult", 1.0), 0.5))
    dirs["bfloat16"] = write_model(cfg16, seed, str(tmp_path / "steady"), overrides=steady)
    rng = random.Random(seed)
    lengths = [rng.choice([1, 2, 5, 30, 70, 130]) for _ in range(5)]
    prompts = [prompt_tokens(cfg["vocab"], n, 40 + i) for i, n in enumerate(lengths)]
    steps = mixed_schedule(rng, lengths, max_live=4)
    page = rng.choice([8, 16, 64])
    for dtype in ("float32", "bfloat16"):
        d = dirs[dtype]
        ref = plain.PlainPupalorn(d)
        eng = make_engine(d, dtype, page_size=page, max_tokens=peak_pages(steps, page) * page, max_requests=4)
        got = {i: [] for i in range(len(lengths))}
        for entries, ends in steps:
            out = eng.step([StepEntry(rid, prompts[rid][lo:hi], list(range(hi - lo))) for rid, lo, hi in entries]).cpu()
            at = 0
            for rid, lo, hi in entries:
                got[rid].append(out[at:at + hi - lo])
                at += hi - lo
            for rid in ends:
                eng.release(rid)
        all_got = torch.cat([torch.cat(got[i]) for i in range(len(lengths))])
        all_ref = torch.cat([ref.logits(p) for p in prompts])
        check_logits(all_got, all_ref, dtype, f"seed {seed} {dtype}: {cfg}", bound(dtype, len(cfg["layers"])))
        eng.cache.check()
