"""The Pupalorn design in the engine against the plain implementation (tests/plain_pupalorn.py): each
mechanism's kernels alone, whole prompts, stepwise decoding, portions down to two tokens, mixed batches
on a pool at the schedule's peak with slots used again, long decoding through every window, first tokens,
other sizes, keys just inside and just outside a window that one score singles out, generation through the
entry point and the trace replay program.

float32 runs are held to the plain implementation under the float32 bound everywhere. Under bfloat16 the
router reads rounded inputs, and where two choice scores lie closer than that rounding the engine may choose
another expert than the plain implementation does (no fault: the design's own statement allows the router's
input to be rounded); such a row misses the bound by far, so bfloat16 comparisons with the plain
implementation allow a few rows beyond it (`FLIPS`), and every fault of a cache, a window or a batch is
looked for in float32, where nothing is allowed."""
import json
import math
import os
import random
import subprocess

import numpy as np
import pytest
import torch

import plain_pupalorn as plain
from conftest import ROOT, prompt_tokens
from gpu_helpers import assert_picks_near_best, hand_context, make_engine, mixed_schedule, peak_pages, step_all
from tolerances import bound, check_logits
from pupalorn_models import CONFIGS, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FLIPS = 0.08      # share of rows that may miss the bfloat16 bound after a router's near-tie went the other way


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    return {name: write_model(cfg, seed, str(tmp_path_factory.mktemp(f"pupalorn_{name}")))
            for name, (cfg, seed) in CONFIGS.items()}


@pytest.fixture(scope="module")
def plains(dirs):
    return {name: plain.PlainPupalorn(d) for name, d in dirs.items()}


def layers(name):
    return len(CONFIGS[name][0]["layers"])


def vocab(name):
    return CONFIGS[name][0]["vocab"]


def check(got, ref, dtype, what, rel):
    """check_logits; under bfloat16 a share FLIPS of the rows may miss the bound."""
    if dtype == "float32":
        return check_logits(got, ref, dtype, what, rel)
    got, ref = got.float().cpu(), ref.float().cpu()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    row_err = (got - ref).abs().max(dim=-1).values / float(ref.abs().max())
    over = int((row_err > rel).sum())
    assert over <= math.ceil(FLIPS * got.shape[0]), f"{what}: {over} of {got.shape[0]} rows beyond {rel:g}"
    assert float(row_err.median()) <= rel / 2, f"{what}: the median row misses half the bound"


def dev(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def i32(a):
    return torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("width,slices,out_dtype", [(64, 1, torch.float32), (36, 3, torch.float32), (1536, 2, torch.bfloat16),
                                                    (200, 1, torch.bfloat16)])
def test_norm_behind_a_sublayer_kernel(width, slices, out_dtype):
    """x += norm(delta) * w_post, then the next norm of the sum, in one launch; with and without a row selection."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(width)
    x, delta = torch.randn(9, width, generator=g) * 2, torch.randn(slices, 9, width, generator=g) * 5
    w_post, w_next = torch.rand(width, generator=g) - 0.5, torch.rand(width, generator=g) - 0.5
    m, ls = 0.3, torch.rand(width, generator=g) + 0.5
    summed = x + m * plain.offset_norm(delta.sum(0), w_post, 1e-5) * ls
    ref = plain.offset_norm(summed, w_next, 1e-6)
    folded = (1.0 + w_post) * ls * m
    xd, out = dev(x), torch.empty(9, width, dtype=out_dtype, device=DEV)
    d = dev(delta if slices > 1 else delta[0])
    ops.post_norm_add(xd, d, dev(folded), 1e-5, dev(1.0 + w_next), 1e-6, out)
    tol = 2e-6 if out_dtype == torch.float32 else 1e-2
    assert float((xd.cpu() - summed).abs().max()) <= 2e-6 * float(summed.abs().max())
    assert float((out.float().cpu() - ref).abs().max()) <= tol * float(ref.abs().max())
    rows = [7, 0, 3]
    x2, out2 = dev(x), torch.empty(3, width, dtype=out_dtype, device=DEV)
    ops.post_norm_add(x2, d, dev(folded), 1e-5, dev(1.0 + w_next), 1e-6, out2, rows=i32(rows))
    assert torch.equal(x2.cpu(), x), "a row selection must leave the stream as it is"
    assert torch.equal(out2.cpu(), out[rows].cpu())
    x3 = dev(x)
    ops.post_norm_add(x3, d, dev(folded), 1e-5)
    assert torch.equal(x3.cpu(), xd.cpu())


def test_embedding_scale_kernel():
    from imparo_amd.kernels import ops
    table = torch.randn(50, 40).to(torch.bfloat16)
    ids = [3, 49, 0, 3]
    for t in (table, table.float()):
        out = torch.empty(4, 40, dtype=torch.float32, device=DEV)
        ops.embed_gather(dev(t, t.dtype), i32(ids), out, 0.3)
        assert torch.equal(out.cpu(), t.float()[ids] * torch.tensor(0.3, dtype=torch.float32))


@pytest.mark.parametrize("R,top", [(6, 2), (3, 1), (5, 4), (13, 5), (70, 8), (1, 1)])
def test_route_kernel(R, top):
    """Scores over all outputs, the choice by score + correction, the weights the scores as they are."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(R)
    z, corr = torch.randn(37, R, generator=g) * 2, 0.2 * torch.randn(R, generator=g)
    s = torch.softmax(z, dim=-1)
    want = torch.topk(s + corr, top, dim=-1).indices
    choice = torch.empty(37, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(37, top, dtype=torch.float32, device=DEV)
    ops.moe_route(dev(z), dev(corr), choice, weight, top)
    assert torch.equal(choice.cpu().long(), want)               # in the order of the choice, largest first
    assert float((weight.cpu() - torch.gather(s, 1, want)).abs().max()) < 1e-6
    plain_choice = torch.topk(s, top, dim=-1).indices
    if R > top:
        assert not torch.equal(plain_choice, want), "the correction changes no choice in this case"
    assert float(weight.cpu().sum(-1).max()) <= 1.0 + 1e-6 and (R == top or float(weight.cpu().sum(-1).min()) < 0.999)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,F,X,I,top", [(50, 64, 40, 4, 2, 2), (7, 96, 20, 8, 1, 3), (300, 128, 64, 16, 2, 4), (1, 36, 10, 1, 0, 1),
                                           (33, 64, 16, 2, 3, 4), (900, 64, 24, 3, 0, 1), (5, 64, 8, 0, 3, 2)])
def test_routed_experts_part(T, E, F, X, I, top, dtype):
    """The whole feed-forward part against the plain mixture, fed with rows that are bfloat16 values already."""
    from imparo_amd.config.plan import PartSpec
    from imparo_amd.parts.moe import RoutedExperts
    g = torch.Generator().manual_seed(T + E)
    bf = lambda t: t.to(torch.bfloat16).float()
    h = bf(torch.randn(T, E, generator=g))
    Wr, corr = bf(torch.randn(X + I, E, generator=g) * 1.5 / math.sqrt(E)), bf(0.1 * torch.randn(X + I, generator=g))
    ups = [bf(torch.randn(F, E, generator=g) / math.sqrt(E)) for _ in range(X)]
    downs = [bf(torch.randn(E, F, generator=g) / math.sqrt(F)) for _ in range(X)]
    ref = plain.mixture(h, Wr, corr, top, ups, downs)
    spec = PartSpec("routed_experts", "m", dict(width=E, hidden=F, experts=X, identity=I, top=top))
    tensors = {"m.router": Wr, "m.correction": corr}
    for e in range(X):
        tensors[f"m.e{e}.up"], tensors[f"m.e{e}.down"] = ups[e], downs[e]
    assert set(RoutedExperts.declare(spec)) == set(tensors)
    part = RoutedExperts(spec, tensors, torch.device(DEV), dtype)
    ctx = hand_context([(0, T)], 16, T // 16 + 2, dtype, torch.device(DEV))
    for _ in range(2):                                          # again on the same workspace: nothing is left behind
        got = part.forward(ctx, dev(h, part.in_dtype)).cpu()
        rel = 2e-6 if dtype == torch.float32 or part.in_dtype == torch.float32 else 6e-3    # the hidden is rounded to bfloat16
        assert float((got - ref).abs().max()) <= rel * float(ref.abs().max()), (T, E, F, X, I, top)
    # the weighted sum left to the launch of the norm behind the part: the same bits as sum, then norm
    from imparo_amd.kernels import ops
    g2 = torch.Generator().manual_seed(1)
    x, w_post, w_next = torch.randn(T, E, generator=g2), torch.rand(E, generator=g2) + 0.5, torch.rand(E, generator=g2) + 0.5
    x1, out1 = dev(x), torch.empty(T, E, dtype=torch.float32, device=DEV)
    ops.post_norm_add(x1, part.forward(ctx, dev(h, part.in_dtype)), dev(w_post), 1e-5, dev(w_next), 1e-6, out1)
    x2, out2 = dev(x), torch.empty(T, E, dtype=torch.float32, device=DEV)
    ops.post_norm_add(x2, part.forward_rows(ctx, dev(h, part.in_dtype)), dev(w_post), 1e-5, dev(w_next), 1e-6, out2)
    assert torch.equal(x1.cpu(), x2.cpu()) and torch.equal(out1.cpu(), out2.cpu())
    rows = i32([T - 1, 0])
    out3 = torch.empty(2, E, dtype=torch.float32, device=DEV)
    x3 = dev(x)
    ops.post_norm_add(x3, part.forward_rows(ctx, dev(h, part.in_dtype)), dev(w_post), 1e-5, dev(w_next), 1e-6, out3, rows=rows)
    assert torch.equal(x3.cpu(), x) and torch.equal(out3.cpu(), out1.cpu()[[T - 1, 0]])


def attention_case(H, G, D, V, segments, page, dtype, window, boost=None, seed=0, kernel="wave"):
    """q, k, v for rows given as (start, tokens) whose earlier positions are in the cache; pages in a shuffled
    order. -> (kernel output [tokens, H * V], plain output). `boost` (row, key position): that key is made to
    match the row's last query, so that it takes most of the weight if it is seen at all."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(seed + D + V)
    bf = (lambda t: t.to(torch.bfloat16).float()) if dtype == torch.bfloat16 else (lambda t: t)
    scale = 1.0 / math.sqrt(D)
    n_pages = sum((p0 + n + page - 1) // page for p0, n in segments) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    kc = torch.zeros(n_pages, G, page, D)
    vc = torch.full((n_pages, G, page, V), 1e4)                 # what a stale page holds must never be seen
    q_all, ref_all, tables = [], [], []
    for r, (p0, n) in enumerate(segments):
        L = p0 + n
        q, k, v = bf(torch.randn(L, H, D, generator=g)), bf(torch.randn(L, G, D, generator=g)), bf(torch.randn(L, G, V, generator=g))
        if boost is not None and boost[0] == r:
            k[boost[1]] = bf(q[L - 1, ::H // G] * 3.0)
        ref_all.append(plain.windowed_attention(q, k, v, torch.arange(L), scale, window)[p0:])
        q_all.append(q[p0:])
        pages = [order.pop() for _ in range((L + page - 1) // page)]
        tables.append(pages)
        for p in range(L):
            kc[pages[p // page], :, p % page] = k[p]
            vc[pages[p // page], :, p % page] = v[p]
    ctx = hand_context(segments, page, n_pages, dtype, torch.device(DEV), tables=tables)
    q = dev(torch.cat(q_all), dtype)
    out = torch.empty(q.shape[0], H * V, dtype=dtype, device=DEV)
    if kernel == "wave":
        ops.attention(q, dev(kc, dtype), dev(vc, dtype), out, ctx.positions, ctx.row_of_token, ctx.block_tables[0], scale, window)
        return out.float().cpu(), torch.cat(ref_all)
    # the matrix-core kernels with exact weights: V transposed inside a page, single tokens and portions apart
    assert D == V and dtype == torch.bfloat16
    kd, vd = dev(kc, dtype), dev(vc.permute(0, 1, 3, 2), dtype)
    if ctx.n_single_rows:
        splits = (ctx.max_context + ops.decode_split() - 1) // ops.decode_split()
        part_o = torch.zeros(ctx.n_single_rows * H * splits * D, device=DEV)
        part_ml = torch.zeros(ctx.n_single_rows * H * splits * 2, device=DEV)
        ops.attention_decode(q, kd, vd, out, part_o, part_ml, ctx.single_rows, ctx.n_single_rows, ctx.seg_start,
                             ctx.positions, ctx.block_tables[0], scale, window, ctx.max_context, exact=True)
    if ctx.n_portion_rows:
        tiles = sum((n + 63) // 64 for n in ctx.host_seg_len if n > 1)
        ops.attention_prefill(q, kd, vd, out, ctx.portion_rows, ctx.n_portion_rows, tiles, ctx.seg_start, ctx.seg_len,
                              ctx.positions, ctx.block_tables[0], scale, window, exact=True)
    return out.float().cpu(), torch.cat(ref_all)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V,page,window", [(4, 2, 16, 32, 16, 24), (2, 2, 32, 16, 8, None), (3, 1, 24, 40, 64, 33),
                                                 (2, 1, 12, 20, 16, 5), (4, 1, 64, 128, 32, 1), (5, 5, 128, 128, 64, 90)])
def test_attention_kernel_with_values_of_their_own_size(H, G, D, V, page, window, dtype):
    """A portion behind cached keys beside single tokens and a fresh prompt, pages in a shuffled order."""
    got, ref = attention_case(H, G, D, V, [(150, 37), (299, 1), (0, 70), (63, 1), (0, 1)], page, dtype, window)
    rel = 2e-6 if dtype == torch.float32 else 1e-2
    assert float((got - ref).abs().max()) <= rel * float(ref.abs().max())


@pytest.mark.parametrize("D", [16, 64, 80, 128])
@pytest.mark.parametrize("n_last", [1, 5, 70])
@pytest.mark.parametrize("window,page", [(24, 16), (64, 64), (65, 64), (2, 32), (1, 16), (300, 64)])
def test_a_key_at_the_windows_edge_on_the_matrix_cores(window, page, n_last, D):
    """The same two cases through the matrix-core kernels with exact weights (decode and both prompt kernels)."""
    L = 5 * 64 + 7
    for key, seen in ((L - window, True), (L - window - 1, False)):
        got, ref = attention_case(4, 2, D, D, [(L - n_last, n_last), (40, 1)], page, torch.bfloat16, window, boost=(0, key),
                                  seed=key, kernel="mfma")
        assert float((got - ref).abs().max()) <= 1e-2 * float(ref.abs().max()), (key, seen)
        other, _ = attention_case(4, 2, D, D, [(L - n_last, n_last), (40, 1)], page, torch.bfloat16, window + (-1 if seen else 1),
                                  boost=(0, key), seed=key, kernel="mfma")
        assert float((other[n_last - 1] - ref[n_last - 1]).abs().max()) > 0.2 * float(ref[n_last - 1].abs().max()), (key, seen)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_last", [1, 5])
@pytest.mark.parametrize("window,page", [(24, 16), (64, 64), (65, 64), (9, 8), (1, 16)])
def test_a_key_at_the_windows_edge(window, page, n_last, dtype):
    """The oldest key a query may see carries most of its weight; the key one further back must carry none.
    The query is the last of a portion (n_last 5) or a single decoded token (n_last 1)."""
    L = 3 * 64 + 7
    for key, seen in ((L - window, True), (L - window - 1, False)):
        got, ref = attention_case(2, 1, 16, 24, [(L - n_last, n_last)], page, dtype, window, boost=(0, key), seed=key)
        rel = 2e-6 if dtype == torch.float32 else 1e-2
        assert float((got - ref).abs().max()) <= rel * float(ref.abs().max()), (key, seen)
        # the case shows the fault it is made for: without the boosted key (or with it) the row would differ by far
        other, _ = attention_case(2, 1, 16, 24, [(L - n_last, n_last)], page, dtype, window + (-1 if seen else 1),
                                  boost=(0, key), seed=key)
        assert float((other[-1] - ref[-1]).abs().max()) > 0.2 * float(ref[-1].abs().max()), (key, seen)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds(dtype):
    got, ref = attention_case(4, 2, 32, 16, [(899, 1), (880, 20)], 16, dtype, None, boost=(0, 3))
    assert float((got - ref).abs().max()) <= (2e-6 if dtype == torch.float32 else 1e-2) * float(ref.abs().max())
    got, ref = attention_case(4, 2, 32, 16, [(899, 1), (880, 20)], 16, dtype, None, boost=(1, 17))
    assert float((got - ref).abs().max()) <= (2e-6 if dtype == torch.float32 else 1e-2) * float(ref.abs().max())


@pytest.mark.parametrize("D", [64, 128, 48])
@pytest.mark.parametrize("n_last", [1, 40])
def test_matrix_core_attention_keeps_its_weights_exact(D, n_last):
    """Keys in pairs that score nearly alike and carry opposite values: the result is the small difference of
    two weights, which their rounding to bfloat16 would drown. The matrix-core kernels' exact form must carry
    it; their plain form, which rounds the weights, must miss it by far (so the case can fail)."""
    from imparo_amd.kernels import ops
    H, G, page, L, window = 4, 2, 64, 452, 300
    g = torch.Generator().manual_seed(D + n_last)
    bf = lambda t: t.to(torch.bfloat16).float()
    q, k, v = bf(torch.randn(L, H, D, generator=g)), bf(torch.randn(L, G, D, generator=g)), bf(torch.randn(L, G, D, generator=g))
    k[1::2] = k[0::2]
    k[1::2, :, 0] = bf(k[0::2, :, 0] * (1.0 + 2.0 ** -7))
    v[1::2] = -v[0::2]
    scale = 1.0 / math.sqrt(D)
    ref = plain.windowed_attention(q.double(), k.double(), v.double(), torch.arange(L), scale, window)[L - n_last:].float()
    n_pages = L // page + 2
    tables = [list(range(n_pages - 1, n_pages - 1 - (L + page - 1) // page, -1))]
    ctx = hand_context([(L - n_last, n_last)], page, n_pages, torch.bfloat16, torch.device(DEV), tables=tables)
    kc = torch.zeros(n_pages, G, page, D)
    vc = torch.zeros(n_pages, G, D, page)
    for p_ in range(L):
        kc[tables[0][p_ // page], :, p_ % page] = k[p_]
        vc[tables[0][p_ // page], :, :, p_ % page] = v[p_]
    kc, vc, qd = dev(kc, torch.bfloat16), dev(vc, torch.bfloat16), dev(q[L - n_last:], torch.bfloat16)
    errs = {}
    for exact in (True, False):
        out = torch.zeros(n_last, H * D, dtype=torch.bfloat16, device=DEV)
        if n_last == 1:
            splits = (L + ops.decode_split() - 1) // ops.decode_split()
            part_o = torch.zeros(H * splits * D, device=DEV)
            part_ml = torch.zeros(H * splits * 2, device=DEV)
            ops.attention_decode(qd, kc, vc, out, part_o, part_ml, ctx.single_rows, 1, ctx.seg_start, ctx.positions,
                                 ctx.block_tables[0], scale, window, L, exact=exact)
        else:
            ops.attention_prefill(qd, kc, vc, out, ctx.portion_rows, 1, (n_last + 63) // 64, ctx.seg_start, ctx.seg_len,
                                  ctx.positions, ctx.block_tables[0], scale, window, exact=exact)
        # the queries at odd positions see whole pairs only (an even window, an even first position)
        sel = [i for i in range(n_last) if (L - n_last + i) % 2 == 1]
        errs[exact] = float((out.float().cpu()[sel] - ref[sel]).abs().max()) / float(ref[sel].abs().max())
    assert errs[True] <= 2e-2, errs
    assert errs[False] > 4 * errs[True], f"rounded weights do not show in this case: {errs}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V,rot,n", [(4, 2, 16, 32, 8, 5), (2, 1, 12, 20, 4, 130), (3, 3, 24, 40, 0, 7), (4, 2, 64, 64, 32, 200),
                                           (2, 2, 32, 16, 32, 100)])
def test_head_norm_rotation_and_cache_write(H, G, D, V, rot, n, dtype):
    """Rows of [queries | keys | values of another size] and rows of queries only, at far positions."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(D * n)
    page, p0 = 16, 70000
    freq = plain.inverse_frequencies(rot, 10000.0, dict(factor=8.0, low=1.0, high=4.0, original=64)).float() if rot else torch.zeros(0)
    pos = torch.arange(p0, p0 + n)
    row = torch.randn(n, (H + G) * D + G * V, generator=g)
    wq, wk = torch.rand(D, generator=g) + 0.5, torch.rand(D, generator=g) + 0.5
    # angles are float32 products (position x frequency), as the design has them
    q_ref = plain.rotate(plain.rms(row[:, :H * D].reshape(n, H, D), 1e-5) * wq, pos, freq)
    k_ref = plain.rotate(plain.rms(row[:, H * D:(H + G) * D].reshape(n, G, D), 1e-5) * wk, pos, freq)
    v_ref = row[:, (H + G) * D:].reshape(n, G, V)
    n_pages = (p0 + n) // page + 1
    ctx = hand_context([(p0, n)], page, n_pages, dtype, torch.device(DEV), tables=[list(range(n_pages))])
    kc = torch.zeros(n_pages, G, page, D, dtype=dtype, device=DEV)
    vc = torch.zeros(n_pages, G, page, V, dtype=dtype, device=DEV)
    q = torch.empty(n, H, D, dtype=dtype, device=DEV)
    f = dev(freq) if rot else None
    ops.qk_norm_rope_store(dev(row), dev(wq), dev(wk), 1e-5, f, ctx.positions, ctx.row_of_token, ctx.block_tables[0], page,
                           q, kc, vc, H, G, D, value_dim=V)
    rel = 3e-6 if dtype == torch.float32 else 6e-3
    flat = lambda c: c.float().cpu().permute(0, 2, 1, 3).reshape(n_pages * page, G, -1)[p0:p0 + n]
    for got, ref in ((q.float().cpu(), q_ref), (flat(kc), k_ref), (flat(vc), v_ref)):
        assert float((got - ref.float()).abs().max()) <= rel * float(ref.abs().max())
    q2 = torch.empty(n, H, D, dtype=dtype, device=DEV)
    ops.qk_norm_rope_store(dev(row[:, :H * D]), dev(wq), dev(wq), 1e-5, f, ctx.positions, ctx.row_of_token, None, page,
                           q2, None, None, H, 0, D, value_dim=V)
    assert torch.equal(q2.cpu(), q.cpu()), "queries alone must come out as they do beside keys and values"


# ------------------------------------------------------------------ the model
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_whole_prompt_and_stepwise(dirs, plains, name, dtype):
    """A prompt whole; then most of it whole and its last 50 tokens one by one (captured steps)."""
    from imparo_amd.engine import StepEntry
    tokens = prompt_tokens(vocab(name), 170, 7)
    ref = plains[name].logits(tokens)
    rel = bound(dtype, layers(name))
    eng = make_engine(dirs[name], dtype)
    whole = eng.step([StepEntry("w", tokens, list(range(170)))]).cpu()
    eng.release("w")
    check(whole, ref, dtype, f"{name} whole", rel)
    head = eng.step([StepEntry("d", tokens[:120], list(range(120)))]).cpu()
    tail = [eng.step([StepEntry("d", [t], [0])]).cpu() for t in tokens[120:]]
    eng.release("d")
    stepwise = torch.cat([head] + tail)
    check(stepwise, ref, dtype, f"{name} stepwise", rel)
    if dtype == "float32":
        check_logits(stepwise, whole, dtype, f"{name} stepwise against whole", 2e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 16), ("B", 8), ("C", 16), ("D", 64), ("E", 32)])
def test_portions_of_changing_size(dirs, plains, name, page, dtype):
    """Portions down to two tokens, cut inside pages and windows, also without captured steps."""
    tokens = prompt_tokens(vocab(name), 160, 8)
    ref = plains[name].logits(tokens)
    for cuts, graphs in (((2, 3, 17, 2, 1, 31, 1, 1, 5), True), ((64, 2, 9), False), ((1,), True)):
        eng = make_engine(dirs[name], dtype, page_size=page, use_graphs=graphs)
        got = step_all(eng, "p", tokens if cuts != (1,) else tokens[:45], cuts)
        check(got, ref[:got.shape[0]], dtype, f"{name} cuts {cuts}", bound(dtype, layers(name)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_mixed_batches_on_a_full_pool(dirs, plains, name, dtype):
    """Six unequal requests, at most four live, portions beside single tokens, on a pool of exactly the
    schedule's peak and four slots: pages are used again. Each request's logits are those it has alone."""
    from imparo_amd.engine import StepEntry
    rng = random.Random(5)
    lengths = [70, 33, 1, 90, 2, 51]
    prompts = [prompt_tokens(vocab(name), n, 20 + i) for i, n in enumerate(lengths)]
    steps = mixed_schedule(rng, lengths, max_live=4)
    page = 8
    # no window gives pages back early here: the pool is sized as if every position stayed
    eng = make_engine(dirs[name], dtype, page_size=page, max_tokens=peak_pages(steps, page) * page, max_requests=4)
    got = {i: [] for i in range(len(lengths))}
    for entries, ends in steps:
        out = eng.step([StepEntry(rid, prompts[rid][lo:hi], list(range(hi - lo))) for rid, lo, hi in entries]).cpu()
        at = 0
        for rid, lo, hi in entries:
            got[rid].append(out[at:at + hi - lo])
            at += hi - lo
        for rid in ends:
            eng.release(rid)
    for i, p in enumerate(prompts):
        check(torch.cat(got[i]), plains[name].logits(p), dtype, f"{name} request {i}", bound(dtype, layers(name)))
    eng.cache.check()
    assert eng.free_pages() == [g.pool.n_pages for g in eng.cache.groups]


def test_long_decoding_and_first_tokens(dirs, plains):
    """One prompt token, then 330 single-token steps: every window passes over decoded tokens many times and
    the cache gives back the pages behind it; and requests of one and of two tokens alone."""
    from imparo_amd.engine import StepEntry
    tokens = prompt_tokens(vocab("A"), 331, 3)
    ref = plains["A"].logits(tokens)
    for dtype in ("float32", "bfloat16"):
        eng = make_engine(dirs["A"], dtype, page_size=8)
        got = torch.cat([eng.step([StepEntry("r", [t], [0])]).cpu() for t in tokens])
        check(got, ref, dtype, "long decoding", bound(dtype, layers("A")))
        eng.release("r")
        two = eng.step([StepEntry("x", tokens[:1], [0]), StepEntry("y", tokens[:2], [0, 1])]).cpu()
        check_logits(two, torch.cat([ref[:1], ref[:2]]), dtype, "first tokens", bound(dtype, layers("A")))


def test_layer_scale_and_multiplier_matter(dirs, plains, tmp_path):
    """Values that a model may happen to make 1: with other layer scales the logits move, and by what the plain
    implementation says."""
    from imparo_amd.engine import StepEntry
    cfg, seed = CONFIGS["B"]          # no multiplier and no embedding scale in the file: both 1
    tokens = prompt_tokens(cfg["vocab"], 40, 4)
    eng = make_engine(dirs["B"], "float32")
    base = eng.step([StepEntry("a", tokens, list(range(40)))]).cpu()
    other = dict(cfg, residual_mult=0.25, embedding=dict(scale=3.0))
    d = write_model(other, seed, str(tmp_path / "other"))
    got = make_engine(d, "float32").step([StepEntry("a", tokens, list(range(40)))]).cpu()
    check_logits(got, plain.PlainPupalorn(d).logits(tokens), "float32", "other constants")
    assert float((got - base).abs().max()) > 0.05 * float(base.abs().max())


def test_generation_through_the_entry_point(dirs, plains):
    from imparo_amd import generate
    prompts = [prompt_tokens(vocab("A"), n, 50 + n) for n in (1, 6, 29, 13, 40)]
    want = [plains["A"].greedy(p, 12) for p in prompts]
    assert all(len(set(w)) > 4 for w in want), f"the plain continuation hardly moves: {want}"
    assert generate(dirs["A"], prompts, max_tokens=12, dtype="float32", page_size=8) == want
    # three at a time under a small token budget: prompts in portions beside decoding rows
    os.environ["IMPARO_BATCH"] = "5"
    try:
        got = generate(dirs["A"], prompts, max_tokens=12, dtype="float32", page_size=8, parallel=3, max_batch_tokens=11)
    finally:
        del os.environ["IMPARO_BATCH"]
    assert got == want
    got16 = generate(dirs["A"], prompts, max_tokens=12, dtype="bfloat16", parallel=3)
    assert all(len(out) == 12 for out in got16)


def test_trace_replay_program(dirs, plains, tmp_path):
    tokens = prompt_tokens(vocab("B"), 45, 1)
    other = prompt_tokens(vocab("B"), 9, 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": tokens[:20], "want": [0, 19]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": tokens[20:44], "want": []},
                                {"id": "b", "tokens": other, "want": [8]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": tokens[44:], "want": [0]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", dirs["B"], "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    V = vocab("B")
    ref, ref_other = plains["B"].logits(tokens), plains["B"].logits(other)
    read = lambda n: torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, V))
    check_logits(read(0), ref[[0, 19]], "float32", "step 0")
    check_logits(read(1), ref_other[[8]], "float32", "step 1")
    check_logits(read(2), ref[[44]], "float32", "step 2")
