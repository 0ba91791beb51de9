"""The Tumadra design in the engine against the plain implementation (tests/plain_tumadra.py): each
mechanism's kernels alone, whole prompts, stepwise decoding, portions down to two tokens, mixed batches
on a pool at the schedule's peak with slots used again, long decoding, first tokens, other sizes, a far
key that one score singles out, generation through the entry point and the trace replay program."""
import json
import math
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_tumadra as plain
from conftest import ROOT, prompt_tokens
from gpu_helpers import assert_picks_near_best, make_engine, mixed_schedule, peak_pages, step_all
from tolerances import BF16_REL, bound, check_logits
from tumadra_models import CONFIGS, n_layer_runs, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    return {name: write_model(cfg, seed, str(tmp_path_factory.mktemp(f"tumadra_{name}")))
            for name, (cfg, seed) in CONFIGS.items()}


@pytest.fixture(scope="module")
def plains(dirs):
    return {name: plain.PlainTumadra(d) for name, d in dirs.items()}


def runs(name):
    return n_layer_runs(CONFIGS[name][0])


def vocab(name):
    return CONFIGS[name][0]["vocab"]


# ------------------------------------------------------------------ mechanisms alone
def dev(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def i32(a):
    return torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)


@pytest.mark.parametrize("width,groups", [(64, 2), (96, 1), (32, 8), (1536, 4), (200, 5)])
def test_group_norm_kernel(width, groups):
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(width)
    x, w = torch.randn(7, width, generator=g) * 3, torch.rand(width, generator=g) + 0.5
    delta = torch.randn(3, 7, width, generator=g)
    ref = plain.group_norm(x, w, groups, 1e-5)
    out = torch.empty(7, width, device=DEV)
    ops.group_rms_norm(dev(x), dev(w), groups, 1e-5, out)
    assert torch.allclose(out.cpu(), ref, atol=2e-6, rtol=2e-6)
    # slices of a delta are added first and written back; rows select
    xd = dev(x)
    ops.group_rms_norm(xd, dev(w), groups, 1e-5, out, delta=dev(delta), write_back=True)
    summed = x + delta.sum(0)
    assert torch.allclose(xd.cpu(), summed, atol=1e-5)
    assert torch.allclose(out.cpu(), plain.group_norm(summed, w, groups, 1e-5), atol=3e-6, rtol=3e-6)
    rows = [5, 0, 5]
    picked = torch.empty(3, width, device=DEV, dtype=torch.bfloat16)
    ops.group_rms_norm(dev(x), dev(w), groups, 1e-5, picked, delta=dev(delta[0]), rows=i32(rows))
    want = plain.group_norm((x + delta[0])[rows], w, groups, 1e-5)
    assert torch.allclose(picked.float().cpu(), want, atol=2e-2, rtol=1e-2)


def test_token_shift_kernels_carry_the_last_row():
    """Segments of 1, 2 and 5 tokens in slots used before: the first token of each reads what the slot
    holds, the slot then holds the segment's last unshifted row; the norm's fused form does the same."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    width = 48
    h, mix = torch.randn(8, width, generator=g), torch.rand(width, generator=g)
    state = torch.randn(4, width, generator=g)
    seg_start, seg_len, slots = [0, 1, 3], [1, 2, 5], [2, 0, 3]
    row = [0, 1, 1, 2, 2, 2, 2, 2]
    st = dev(state)
    out = torch.empty(8, width, device=DEV)
    ops.token_shift(dev(h), dev(mix), st, i32(row), i32(seg_start), i32(seg_len), i32(slots), out)
    for r in range(3):
        seq = torch.cat([state[slots[r]][None], h[seg_start[r]:seg_start[r] + seg_len[r]]])
        want = plain.token_shift(seq, mix)[1:]
        assert torch.allclose(out[seg_start[r]:seg_start[r] + seg_len[r]].cpu(), want, atol=1e-6)
        assert torch.equal(st[slots[r]].cpu(), h[seg_start[r] + seg_len[r] - 1])
    assert torch.equal(st[1].cpu(), state[1])
    # single tokens: norm and shift in one launch
    x, w = torch.randn(3, width, generator=g), torch.rand(width, generator=g) + 0.5
    st = dev(state)
    fused = torch.empty(3, width, device=DEV)
    ops.group_rms_norm(dev(x), dev(w), 4, 1e-5, fused, shift_mix=dev(mix), shift_state=st, slot=i32([3, 1, 0]))
    normed = plain.group_norm(x, w, 4, 1e-5)
    for r, s in enumerate([3, 1, 0]):
        want = normed[r] + (state[s] - normed[r]) * mix
        assert torch.allclose(fused[r].cpu(), want, atol=2e-6)
        assert torch.allclose(st[s].cpu(), normed[r], atol=2e-6)


def test_sinusoid_embedding_kernel_far_positions():
    from imparo_amd.kernels import ops
    width, V = 50, 30
    g = torch.Generator().manual_seed(4)
    table = torch.randn(V, width, generator=g)
    ids, pos = [3, 29, 0, 7], [0, 1, 4097, 100000]
    i = np.arange(width // 2, dtype=np.float32)
    inv = np.power(np.float32(10000.0), (np.float32(-2.0) * i / np.float32(width)).astype(np.float32)).astype(np.float32)
    out = torch.empty(4, width, device=DEV)
    ops.embed_sinusoid(dev(table), i32(ids), i32(pos), dev(torch.from_numpy(inv)), out)
    ref = table[ids].double() + plain.sinusoid(torch.tensor(pos), width, torch.float64)
    # float32 angles: an angle of 1e5 carries an error of 4e-3 at most, small angles almost none
    err = (out.cpu().double() - ref).abs()
    assert float(err[:2].max()) < 1e-6 and float(err[2].max()) < 5e-4 and float(err[3].max()) < 1e-2
    angle = (np.float32(100000) * inv).astype(np.float32)
    assert np.allclose(out[3, 0::2].cpu().numpy() - table[ids[3], 0::2].numpy(), np.sin(angle.astype(np.float64)), atol=2e-6)


@pytest.mark.parametrize("width,pad", [(44, 4), (96, 0), (1000, 0)])
def test_poly_norm_kernel(width, pad):
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(width)
    z = torch.randn(5, width + pad, generator=g) * 2
    coef = torch.tensor([0.9, -0.4, 0.3, 0.05])
    out = torch.full((5, width + pad), 7.0, device=DEV)
    ops.poly_norm(dev(z), dev(coef), 1e-5, out, width=width)
    zz = z[:, :width]
    ref = 0.9 * plain.rms(zz, 1e-5) - 0.4 * plain.rms(zz ** 2, 1e-5) + 0.3 * plain.rms(zz ** 3, 1e-5) + 0.05
    assert torch.allclose(out[:, :width].cpu(), ref, atol=1e-5, rtol=1e-5)
    assert pad == 0 or float(out[:, width:].abs().max()) == 0.0


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_causal_conv_kernel_continues(taps):
    """A sequence cut into segments of 1, 2, 1 and 6 tokens (shorter than the history, then longer), another
    request between them; the history is what the cuts carry."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(taps)
    C, ld = 40, 90
    u = torch.randn(10, ld, generator=g)
    other = torch.randn(3, ld, generator=g)
    w, b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    ref = torch.nn.functional.silu(plain.causal_conv(u[:, :C], w, b))
    ref_other = torch.nn.functional.silu(plain.causal_conv(other[:, :C], w, b))
    state = dev(torch.zeros(3, taps - 1, C)) if taps > 1 else None
    got, got_other, at = [], [], 0
    for n in (1, 2, 1, 6):
        if n == 1:       # every row one token, the other request beside it: the one-launch form
            rows = torch.cat([u[at:at + 1], other[len(got_other):len(got_other) + 1]])
            out = torch.empty(2, C, device=DEV)
            ops.causal_conv(dev(rows), C, dev(w), dev(b), state, i32([0, 1]), i32([0, 1]), i32([1, 1]), i32([2, 0]),
                            out, single_tokens=True)
            got.append(out[0:1].cpu())
            got_other.append(out[1:2].cpu())
        else:
            out = torch.empty(n, C, device=DEV)
            ops.causal_conv(dev(u[at:at + n]), C, dev(w), dev(b), state, i32([0] * n), i32([0]), i32([n]), i32([2]), out)
            got.append(out.cpu())
        at += n
    assert torch.allclose(torch.cat(got), ref, atol=1e-5, rtol=1e-5)
    assert torch.allclose(torch.cat(got_other), ref_other[:2], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("C,N", [(24, 8), (40, 20), (16, 1), (8, 80)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_selective_scan_kernel_continues(C, N, dtype):
    """One sequence in segments of 1 to 200 tokens, the long ones walked in chunks side by side: the state
    carries from segment to segment and from chunk to chunk; other slots stay untouched."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(C * N)
    cuts = (1, 7, 2, 1, 12, 200, 97, 130)
    T = sum(cuts)
    dt_raw, x = torch.randn(T, C, generator=g) - 2, torch.randn(T, C, generator=g).to(dtype).float()
    bc, z = torch.randn(T, 2 * N, generator=g), torch.randn(T, 2 * C, generator=g)
    A, D = -torch.rand(C, N, generator=g) * 6, torch.randn(C, generator=g)
    ref = plain.scan(torch.nn.functional.softplus(dt_raw), x, bc[:, :N], bc[:, N:], A, D) * torch.nn.functional.silu(z[:, C:])
    state = dev(torch.zeros(5, C, N))
    chunk = ops.selective_scan_chunk()
    got, at = [], 0
    for n in cuts:
        out = torch.empty(n, C, device=DEV, dtype=dtype)
        zz = dev(z[at:at + n])
        n_chunks = -(-n // chunk) if n > chunk + chunk // 2 else 1
        scratch = torch.full((ops.selective_scan_scratch(1, n_chunks, C, N),), float("nan"), device=DEV) if n_chunks > 1 else None
        ops.selective_scan(dev(dt_raw[at:at + n]), dev(x[at:at + n], dtype), dev(bc[at:at + n]), zz[:, C:], 2 * C, dev(A),
                           dev(D), state, i32([0]), i32([n]), i32([3]), out, scratch, n_chunks)
        got.append(out.float().cpu())
        at += n
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(torch.cat(got), ref, atol=tol * float(ref.abs().max()), rtol=tol)
    assert float(state[[0, 1, 2, 4]].abs().max()) == 0.0


def test_selective_scan_kernel_rows_of_unequal_length():
    """Three requests in one launch, 150, 1 and 70 tokens: chunks for the long one only; each equals its own run."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(77)
    C, N, lens = 24, 12, [150, 1, 70]
    T = sum(lens)
    dt_raw, x = torch.randn(T, C, generator=g) - 2, torch.randn(T, C, generator=g)
    bc, z = torch.randn(T, 2 * N, generator=g), torch.randn(T, 2 * C, generator=g)
    A, D = -torch.rand(C, N, generator=g) * 6, torch.randn(C, generator=g)
    first = torch.randn(4, C, N, generator=g)
    state = dev(first)
    out = torch.empty(T, C, device=DEV)
    chunk = ops.selective_scan_chunk()
    n_chunks = -(-max(lens) // chunk)
    scratch = torch.full((ops.selective_scan_scratch(3, n_chunks, C, N),), float("nan"), device=DEV)
    zz = dev(z)
    ops.selective_scan(dev(dt_raw), dev(x), dev(bc), zz[:, C:], 2 * C, dev(A), dev(D), state, i32([0, 150, 151]),
                       i32(lens), i32([2, 0, 3]), out, scratch, n_chunks)
    at = 0
    for n, s in zip(lens, [2, 0, 3]):
        S = first[s].clone()
        sl = slice(at, at + n)
        ref = plain.scan(torch.nn.functional.softplus(dt_raw[sl]), x[sl], bc[sl, :N], bc[sl, N:], A, D, S) \
            * torch.nn.functional.silu(z[sl, C:])
        assert torch.allclose(out[sl].cpu(), ref, atol=2e-5 * float(ref.abs().max()), rtol=2e-5)
        assert torch.allclose(state[s].cpu(), S, atol=1e-5, rtol=1e-5)
        at += n
    assert torch.equal(state[1].cpu(), first[1])


def attention_case(H, G, D, V, n_ctx, page, dtype, far=None, seed=0):
    """Writes n_ctx keys into scrambled pages in portions, then asks every position's query; returns the
    kernel's output per number of splits and the plain one."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n_ctx, H, 2, D, generator=g)
    k = torch.randn(n_ctx, G, 2, D, generator=g)
    v = torch.randn(n_ctx, G, V, generator=g)
    gate = torch.randn(n_ctx, H * V, generator=g)
    if far is not None:           # one key far back that the last queries' second map singles out
        k[far, :, 1] = 4.0 * q[-1, 0, 1] / q[-1, 0, 1].norm()
        q[-3:, :, 1] = 3.0 * q[-1, 0, 1]
        v[far] = 5.0
    q, k, v = [t.to(dtype).float() for t in (q, k, v)]
    scale, lam, diff, eps = 1.0 / math.sqrt(D), 0.65, 0.35, 1e-5
    ref = plain.differential_core(q, k, v, torch.arange(n_ctx), scale, lam, diff, eps) * torch.sigmoid(gate)
    n_pages = -(-n_ctx // page) + 3
    order = list(range(n_pages))
    random.Random(seed).shuffle(order)
    table = i32([order[:-(-n_ctx // page)]])
    k_cache = torch.zeros(n_pages, 2 * G, page, D, device=DEV, dtype=dtype)
    v_cache = torch.zeros(n_pages, G, page, V, device=DEV, dtype=dtype)
    rows = torch.cat([q.reshape(n_ctx, -1), k.reshape(n_ctx, -1), v.reshape(n_ctx, -1), gate], dim=1)
    q_dev = torch.empty(n_ctx, H, 2, D, device=DEV, dtype=dtype)
    pos, row = i32(list(range(n_ctx))), i32([0] * n_ctx)
    ops.diff_qkv_store(dev(rows), pos, row, table, page, q_dev, k_cache, v_cache, H, G, D, V, 0.0, 0)
    outs = {}
    for n_splits in (1, -(-n_ctx // ops.diff_attention_split())):
        out = torch.empty(n_ctx, H * V, device=DEV, dtype=dtype)
        part = torch.zeros(n_ctx * H * n_splits * (2 * V + 4), device=DEV) if n_splits > 1 else None
        ops.diff_attention(q_dev, k_cache, v_cache, dev(gate), H * V, out, pos, row, table, scale, None, lam, eps,
                           1.0 - diff, part, n_splits)
        outs[n_splits] = out.float().cpu()
    return outs, ref


@pytest.mark.parametrize("H,G,D,V,page", [(4, 2, 16, 32, 16), (3, 1, 24, 40, 64), (1, 1, 8, 8, 8), (2, 2, 20, 130, 32),
                                          (8, 1, 16, 96, 16), (8, 2, 36, 64, 32)])
def test_differential_attention_kernel_float32(H, G, D, V, page):
    """Every position of 700 keys over scrambled pages, whole and in splits of the keys; one to eight heads
    on a key/value head."""
    outs, ref = attention_case(H, G, D, V, 700, page, torch.float32, seed=H)
    for n_splits, out in outs.items():
        assert torch.allclose(out, ref, atol=2e-5, rtol=1e-4), f"{n_splits} splits: {float((out - ref).abs().max())}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_differential_attention_finds_a_far_key(dtype):
    """Key 5 of 900 carries most of the last queries' second map: a kernel that loses it (a page's or a
    split's edge, a wrong map) is off by far more than rounding."""
    outs, ref = attention_case(2, 1, 32, 16, 900, 16, dtype, far=5, seed=9)
    without, _ = attention_case(2, 1, 32, 16, 900, 16, dtype, far=None, seed=9)
    tol = 1e-4 if dtype == torch.float32 else 4e-2
    for n_splits, out in outs.items():
        assert float((out[-3:] - without[n_splits][-3:]).abs().max()) > 0.3          # the far key matters
        assert float((out - ref).abs().max()) < tol, f"{n_splits} splits"


@pytest.mark.parametrize("H,G,D,V,page", [(4, 2, 16, 32, 16), (3, 1, 24, 40, 64), (1, 1, 8, 8, 16), (4, 1, 64, 128, 32),
                                          (2, 2, 36, 20, 16)])
def test_differential_attention_matrix_core_kernel(H, G, D, V, page):
    """The kernel for portions (bfloat16): a portion of 403 queries behind 297 cached keys, beside a row of
    one token that it must leave alone and a short row of three; a far key that the second map singles out."""
    from imparo_amd.kernels import ops
    g = torch.Generator().manual_seed(H * 10 + D)
    n_ctx, cut = 700, 297
    q = torch.randn(n_ctx, H, 2, D, generator=g)
    k = torch.randn(n_ctx, G, 2, D, generator=g)
    v = torch.randn(n_ctx, G, V, generator=g)
    gate = torch.randn(n_ctx, H * V, generator=g)
    k[5, :, 1] = 4.0 * q[-1, 0, 1] / q[-1, 0, 1].norm()
    q[-3:, :, 1] = 3.0 * q[-1, 0, 1]
    v[5] = 5.0
    q, k, v = [t.to(torch.bfloat16).float() for t in (q, k, v)]
    scale, lam, diff, eps = 1.0 / math.sqrt(D), 0.65, 0.35, 1e-5
    ref = plain.differential_core(q, k, v, torch.arange(n_ctx), scale, lam, diff, eps) * torch.sigmoid(gate)
    n_pages = 2 * (-(-n_ctx // page)) + 2
    order = list(range(n_pages))
    random.Random(D).shuffle(order)
    per = -(-n_ctx // page)
    # request 0 holds all 700 keys; request 1 holds the first 3 of the same sequence in pages of its own
    table = i32([order[:per], order[per:2 * per]])
    k_cache = torch.zeros(n_pages, 2 * G, page, D, device=DEV, dtype=torch.bfloat16)
    v_cache = torch.zeros(n_pages, G, page, V, device=DEV, dtype=torch.bfloat16)
    rows = torch.cat([q.reshape(n_ctx, -1), k.reshape(n_ctx, -1), v.reshape(n_ctx, -1), gate], dim=1)
    store = lambda sel, row: ops.diff_qkv_store(
        dev(rows[sel]), i32(sel), i32([row] * len(sel)), table, page,
        torch.empty(len(sel), H, 2, D, device=DEV, dtype=torch.bfloat16), k_cache, v_cache, H, G, D, V, 0.0, 0)
    store(list(range(cut)), 0)
    # the step: request 0's last 403 tokens, a single token of request 0's twin... kept simple: request 1 brings 3 tokens
    sel = list(range(cut, n_ctx)) + [0, 1, 2]
    row_of = [0] * (n_ctx - cut) + [1] * 3
    q_dev = torch.empty(len(sel), H, 2, D, device=DEV, dtype=torch.bfloat16)
    ops.diff_qkv_store(dev(rows[sel]), i32(sel), i32(row_of), table, page, q_dev, k_cache, v_cache, H, G, D, V, 0.0, 0)
    out = torch.full((len(sel), H * V), 9.0, device=DEV, dtype=torch.bfloat16)
    ops.diff_attention_tiles(q_dev, k_cache, v_cache, dev(gate[sel]), H * V, out, i32(sel), i32([0, n_ctx - cut]),
                             i32([n_ctx - cut, 3]), n_ctx - cut, table, scale, None, lam, eps, 1.0 - diff, min_len=2)
    got = out.float().cpu()
    assert float((got - ref[sel]).abs().max()) < 4e-2
    # with min_len 4 the short row is left alone
    out.fill_(9.0)
    ops.diff_attention_tiles(q_dev, k_cache, v_cache, dev(gate[sel]), H * V, out, i32(sel), i32([0, n_ctx - cut]),
                             i32([n_ctx - cut, 3]), n_ctx - cut, table, scale, None, lam, eps, 1.0 - diff, min_len=4)
    assert float((out[:-3].float().cpu() - ref[sel[:-3]]).abs().max()) < 4e-2 and bool((out[-3:] == 9.0).all())
    # and the wave kernel takes exactly the rows below a length
    ops.diff_attention(q_dev, k_cache, v_cache, dev(gate[sel]), H * V, out, i32(sel), i32(row_of), table, scale, None, lam,
                       eps, 1.0 - diff, None, 1, seg_len=i32([n_ctx - cut, 3]), below=4)
    assert float((out.float().cpu() - ref[sel]).abs().max()) < 4e-2


# ------------------------------------------------------------------ the model in the engine
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_prompt_and_stepwise(dirs, plains, name, dtype):
    """A prompt whole; then most of it whole and its last 40 tokens one by one (captured steps)."""
    from imparo_amd.engine import StepEntry
    tokens = prompt_tokens(vocab(name), 150, 7)
    ref = plains[name].logits(tokens)
    rel = bound(dtype, runs(name))
    eng = make_engine(dirs[name], dtype)
    whole = eng.step([StepEntry("w", tokens, list(range(150)))]).cpu()
    eng.release("w")
    check_logits(whole, ref, dtype, f"{name} whole", rel)
    head = eng.step([StepEntry("d", tokens[:110], list(range(110)))]).cpu()
    tail = [eng.step([StepEntry("d", [t], [0])]).cpu() for t in tokens[110:]]
    eng.release("d")
    stepwise = torch.cat([head] + tail)
    check_logits(stepwise, ref, dtype, f"{name} stepwise", rel)
    if dtype == "float32":
        check_logits(stepwise, whole, dtype, f"{name} stepwise against whole", 2e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 16), ("B", 8), ("D", 16)])
def test_portions_of_changing_size(dirs, plains, name, page, dtype):
    """Portions down to two tokens, cut inside pages, also without launch-by-launch graphs."""
    tokens = prompt_tokens(vocab(name), 140, 8)
    ref = plains[name].logits(tokens)
    for cuts, graphs in (((2, 3, 17, 2, 1, 31, 1, 1, 5), True), ((64, 2, 9), False), ((1,), True)):
        eng = make_engine(dirs[name], dtype, page_size=page, use_graphs=graphs)
        got = step_all(eng, "p", tokens if cuts != (1,) else tokens[:40], cuts)
        check_logits(got, ref[:got.shape[0]], dtype, f"{name} cuts {cuts}", bound(dtype, runs(name)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_batches_on_a_full_pool(dirs, plains, name, dtype):
    """Six unequal requests, at most four live, portions beside single tokens, on a pool of exactly the
    schedule's peak and four slots: pages and slots are used again. Each request's logits are those it
    has alone."""
    from imparo_amd.engine import StepEntry
    rng = random.Random(5)
    lengths = [70, 33, 1, 90, 2, 51]
    prompts = [prompt_tokens(vocab(name), n, 20 + i) for i, n in enumerate(lengths)]
    steps = mixed_schedule(rng, lengths, max_live=4)
    page = 8
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
        check_logits(torch.cat(got[i]), plains[name].logits(p), dtype, f"{name} request {i}", bound(dtype, runs(name)))
    eng.cache.check()
    assert eng.free_pages() == [g.pool.n_pages for g in eng.cache.groups]


def test_long_decoding_and_first_tokens(dirs, plains):
    """One prompt token, then 330 single-token steps over many pages (the query temperature passes 40
    of its steps); and requests of one and of two tokens alone."""
    from imparo_amd.engine import StepEntry
    tokens = prompt_tokens(vocab("A"), 331, 3)
    ref = plains["A"].logits(tokens)
    for dtype in ("float32", "bfloat16"):
        eng = make_engine(dirs["A"], dtype, page_size=8)
        got = torch.cat([eng.step([StepEntry("r", [t], [0])]).cpu() for t in tokens])
        check_logits(got, ref, dtype, "long decoding", bound(dtype, runs("A")))
        eng.release("r")
        two = eng.step([StepEntry("x", tokens[:1], [0]), StepEntry("y", tokens[:2], [0, 1])]).cpu()
        check_logits(two, torch.cat([ref[:1], ref[:2]]), dtype, "first tokens", bound(dtype, runs("A")))


def test_generation_through_the_entry_point(dirs, plains):
    from imparo_amd import generate
    prompts = [prompt_tokens(vocab("A"), n, 50 + n) for n in (1, 6, 29, 13, 40)]
    want = [plains["A"].greedy(p, 12) for p in prompts]
    assert all(len(set(w)) > 4 for w in want), f"the plain continuation hardly moves: {want}"
    assert generate(dirs["A"], prompts, max_tokens=12, dtype="float32", page_size=8) == want
    # three at a time under a small token budget: prompts in portions beside decoding rows, slots used again
    os.environ["IMPARO_BATCH"] = "5"
    try:
        got = generate(dirs["A"], prompts, max_tokens=12, dtype="float32", page_size=8, parallel=3, max_batch_tokens=11)
    finally:
        del os.environ["IMPARO_BATCH"]
    assert got == want
    got16 = generate(dirs["A"], prompts, max_tokens=12, dtype="bfloat16", parallel=3)
    for p, out in zip(prompts, got16):
        assert len(out) == 12
        assert_picks_near_best(plains["A"], p, out, 2 * bound("bfloat16", runs("A")), "bfloat16")


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
