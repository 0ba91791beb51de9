"""Differential attention over the paged cache.

Every query head holds two softmax maps over the same values: q and k carry
two halves a head (map 1, map 2), a_m = softmax(q_m . k_m * scale) v, and the
head's output is o = a_1 - lambda a_2 with one lambda a layer,
lambda = exp(sum(lq1 * lk1)) - exp(sum(lq2 * lk2)) + diff. o is divided by its
root mean square over the head's values (no weight), multiplied by 1 - diff,
gated element by element with sigmoid(Wg h) and projected out. Query head h
reads key/value head floor(h / (heads / kv_heads)). There is no rotation;
`q_temp` (coef, every) multiplies the query at position p by
1 + coef * ln(floor((p + 1) / every) + 1). q, k and v carry biases where
`qkv_bias` says so. Scores, softmax, the combination and the norm are float32.

One projection makes [q | k | v | gate logits]; keys and values go into pages
K [2 kv_heads, PAGE, dim] and V [kv_heads, PAGE, vdim] before the same batch's
attention."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.pages import PAGE, PagedArray, PagedSpec
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_projection
from .registry import register_part

_DEFAULT_NAMES = dict(q="q", k="k", v="v", g="g", o="o", lq1="lq1", lk1="lk1", lq2="lq2", lk2="lk2", bias="b")


class DifferentialAttention:
    role = "mixer"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        suffix = names.pop("bias")
        out = {k: f"{spec.prefix}.{v}" for k, v in names.items()}
        out["bias"] = suffix
        return out

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, H, G, D, V = spec["width"], spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
        out: Declared = {
            n["q"]: (TensorDecl((H * 2 * D, E)), "matrix"),
            n["k"]: (TensorDecl((G * 2 * D, E)), "matrix"),
            n["v"]: (TensorDecl((G * V, E)), "matrix"),
            n["o"]: (TensorDecl((E, H * V)), "matrix"),
        }
        for x in ("lq1", "lk1", "lq2", "lk2"):
            out[n[x]] = (TensorDecl((D,), "vector"), "bias")
        if spec.get("gate", True):
            out[n["g"]] = (TensorDecl((H * V, E)), "matrix")
        if spec.get("qkv_bias", True):
            for x, rows in (("q", H * 2 * D), ("k", G * 2 * D), ("v", G * V)):
                out[f"{n[x]}.{n['bias']}"] = (TensorDecl((rows,), "vector"), "bias")
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.heads, self.kv_heads = spec["width"], spec["heads"], spec["kv_heads"]
        self.dim, self.vdim = spec["dim"], spec["vdim"]
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads cannot share {self.kv_heads} kv heads evenly")
        if self.dim > 256 or self.vdim > 512:
            raise ValueError(f"the differential attention kernels take maps of up to 256 and values of up to 512 "
                             f"a head, got {self.dim} and {self.vdim}")
        self.scale = float(spec["scale"])
        self.diff = float(spec["diff"])
        self.eps = float(spec["eps"])
        self.window: Optional[int] = spec.get("window")
        temp = spec.get("q_temp") or {}
        self.temp_coef, self.temp_every = float(temp.get("coef", 0.0)), int(temp.get("every", 0))
        self.gated = bool(spec.get("gate", True))
        names = ["q", "k", "v"] + (["g"] if self.gated else [])
        ws = [tensors[n[x]] for x in names]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        bias = None
        if spec.get("qkv_bias", True):
            bs = [tensors[f"{n[x]}.{n['bias']}"].to(torch.float32) for x in ("q", "k", "v")]
            if self.gated:
                bs.append(torch.zeros(self.heads * self.vdim))
            bias = torch.cat(bs).to(device)
        # one projection for q | k | v | gate logits: the same dot products, one launch
        self.qkvg = Linear(place_projection(torch.cat(ws, dim=0), engine_dtype, device), bias)
        self.gate_at = (self.heads + self.kv_heads) * 2 * self.dim + self.kv_heads * self.vdim
        if engine_dtype != torch.float32 and (self.heads * self.vdim) % 8:
            raise ValueError(f"under bfloat16 the output projection walks its {self.heads} x {self.vdim} inputs in steps "
                             f"of 8; run this model with dtype float32")
        self.out = Linear(place_matrix(tensors[n["o"]], engine_dtype, device))
        l = {x: tensors[n[x]].to(torch.float32) for x in ("lq1", "lk1", "lq2", "lk2")}
        self.lam = float(torch.exp((l["lq1"] * l["lk1"]).sum()) - torch.exp((l["lq2"] * l["lk2"]).sum())) + self.diff

    @property
    def in_dtype(self) -> torch.dtype:
        return self.qkvg.in_dtype

    def cache_spec(self, page_size: int) -> PagedSpec:
        return PagedSpec((PagedArray("k", (2 * self.kv_heads, PAGE, self.dim)),
                          PagedArray("v", (self.kv_heads, PAGE, self.vdim))), self.window)

    def _splits(self, ctx: StepContext, tokens: int) -> int:
        """Few queries over long contexts: the keys in pieces, so that more of the chip works."""
        split = ops.diff_attention_split()
        if tokens * self.heads > 512 or ctx.max_context <= 2 * split:
            return 1
        return -(-ctx.max_context // split)

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        T = h.shape[0]
        rows = self.qkvg(ctx, h, torch.float32, "qkvg", alias="mixer_in")
        arrays, table = ctx.paged(site)
        k_cache, v_cache = arrays["k"], arrays["v"]
        q = ctx.workspace.get("q", (T, self.heads, 2, self.dim), ctx.dtype)
        ops.diff_qkv_store(rows, ctx.positions, ctx.row_of_token, table if owns_cache else None, ctx.page_size, q,
                           k_cache if owns_cache else None, v_cache if owns_cache else None, self.heads,
                           self.kv_heads, self.dim, self.vdim, self.temp_coef, self.temp_every)
        o = ctx.workspace.get("attn_out", (T, self.heads * self.vdim), ctx.dtype, alias="mixer_mid")
        gate = rows[:, self.gate_at:] if self.gated else None
        # rows that bring portions go to the matrix cores where the sizes allow; single tokens to the wave
        # kernel, their keys in splits when few of them walk long contexts
        tiles = (ctx.max_seg_len > 1 and ctx.single_rows is not None
                 and ops.diff_attention_tiles_takes(ctx.dtype, ctx.page_size, self.dim, self.vdim))
        if tiles:
            ops.diff_attention_tiles(q, k_cache, v_cache, gate, rows.shape[1], o, ctx.positions, ctx.seg_start,
                                     ctx.seg_len, ctx.max_seg_len, table, self.scale, self.window, self.lam, self.eps,
                                     1.0 - self.diff, min_len=2)
        if not tiles or ctx.n_single_rows:
            singles = ctx.n_single_rows if tiles else T
            n_splits = self._splits(ctx, singles)
            part = None
            if n_splits > 1:
                part = ctx.workspace.get("diff_attn_part", (T * self.heads * n_splits * (2 * self.vdim + 4),),
                                         torch.float32)
            ops.diff_attention(q, k_cache, v_cache, gate, rows.shape[1], o, ctx.positions, ctx.row_of_token, table,
                               self.scale, self.window, self.lam, self.eps, 1.0 - self.diff, part, n_splits,
                               seg_len=ctx.seg_len if tiles else None, below=2 if tiles else 0)
        if o.dtype != self.out.in_dtype:
            raise ValueError("the output projection's weight dtype differs from the attention output's")
        return self.out(ctx, o, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


register_part("mixer", "differential_attention", DifferentialAttention)
