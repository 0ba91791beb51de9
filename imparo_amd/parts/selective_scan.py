"""Selective state-space mixer (a selective scan with a short causal conv).

[x | z] = Win h; x through a causal per-channel convolution (`taps` wide, the
last tap the current token's, zeros before the start) with bias and SiLU;
[dt | B | C] = Wx x; dt = softplus(Wdt dt + b), one per channel; A = -exp(A_log);
per channel c and state n: S <- exp(dt_c A[c, n]) S + dt_c x_c B_n,
y_c = sum_n S[c, n] C_n + D_c x_c; the mixer's result is Wo (y * silu(z)).
A request's state is the float32 matrix S [channels, states] and the conv's
last taps - 1 inputs. Step sizes, decays, exponentials and the state are
float32 whatever the engine's dtype."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.pages import FixedArray, FixedSpec
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import Linear, place_matrix, place_projection, place_vector
from .registry import register_part

_DEFAULT_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b",
                  "A_log": "A_log", "D": "D", "o": "o"}


class SelectiveScan:
    role = "mixer"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        E, C, N, R, L = spec["width"], spec["inner"], spec["state"], spec["dt_rank"], spec["taps"]
        return {
            n["in"]: (TensorDecl((2 * C, E)), "matrix"),
            n["conv"]: (TensorDecl((C, L), "vector"), "conv"),
            n["conv_bias"]: (TensorDecl((C,), "vector"), "bias"),
            n["x"]: (TensorDecl((R + 2 * N, C)), "matrix"),
            n["dt"]: (TensorDecl((C, R)), "matrix"),
            n["dt_bias"]: (TensorDecl((C,), "vector"), "bias"),
            n["A_log"]: (TensorDecl((C, N), "vector"), "wide"),
            n["D"]: (TensorDecl((C,), "vector"), "norm"),
            n["o"]: (TensorDecl((E, C)), "matrix"),
        }

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.inner, self.n_state = spec["width"], spec["inner"], spec["state"]
        self.dt_rank, self.taps = spec["dt_rank"], spec["taps"]
        if not 1 <= self.taps <= 64:
            raise ValueError(f"the conv kernels take 1 to 64 taps, got {self.taps}")
        if self.n_state > 512:
            raise ValueError(f"the scan kernel takes up to 512 states a channel, got {self.n_state}")
        R, N = self.dt_rank, self.n_state
        self.in_proj = Linear(place_projection(tensors[n["in"]], engine_dtype, device))
        wx, wdt = tensors[n["x"]], tensors[n["dt"]]
        if wx.dtype != wdt.dtype:
            wx, wdt = wx.to(torch.float32), wdt.to(torch.float32)
        # The step's low-rank input is a product's inner size, which the bfloat16 kernels walk in steps of 8:
        # it is filled up with units of zero weight on both sides, which add nothing to any sum.
        if engine_dtype != torch.float32 and self.inner % 8:
            wx, wdt = wx.to(torch.float32), wdt.to(torch.float32)      # the scan's side of the mixer in float32 then
        fill = (-R) % 8 if (engine_dtype != torch.float32 and wx.dtype != torch.float32) else 0
        low, step = wx[:R], wdt
        if fill:
            low = torch.cat([low, low.new_zeros(fill, self.inner)])
            step = torch.cat([step, step.new_zeros(self.inner, fill)], dim=1)
        # [dt | B | C] = Wx x as two products: the step's input goes on into a product, B and C into the scan
        self.x_low = Linear(place_matrix(low, engine_dtype, device))
        self.x_bc = Linear(place_matrix(wx[R:], engine_dtype, device))
        self.dt_proj = Linear(place_matrix(step, engine_dtype, device), place_vector(tensors[n["dt_bias"]], device))
        self.out_proj = Linear(place_projection(tensors[n["o"]], engine_dtype, device))
        self.conv_weight = place_vector(tensors[n["conv"]].reshape(self.inner, self.taps), device)
        self.conv_bias = place_vector(tensors[n["conv_bias"]], device)
        self.A = (-torch.exp(tensors[n["A_log"]].to(torch.float32))).to(device).contiguous()
        self.D = place_vector(tensors[n["D"]], device)

    @property
    def in_dtype(self) -> torch.dtype:
        return self.in_proj.in_dtype

    def cache_spec(self, page_size: int) -> FixedSpec:
        arrays = (FixedArray("scan", (self.inner, self.n_state), "float32", 0.0),)
        if self.taps > 1:
            arrays += (FixedArray("conv", (self.taps - 1, self.inner), "float32", 0.0),)
        return FixedSpec(arrays=arrays)

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        if not owns_cache:
            raise ValueError("a scan's state cannot be read from another layer")
        T = h.shape[0]
        state = ctx.fixed_arrays(site)
        act = self.x_low.in_dtype
        xz = self.in_proj(ctx, h, torch.float32, "scan_xz", alias="mixer_in")
        x = ctx.workspace.get("scan_x", (T, self.inner), act)
        ops.causal_conv(xz, self.inner, self.conv_weight, self.conv_bias, state.get("conv"), ctx.row_of_token,
                        ctx.seg_start, ctx.seg_len, ctx.slot, x, silu=True, single_tokens=ctx.max_seg_len == 1)
        low = self.x_low(ctx, x, self.dt_proj.in_dtype, "scan_low")
        bc = self.x_bc(ctx, x, torch.float32, "scan_bc")
        dt = self.dt_proj(ctx, low, torch.float32, "scan_dt")
        y = ctx.workspace.get("scan_y", (T, self.inner), self.out_proj.in_dtype, alias="mixer_mid")
        if y.dtype != x.dtype:
            raise ValueError("the scan's input and output projections differ in dtype")
        # a long portion is walked in chunks side by side (their end states meet in scratch)
        chunk = ops.selective_scan_chunk()
        n_chunks = -(-ctx.max_seg_len // chunk) if ctx.max_seg_len > chunk + chunk // 2 else 1
        scratch = None
        if n_chunks > 1:
            scratch = ctx.workspace.get("scan_chunks", (ops.selective_scan_scratch(ctx.n_rows, n_chunks, self.inner,
                                                                                   self.n_state),), torch.float32)
        ops.selective_scan(dt, x, bc, xz[:, self.inner:], 2 * self.inner, self.A, self.D, state["scan"],
                           ctx.seg_start, ctx.seg_len, ctx.slot, y, scratch, n_chunks)
        return self.out_proj(ctx, y, torch.float32, "mixer_out", sliced_ok=True, into=ctx.stream)


register_part("mixer", "selective_scan", SelectiveScan)
