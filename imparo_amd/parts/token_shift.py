"""Token shift: what a mixer reads is mixed with what the token before it
would have read, element by element.

h_t <- h_t + (h_{t-1} - h_t) * mix, with h_{t-1} the previous token's input
as it was before this replacement and zeros before a sequence's first token.
The last token's unshifted input is state of the block, one float32 row per
request, so that a sequence cut into steps continues where it stopped."""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from ..cache.pages import FixedArray
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import place_vector
from .registry import register_part

STATE_NAME = "shift_prev"


class TokenShift:
    role = "shift"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _tensor(spec: PartSpec) -> str:
        return spec.get("tensor") or f"{spec.prefix}.weight"

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        return {cls._tensor(spec): (TensorDecl((spec["width"],), "vector"), "bias")}

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        self.width = spec["width"]
        self.mix = place_vector(tensors[self._tensor(spec)], device)

    def state_arrays(self) -> Tuple[FixedArray, ...]:
        return (FixedArray(STATE_NAME, (self.width,), "float32", 0.0),)

    def state(self, ctx: StepContext, site: int) -> torch.Tensor:
        return ctx.fixed_arrays(site)[STATE_NAME]

    def forward(self, ctx: StepContext, site: int, h: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """`h`: the normed rows in float32. Returns the shifted rows in `out_dtype`; the state moves on."""
        out = ctx.workspace.get("normed", tuple(h.shape), out_dtype)
        return ops.token_shift(h, self.mix, self.state(ctx, site), ctx.row_of_token, ctx.seg_start, ctx.seg_len,
                               ctx.slot, out)


register_part("shift", "token_shift", TokenShift)
