"""What stands between the residual stream and a sublayer in a block: a short convolution over time on
the sublayer's input, and a gate on its result."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.pages import StateSpec
from ..kernels import ops
from .base import StepContext
from .registry import register_conv, register_gate


class CausalConv:
    """h_t <- h_t + sum_j w[:, j] * h_(t - taps + 1 + j) on each channel, zeros before a request's start.
    The last taps - 1 inputs of a request are its state: [taps - 1, width] float32 a slot, position p at
    ring place p % (taps - 1), so that nothing is shifted from step to step. A step's later tokens read
    its earlier ones from the step's own rows; whoever updates the rows afterwards keeps the last of
    them (`ops.gated_norm_add(..., keep=)` or `keep`)."""

    replayable = True
    takes_padding_rows = True  # (position 0 of the first request: they read no history, and none is kept of them)

    def __init__(self, spec, store, dtype: torch.dtype):
        self.width, self.taps, self.dtype = spec.width, int(spec.taps), dtype
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {self.taps} taps (1 to {ops.CONV_MAX_TAPS} are taken)")
        self.weight = store.fetch(spec.tensors["weight"], (self.width, self.taps), "vector")

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.taps - 1, self.width)) if self.taps > 1 else None

    def forward(self, x: torch.Tensor, ctx: StepContext, state, cast_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The convolved rows in the compute dtype (x: the step's float32 rows); `cast_out` gets x itself
        rounded to the compute dtype in the same pass."""
        out = ctx.workspace.get("conv_out", (x.shape[0], self.width), self.dtype)
        ops.causal_conv(out, x, self.weight, state, ctx, cast_out=cast_out)
        return out

    def keep(self, x: torch.Tensor, ctx: StepContext, state) -> None:
        if state is not None:
            ops.keep_rows(x, state, ctx)


class SigmoidGate:
    """The logits of a gate on a sublayer's result, z = W h + b (32-bit sums, kept in 32 bits); the
    result is multiplied by sigmoid(z) where the block adds it to the stream."""

    replayable = True
    takes_padding_rows = True

    def __init__(self, spec, store, dtype: torch.dtype):
        self.width, self.dtype = spec.width, dtype
        t = spec.tensors
        self.weight = store.fetch(t["weight"], (self.width, self.width), "matrix")
        self.bias = store.fetch(t["bias"], (self.width,), "vector") if "bias" in t else None

    def forward(self, h: torch.Tensor, ctx: StepContext, name: str) -> torch.Tensor:
        from .linear import linear

        z = ctx.workspace.get(name, (h.shape[0], self.width), torch.float32)
        linear(h, self.weight, self.bias, out=z)
        return z


register_conv("causal_conv", CausalConv)
register_gate("sigmoid_gate", SigmoidGate)
