"""Norms."""

from __future__ import annotations

from typing import Mapping, Optional

import torch

from .base import Norm
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """`weight * x * rsqrt(mean(x^2) + eps)`: no centring, no bias, weight used as is.

    weight_offset: for checkpoints that store the weight as its distance from a constant (usually
    1: `(1 + w) * x * rsqrt(...)`).  The sum offset + w is made once, in 32-bit, when the weights
    are bound, and kept in 32-bit whatever the stored precision (1 + w does not fit bfloat16), so
    every kernel that takes a norm weight, fused ones included, serves both conventions.

    Formula: src/mini_llm_runtime/qwen_model_runner.py:22-26.  Statistics and the
    scaling are computed in 32-bit from the 32-bit residual stream; the result is
    rounded once to the engine's dtype.
    """

    replayable = True
    can_defer = True

    def __init__(self, size: int, eps: float, weight_offset: float = 0.0) -> None:
        if size <= 0 or not eps >= 0:
            raise ValueError("RMSNorm needs size > 0 and eps >= 0")
        self.size = int(size)
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        init = "normal" if self.weight_offset else "one_plus_normal"  # the effective weight is around one either way
        return {"weight": ParamSpec((self.size,), init=init, keep_stored_precision=True)}

    def bind(self, params: Mapping[str, torch.Tensor], *, dtype: torch.dtype, device: torch.device) -> None:
        weight = params["weight"]
        if self.weight_offset:
            weight = weight.to(torch.float32) + self.weight_offset
        self.weight = weight

    def forward(self, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor] = None, defer: bool = False):
        """defer: the consumer takes a norm that has not run (see `Part.takes_pending_norm`); the
        kernel library decides whether there is something to gain."""
        if defer:
            make = getattr(ctx.ops, "defer_norm", None)
            pending = make(x, self.weight, self.eps, delta) if make is not None else None
            if pending is not None:
                return pending
        return ctx.ops.rmsnorm(x, self.weight, self.eps, delta=delta)

