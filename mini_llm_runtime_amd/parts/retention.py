"""Linear attention with a fixed decay: a matrix state per head instead of cached keys."""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..cache.spec import SlotStateSpec
from ..kernels.limits import MAX_STATE_ROWS
from .base import Mixer, Part, PositionEncoding
from .context import StepContext
from .registry import build_part, register_part
from .spec import ParamSpec, PartSpec


@register_part("mixer", "retention")
class Retention(Mixer):
    """Per head i with decay g_i, state S (head_dim x value_dim, 32-bit, zero at a request's start):

        S_t = g_i S_(t-1) + k_t v_t^T,    o_t = S_t^T q_t,

    q = rotate(Wq h), k = rotate(Wk h) * head_dim^-0.5, v = Wv h; no softmax and no denominator.
    Every head's o_t is divided by its root mean square (eps inside the root, no weight); the heads
    side by side are multiplied by silu(Wg h) and projected by Wo.

    The state is all a request keeps (one slot of the cache manager's state banks per request), so a
    prompt can be cut anywhere: a step reads the state its request's previous step left, runs its
    tokens in order and leaves the state behind its last one.  Rotation, scaling, decay, state and
    the heads' norm are 32-bit; the four input products are one (rows q, k, v, gate).
    """

    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        head_dim: int,
        value_dim: int,
        decay: Sequence[float],
        norm_eps: float,
        position: Optional[PartSpec] = None,
    ) -> None:
        if min(hidden_size, num_heads, head_dim, value_dim) <= 0:
            raise ValueError("Retention sizes must be > 0")
        if head_dim > MAX_STATE_ROWS:  # refused here, not at the first step
            raise ValueError(f"head_dim {head_dim}: the retention kernels take heads of up to {MAX_STATE_ROWS} dims")
        if len(decay) != num_heads or not all(0.0 <= float(g) <= 1.0 for g in decay):
            raise ValueError("Retention needs one decay within 0..1 per head")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        self.decay_values = tuple(float(g) for g in decay)
        self.norm_eps = float(norm_eps)
        self.key_scale = float(head_dim) ** -0.5
        self.position: Optional[PositionEncoding] = build_part("position", position) if position is not None else None
        self.in_weight: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None
        self.decay: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        rows = 2 * self.num_heads * self.head_dim + 2 * self.num_heads * self.value_dim
        return {
            "in_weight": ParamSpec((rows, self.hidden_size)),
            "o_weight": ParamSpec((self.hidden_size, self.num_heads * self.value_dim)),
        }

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        super().bind(params, dtype=dtype, device=device)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)

    def children(self) -> dict[str, Part]:
        return {"position": self.position} if self.position is not None else {}

    def cache_spec(self) -> SlotStateSpec:
        return SlotStateSpec((self.num_heads, self.head_dim, self.value_dim), "float32")

    def forward(self, ctx: StepContext, h: torch.Tensor, site: int) -> torch.Tensor:
        ops = ctx.ops
        state = ctx.state(site)
        rotation = self.position.rotation(ctx) if self.position is not None else None
        projected = ops.linear(h, self.in_weight, None, out_dtype=torch.float32)  # what enters the recurrence stays 32-bit
        retained = ops.retention_scan(
            projected,
            state.tensor,
            state.read_rows,
            state.write_rows,
            ctx,
            heads=self.num_heads,
            head_dim=self.head_dim,
            value_dim=self.value_dim,
            decay=self.decay,
            key_scale=self.key_scale,
            rotation=rotation,
        )
        gated = ops.retention_gate(
            retained, projected, heads=self.num_heads, value_dim=self.value_dim,
            gate_offset=2 * self.num_heads * self.head_dim + self.num_heads * self.value_dim, eps=self.norm_eps,
        )
        return ops.linear(gated, self.o_weight, None, for_stream=True)
