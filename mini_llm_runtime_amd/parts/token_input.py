"""Parts that feed something of the token itself into the residual stream at a layer."""

from __future__ import annotations

from typing import Optional

import torch

from .base import Part
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


class TokenInput(Part):
    def forward(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        """x: the residual stream in the engine's dtype [T, H]; returns what the layer adds, [T, H]."""
        raise NotImplementedError


@register_part("token_input", "gated_token_embedding")
class GatedTokenEmbedding(TokenInput):
    """A small embedding of the token, gated by the stream and projected up:

        y = Wproj (gelu_tanh(Wgate x) * e[token]),   e: [vocab, dim], Wgate: [dim, H], Wproj: [H, dim].

    gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))).  The gate product's epilogue
    applies the activation and multiplies with the token's row of the table, which it gathers itself.  The arrangement that holds this
    part norms y with `norm_weight` (a plain RMS weight) when it adds it to the stream.
    """

    replayable = True

    def __init__(self, hidden_size: int, dim: int, vocab_size: int, norm_eps: float) -> None:
        if min(hidden_size, dim, vocab_size) <= 0:
            raise ValueError("GatedTokenEmbedding sizes must be > 0")
        self.hidden_size = int(hidden_size)
        self.dim = int(dim)
        self.vocab_size = int(vocab_size)
        self.norm_eps = float(norm_eps)
        self.table: Optional[torch.Tensor] = None
        self.gate_weight: Optional[torch.Tensor] = None
        self.proj_weight: Optional[torch.Tensor] = None
        self.norm_weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {
            "table": ParamSpec((self.vocab_size, self.dim)),
            "gate_weight": ParamSpec((self.dim, self.hidden_size)),
            "proj_weight": ParamSpec((self.hidden_size, self.dim)),
            "norm_weight": ParamSpec((self.hidden_size,), init="one_plus_normal", keep_stored_precision=True),
        }

    def forward(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        ops = ctx.ops
        gated = ops.linear(
            x, self.gate_weight, None, activation="gelu_tanh", multiply=self.table, multiply_rows=ctx.token_ids
        )
        return ops.linear(gated, self.proj_weight, None, for_stream=True)
