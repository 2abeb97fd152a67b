"""Attention mixers."""

from __future__ import annotations

import math
from typing import Optional

import torch

from ..cache.spec import PagedKVSpec
from ..kernels.limits import check_attention_sizes
from .base import Mixer, Part, PositionEncoding
from .context import MixerPlan, PlanInput, StepContext
from .registry import build_part, register_part
from .spec import ParamSpec, PartSpec


@register_part("mixer", "gqa_attention")
class GQAAttention(Mixer):
    """Grouped-query causal self-attention over the paged cache.

    Order of work, from src/mini_llm_runtime/qwen_model_runner.py:75-183: project
    q, k, v (with bias when `qkv_bias`), encode positions into q and k, store the
    encoded k and the raw v in the cache, attend, merge heads, project out.  Query
    head h reads KV head h // (num_heads // num_kv_heads) (:64-72).  Scores are
    scaled by `scale` (default head_dim^-0.5, :157) and a query at position p sees
    the keys 0..p of its own request (:158-175), or only the last `window` of
    them.  Unlike the reference, which runs whole prompts from in-flight tensors
    and single tokens from the pages, every query here reads the pages, after the
    step's own keys were written: a prompt portion and a decoded token are the
    same case.

    The three projections are one matrix product over the row-wise concatenation
    [Wq; Wk; Wv] (made by the weight rules at load time).

    Options that other decoders use:
    chunk: instead of all earlier keys (or the last `window`), a query at position p sees the keys
        of its own run of `chunk` positions only: floor(p / chunk) * chunk .. p.  Runs are counted
        from position 0 of the request, whatever portions its prompt is processed in.  The pages of
        runs that every later query has left behind are given back, as under a window.
    value_dim: value heads of another width than query and key heads.  The kernels and the pages
        know one head size, so when the two differ all heads are laid out at one common size D
        (the larger, rounded up to a multiple of 16) with zero rows in the projections: zeros add
        nothing to a score, zero value dims come out as zeros and meet zero columns of the output
        projection.  The padding is made once, when the weights are bound.
    output_gate: out = Wo (A * sigmoid(Wg h)), A the attended heads side by side [T, heads * value_dim],
        * the Hadamard product, h the input that q, k and v are made from too.  The Wg product runs
        behind the attention kernel and multiplies in its epilogue.
    """

    replayable = True
    takes_pending_norm = True  # `h` goes to the query/key/value product only (not so with a gate)

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: Optional[PartSpec] = None,
        qkv_bias: bool = True,
        o_bias: bool = False,
        window: Optional[int] = None,
        scale: Optional[float] = None,
        chunk: Optional[int] = None,
        value_dim: Optional[int] = None,
        output_gate: bool = False,
    ) -> None:
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError("num_heads must be a positive multiple of num_kv_heads")
        if head_dim <= 0 or (value_dim is not None and value_dim <= 0):
            raise ValueError("head_dim and value_dim must be > 0")
        if window is not None and chunk is not None:
            raise ValueError("a mixer has a window or a chunked mask, not both")
        if chunk is not None and chunk <= 0:
            raise ValueError("chunk must be > 0")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = self.head_dim if value_dim is None else int(value_dim)
        # the one head size that kernels and pages see
        self.kernel_dim = self.head_dim
        if self.value_dim != self.head_dim:
            self.kernel_dim = -(-max(self.head_dim, self.value_dim) // 16) * 16
        check_attention_sizes(num_heads, num_kv_heads, self.kernel_dim)  # refused here, not at the first step
        self.chunk = None if chunk is None else int(chunk)
        self.output_gate = bool(output_gate)
        if self.output_gate:
            self.takes_pending_norm = False  # the gate product reads `h` too, behind the attention
        self.qkv_bias = bool(qkv_bias)
        self.o_bias = bool(o_bias)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position: Optional[PositionEncoding] = (
            build_part("position", position) if position is not None else None
        )
        self.qkv_weight: Optional[torch.Tensor] = None
        self.qkv_bias_vec: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None
        self.o_bias_vec: Optional[torch.Tensor] = None
        self.gate_weight: Optional[torch.Tensor] = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_kv_heads * self.value_dim

    @property
    def out_size(self) -> int:
        """Width of the merged heads: what the output projection (and the gate) works on."""
        return self.num_heads * self.value_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        width = self.q_size + self.kv_size + self.v_size
        specs = {
            "qkv_weight": ParamSpec((width, self.hidden_size)),
            "o_weight": ParamSpec((self.hidden_size, self.out_size)),
        }
        if self.qkv_bias:
            specs["qkv_bias_vec"] = ParamSpec((width,), keep_stored_precision=True)
        if self.o_bias:
            specs["o_bias_vec"] = ParamSpec((self.hidden_size,), keep_stored_precision=True)
        if self.output_gate:
            specs["gate_weight"] = ParamSpec((self.out_size, self.hidden_size))
        return specs

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        super().bind(params, dtype=dtype, device=device)
        D = self.kernel_dim
        if D == self.head_dim == self.value_dim:
            return
        # heads of two widths: every head at the common size D, the added rows and columns zero
        def rows(t, heads, size):  # [heads * size, ...] -> [heads * D, ...]
            t = t.view(heads, size, *t.shape[1:])
            out = t.new_zeros((heads, D, *t.shape[2:]))
            out[:, :size] = t
            return out.view(heads * D, *t.shape[2:])

        def fused(t):
            q, k, v = t.split([self.q_size, self.kv_size, self.v_size])
            return torch.cat(
                [rows(q, self.num_heads, self.head_dim), rows(k, self.num_kv_heads, self.head_dim),
                 rows(v, self.num_kv_heads, self.value_dim)]
            ).contiguous()

        self.qkv_weight = fused(self.qkv_weight)
        if self.qkv_bias_vec is not None:
            self.qkv_bias_vec = fused(self.qkv_bias_vec)
        if self.gate_weight is not None:
            self.gate_weight = rows(self.gate_weight, self.num_heads, self.value_dim).contiguous()
        self.o_weight = rows(self.o_weight.t().contiguous(), self.num_heads, self.value_dim).t().contiguous()

    def children(self) -> dict[str, Part]:
        return {"position": self.position} if self.position is not None else {}

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.num_kv_heads, self.kernel_dim, self.window, chunk=self.chunk)

    def plan(self, ops, shape: PlanInput) -> Optional[MixerPlan]:
        make = getattr(ops, "attention_plan", None)  # the kernel library knows what its kernels want
        return make(shape) if make is not None else None

    def forward(self, ctx: StepContext, h: torch.Tensor, site: int) -> torch.Tensor:
        ops = ctx.ops
        cache = ctx.kv(site)
        rotation = self.position.rotation(ctx) if self.position is not None else None
        pages = dict(
            num_heads=self.num_heads,
            num_kv_heads=self.num_kv_heads,
            head_dim=self.kernel_dim,
            block_size=cache.block_size,
            write=cache.writable,
        )
        if self.position is not None and rotation is None:
            # a position encoding with a rule of its own: it sees the queries and keys between
            # the product and the cache write
            qkv = ops.linear(h, self.qkv_weight, self.qkv_bias_vec)
            tokens = qkv.shape[0]
            D = self.kernel_dim
            q = qkv[:, : self.num_heads * D].view(tokens, self.num_heads, D)
            k = qkv[:, self.num_heads * D : (self.num_heads + self.num_kv_heads) * D].view(tokens, self.num_kv_heads, D)
            self.position.apply(ctx, q, k)
            ops.rope_kv_write(qkv, None, cache.slot_mapping, cache.key, cache.value, **pages)
        else:
            qkv = ops.qkv_rope_write(
                h, self.qkv_weight, self.qkv_bias_vec, rotation, cache.slot_mapping, cache.key, cache.value, **pages
            )
        if cache.writable:
            cache.written()
        cache.reading()
        attended = ops.paged_attention(
            qkv,
            cache.key,
            cache.value,
            cache.block_table,
            ctx,
            num_heads=self.num_heads,
            num_kv_heads=self.num_kv_heads,
            head_dim=self.kernel_dim,
            block_size=cache.block_size,
            scale=self.scale,
            window=self.window,
            defer_merge=not self.output_gate,  # the output product is the only reader
            plan=ctx.plan(getattr(ops, "ATTENTION_PLAN", None)),
            **({"chunk": self.chunk} if self.chunk is not None else {}),
        )
        if self.output_gate:
            attended = ops.linear(h, self.gate_weight, None, activation="sigmoid", multiply=attended)
        return ops.linear(attended, self.o_weight, self.o_bias_vec, for_stream=True)  # the next norm's delta
