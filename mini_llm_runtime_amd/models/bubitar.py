"""The Bubitar decoder as a list of parts.

A decoder whose config.json lists the layers one by one.  Every layer norms its sublayers' inputs
AND outputs (`sandwich_norm`), mixes tokens either by retention (linear attention with a fixed decay
per head and a matrix state) or by attention over cached latents (one compressed vector and one
shared rotated key part per token, a sink in the softmax, a gate per head; a layer may read an
earlier layer's cache), has a dense gated feed-forward with clamped halves and biases (or none), and
ends by adding a gated, projected embedding of the token itself, taken from columns of one table that
all layers share.  The head is a matrix of its own.

Checkpoint tensors: `embed`, `side.embed` [vocab, layers * side dim], `final.norm`, `head`, and per
layer i `l<i>.norm1`, `.norm1b`, `.norm2`, `.norm2b`, `l<i>.mix.{q,k,v,g,o}` (retention) or
`l<i>.mix.{q,dkv,dkv.norm,uk,uv,sink,g,o}` (latent attention; no `dkv*` when the cache is another
layer's), `l<i>.mlp.{gate,up,down}` with `.b` biases, `l<i>.side.{gate,proj,norm}`; linear weights
are stored [out, in].
"""

from __future__ import annotations

from ..config.bubitar import BubitarConfig, BubitarLatentAttention, BubitarRetention, Rotary
from ..parts.spec import LayerSpec, ModelSpec, OrderEntry, PartSpec, WeightRule
from .registry import register_architecture

# positions are only limited by what a rotation can tell apart
_NO_POSITION_LIMIT = 1 << 30


def _rotary(rot: Rotary, part_dim: int) -> PartSpec:
    scaling = None
    if rot.scaling is not None:
        s = rot.scaling
        scaling = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
    return PartSpec("rotary", {"head_dim": part_dim, "theta": rot.base, "rotary_dim": rot.dims, "scaling": scaling})


def bubitar_spec(config: BubitarConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps
    norm = PartSpec("rms_norm", {"size": width, "eps": eps})
    side = config.token_side_dim
    table_shape = (config.vocab, len(config.layers) * side)
    layers: list[LayerSpec] = []
    order: list[OrderEntry] = []
    rules: list[WeightRule] = [WeightRule("embed", "embed.weight")]
    for i, layer in enumerate(config.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        m = layer.mixer
        mix = dst + "mixer."
        if isinstance(m, BubitarRetention):
            mixer = PartSpec(
                "retention",
                {
                    "hidden_size": width, "num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
                    "decay": m.decay, "norm_eps": eps, "position": _rotary(m.rot, m.dim),
                },
            )
            qk, vg = m.heads * m.dim, m.heads * m.vdim
            rules += [
                WeightRule(src + "mix.q", mix + "in_weight", 0, qk),
                WeightRule(src + "mix.k", mix + "in_weight", qk, qk),
                WeightRule(src + "mix.v", mix + "in_weight", 2 * qk, vg),
                WeightRule(src + "mix.g", mix + "in_weight", 2 * qk + vg, vg),
                WeightRule(src + "mix.o", mix + "o_weight"),
            ]
            order.append(OrderEntry(i))
        elif isinstance(m, BubitarLatentAttention):
            shared = m.kv_from is not None
            mixer = PartSpec(
                "latent_attention",
                {
                    "hidden_size": width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
                    "value_dim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "norm_eps": eps,
                    "position": _rotary(m.rot, m.rot_dim), "reads_cache": shared,
                },
            )
            q_rows = m.heads * (m.dim + m.rot_dim)
            kv_rows = 0 if shared else m.kv_rank + m.rot_dim
            rules.append(WeightRule(src + "mix.q", mix + "in_weight", 0, q_rows))
            if not shared:
                rules += [
                    WeightRule(src + "mix.dkv", mix + "in_weight", q_rows, kv_rows),
                    WeightRule(src + "mix.dkv.norm", mix + "latent_norm_weight"),
                ]
            rules += [
                WeightRule(src + "mix.g", mix + "in_weight", q_rows + kv_rows, m.heads),
                WeightRule(src + "mix.uk", mix + "uk_weight"),
                WeightRule(src + "mix.uv", mix + "uv_weight"),
                WeightRule(src + "mix.sink", mix + "sink"),
                WeightRule(src + "mix.o", mix + "o_weight"),
            ]
            order.append(OrderEntry(i, reads_cache_of=m.kv_from))  # a layer runs once: its site is its index
        else:
            raise TypeError(f"layer {i}: unknown mixer configuration {type(m).__name__}")
        norms = {"input": norm, "mixer_out": norm}
        rules += [
            WeightRule(src + "norm1", dst + "norm_input.weight"),
            WeightRule(src + "norm1b", dst + "norm_mixer_out.weight"),
        ]
        feed_forward = None
        f = layer.mlp
        if f is not None:
            norms.update(post_mixer=norm, ff_out=norm)
            feed_forward = PartSpec("clamped_glu", {"hidden_size": width, "intermediate_size": f.ff, "limit": f.limit})
            ff = dst + "feed_forward."
            # gate and up rows (and biases) woven in pairs: the product's epilogue then holds a gate sum
            # beside its up sum (an odd size cannot be woven: gate rows, then up rows)
            weave = dict(block=2, period=4) if f.ff % 2 == 0 else {}
            up_at = 2 if weave else f.ff
            rules += [
                WeightRule(src + "norm2", dst + "norm_post_mixer.weight"),
                WeightRule(src + "norm2b", dst + "norm_ff_out.weight"),
                WeightRule(src + "mlp.gate", ff + "gate_up_weight", 0, f.ff, **weave),
                WeightRule(src + "mlp.up", ff + "gate_up_weight", up_at, f.ff, **weave),
                WeightRule(src + "mlp.gate.b", ff + "gate_up_bias", 0, f.ff, **weave),
                WeightRule(src + "mlp.up.b", ff + "gate_up_bias", up_at, f.ff, **weave),
                WeightRule(src + "mlp.down", ff + "down_weight"),
                WeightRule(src + "mlp.down.b", ff + "down_bias"),
            ]
        token_input = PartSpec(
            "gated_token_embedding", {"hidden_size": width, "dim": side, "vocab_size": config.vocab, "norm_eps": eps}
        )
        ti = dst + "token_input."
        rules += [
            # layer i's columns of the one table
            WeightRule("side.embed", ti + "table", source_shape=table_shape, source_cols=(i * side, side)),
            WeightRule(src + "side.gate", ti + "gate_weight"),
            WeightRule(src + "side.proj", ti + "proj_weight"),
            WeightRule(src + "side.norm", ti + "norm_weight"),
        ]
        layers.append(
            LayerSpec(block="sandwich_norm", mixer=mixer, feed_forward=feed_forward, norms=norms, token_input=token_input)
        )
    rules += [WeightRule("final.norm", "final_norm.weight"), WeightRule("head", "head.weight")]
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        hidden_size=width,
        max_position_embeddings=_NO_POSITION_LIMIT,
        layers=tuple(layers),
        order=tuple(order),
        final_norm=norm,
        tie_word_embeddings=False,
        weight_rules=tuple(rules),
    )


register_architecture(BubitarConfig.architecture, BubitarConfig, bubitar_spec, replace=True)
