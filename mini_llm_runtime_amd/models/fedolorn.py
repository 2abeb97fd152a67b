"""The Fedolorn decoder as a list of parts.

A pre-norm decoder whose layers are listed one by one in its config.json, each with sizes of its
own: RMSNorm whose checkpoint holds weight - 1; attention without any position encoding, with a
mask cut into runs of positions, value heads of their own width, a scale from the config and a
sigmoid output gate; then either a dense feed-forward with a squared ReLU, or a mixture of
experts with sigmoid scores, a correction vector and a choice limited to the best groups, or
nothing.  The embedding is scaled; the head is the embedding table itself, unscaled.

Checkpoint tensors: `embed`, `final.norm`, and per layer i `l<i>.norm1`, `l<i>.norm2`,
`l<i>.mix.{q,k,v,g,o}`, `l<i>.mlp.{up,down}` or `l<i>.mlp.{router,correction}` with
`l<i>.mlp.e<j>.{up,down}`; linear weights are stored [out, in].
"""

from __future__ import annotations

from ..config.fedolorn import FedolornConfig
from ..parts.spec import LayerSpec, ModelSpec, OrderEntry, PartSpec, WeightRule
from .registry import register_architecture

# the design has no position encoding and so no longest sequence of its own
_NO_POSITION_LIMIT = 1 << 30


def fedolorn_spec(config: FedolornConfig) -> ModelSpec:
    width = config.width
    norm = PartSpec("rms_norm", {"size": width, "eps": config.norm_eps, "weight_offset": 1.0})
    layers: list[LayerSpec] = []
    rules: list[WeightRule] = [WeightRule("embed", "embed.weight")]
    for i, layer in enumerate(config.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        a = layer.mixer
        q_rows, k_rows, v_rows = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
        mixer = PartSpec(
            "gqa_attention",
            {
                "hidden_size": width,
                "num_heads": a.heads,
                "num_kv_heads": a.kv_heads,
                "head_dim": a.dim,
                "value_dim": a.vdim,
                "qkv_bias": False,
                "o_bias": False,
                "position": None,
                "scale": a.scale,
                "chunk": a.mask_size,
                "output_gate": True,
            },
        )
        rules += [
            WeightRule(src + "norm1", dst + "norm_input.weight"),
            WeightRule(src + "mix.q", dst + "mixer.qkv_weight", 0, q_rows),
            WeightRule(src + "mix.k", dst + "mixer.qkv_weight", q_rows, k_rows),
            WeightRule(src + "mix.v", dst + "mixer.qkv_weight", q_rows + k_rows, v_rows),
            WeightRule(src + "mix.g", dst + "mixer.gate_weight"),
            WeightRule(src + "mix.o", dst + "mixer.o_weight"),
        ]
        norms = {"input": norm}
        feed_forward = None
        m = layer.mlp
        if m is not None:
            norms["post_mixer"] = norm
            rules.append(WeightRule(src + "norm2", dst + "norm_post_mixer.weight"))
            ff = dst + "feed_forward."
            if m.kind == "dense":
                feed_forward = PartSpec("mlp", {"hidden_size": width, "intermediate_size": m.ff, "activation": "relu2"})
                rules += [WeightRule(src + "mlp.up", ff + "up_weight"), WeightRule(src + "mlp.down", ff + "down_weight")]
            else:
                feed_forward = PartSpec(
                    "routed_experts",
                    {
                        "hidden_size": width,
                        "intermediate_size": m.ff,
                        "experts": m.experts,
                        "top": m.top,
                        "router_scale": m.router_scale,
                        "groups": m.groups_count,
                        "keep_groups": m.groups_keep,
                        "activation": "relu2",
                    },
                )
                rules += [
                    WeightRule(src + "mlp.router", ff + "router_weight"),
                    WeightRule(src + "mlp.correction", ff + "correction"),
                ]
                for e in range(m.experts):
                    rules += [
                        WeightRule(f"{src}mlp.e{e}.up", ff + "up_weight", e * m.ff, m.ff),
                        WeightRule(f"{src}mlp.e{e}.down", ff + "down_weight", e * width, width),
                    ]
        layers.append(LayerSpec(block="pre_norm", mixer=mixer, feed_forward=feed_forward, norms=norms))
    rules.append(WeightRule("final.norm", "final_norm.weight"))
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        hidden_size=width,
        max_position_embeddings=_NO_POSITION_LIMIT,
        layers=tuple(layers),
        order=tuple(OrderEntry(i) for i in range(len(layers))),
        final_norm=norm,
        tie_word_embeddings=True,
        weight_rules=tuple(rules),
        embedding_scale=config.embedding_scale,
    )


register_architecture(FedolornConfig.architecture, FedolornConfig, fedolorn_spec, replace=True)
