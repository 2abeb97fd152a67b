"""A plain, slow implementation of the Fedolorn decoder: whole sequences, no cache, float64 or
float32 torch on the CPU, one function per mechanism.  It shares no code with the engine and is
what the engine's parts, kernels and schedules are compared with.

Notation: x is the residual stream [T, width]; h a normed input; positions count from 0.
A model is a dict `config` (the keys of the design's config.json) and a dict `weights`
(tensor name -> tensor, names as in the design's checkpoints).
"""

from __future__ import annotations

import math

import torch


def zero_centred_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * (1 + w): the stored weight is an offset from one."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + w)


def squared_relu(z: torch.Tensor) -> torch.Tensor:
    return torch.clamp(z, min=0.0) ** 2


def chunk_mask(positions: torch.Tensor, size: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j when j <= i and both lie in the same run of `size`
    positions counted from 0."""
    i = positions[:, None]
    j = positions[None, :]
    return (j <= i) & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))


def gated_chunk_attention(h: torch.Tensor, w: dict, m: dict) -> torch.Tensor:
    """h [T, width].  w: q, k, v, g, o.  m: heads, kv_heads, dim, vdim, scale, mask.size."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, G, d)
    v = (h @ w["v"].T).view(T, G, dv)
    gate = torch.sigmoid(h @ w["g"].T)  # [T, H * dv]
    mask = m.get("mask")
    pos = torch.arange(T)
    visible = chunk_mask(pos, int(mask["size"])) if mask else pos[None, :] <= pos[:, None]
    out = torch.empty(T, H, dv, dtype=h.dtype)
    for head in range(H):
        kv = head // (H // G)
        s = (q[:, head] @ k[:, kv].T) * m["scale"]
        s = s.masked_fill(~visible, -math.inf)
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, kv]
    return (out.reshape(T, H * dv) * gate) @ w["o"].T


def dense_feed_forward(h: torch.Tensor, w: dict) -> torch.Tensor:
    return squared_relu(h @ w["up"].T) @ w["down"].T


def route(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, r: dict):
    """Chosen experts [T, top] and their weights [T, top].  r: experts, top, scale, groups.count,
    groups.keep."""
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    n_groups, keep = groups["count"], groups["keep"]
    s = torch.sigmoid(h @ router.T)  # [T, E]
    choice = s + correction
    per = E // n_groups
    grouped = choice.view(-1, n_groups, per)
    group_score = grouped.topk(min(2, per), dim=-1).values.sum(-1)  # [T, groups]
    best = group_score.topk(keep, dim=-1).indices
    allowed = torch.zeros_like(group_score, dtype=torch.bool).scatter_(1, best, True)
    masked = choice.masked_fill(~allowed[:, :, None].expand(-1, -1, per).reshape(-1, E), -math.inf)
    chosen = masked.topk(top, dim=-1).indices
    return chosen, s.gather(1, chosen) * r["scale"]


def routed_feed_forward(h: torch.Tensor, w: dict, mlp: dict) -> torch.Tensor:
    """w: router, correction, e<i>.up, e<i>.down."""
    chosen, weight = route(h, w["router"], w["correction"], mlp["router"])
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(chosen.shape[1]):
            e = int(chosen[t, j])
            out[t] += weight[t, j] * (squared_relu(h[t] @ w[f"e{e}.up"].T) @ w[f"e{e}.down"].T)
    return out


def _sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config: dict, weights: dict, tokens, dtype=torch.float64, layers_out=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  `layers_out`: a list that receives the residual
    stream after every layer."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"unknown mixer {layer['type']!r}")
        p = f"l{i}."
        h = zero_centred_rms_norm(x, w[p + "norm1"], eps)
        x = x + gated_chunk_attention(h, _sub(w, p + "mix."), layer["mixer"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = zero_centred_rms_norm(x, w[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                x = x + dense_feed_forward(h, _sub(w, p + "mlp."))
            elif mlp["kind"] == "moe":
                x = x + routed_feed_forward(h, _sub(w, p + "mlp."), mlp)
            else:
                raise ValueError(f"unknown feed-forward {mlp['kind']!r}")
        if layers_out is not None:
            layers_out.append(x.clone())
    return zero_centred_rms_norm(x, w["final.norm"], eps) @ w["embed"].T
