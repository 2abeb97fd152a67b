"""A plain, slow implementation of the Bubitar decoder: whole sequences, no cache, no state carried
between calls, float64 torch on the CPU, one function per mechanism.  It shares no code with the
engine and is what the engine's parts, kernels and schedules are compared with.

Notation: x is the residual stream [T, width]; h a normed input; positions count from 0.
A model is a dict `config` (the keys of the design's config.json) and a dict `weights`
(tensor name -> tensor, names as in the design's checkpoints).

`rounded()` switches every matrix product to operands and results rounded to bfloat16 (everything
else stays float64): what rounding alone does to a row of logits, which is the yardstick for a
bfloat16 engine where a model is ill-conditioned (a sublayer's output near zero before its norm).
"""

from __future__ import annotations

import contextlib
import math

import torch

_ROUND = [False]


@contextlib.contextmanager
def rounded():
    _ROUND.append(True)
    try:
        yield
    finally:
        _ROUND.pop()


def _r(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).double() if _ROUND[-1] else t


def mm(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """a @ w^T, the one place where products happen."""
    return _r(_r(a) @ w.T)


def rms_norm(x: torch.Tensor, w, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps), times w unless w is None."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def rotary_frequencies(rot: dict) -> tuple[torch.Tensor, float]:
    """(frequency of every pair, amplitude of cosines and sines) of a rotation over rot["dims"] dims."""
    n, base = rot["dims"], rot["base"]
    pair = torch.arange(n // 2, dtype=torch.float64)
    f = base ** (-2.0 * pair / n)
    s = rot.get("scaling")
    if not s:
        return f, 1.0

    def pair_turning(times: float) -> float:
        return n * math.log(s["original"] / (2.0 * math.pi * times)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_turning(s["fast"])), 0)
    hi = min(math.ceil(pair_turning(s["slow"])), n - 1)
    ramp = torch.clamp((pair - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(s["factor"]) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, heads, d]: dims j and j + n/2 (j < n/2, n = rot["dims"]) turn by positions * f_j; the rest pass."""
    n = rot["dims"]
    f, amplitude = rotary_frequencies(rot)
    angle = positions.double()[:, None] * f[None, :]
    c = (torch.cos(angle) * amplitude)[:, None, :]
    s = (torch.sin(angle) * amplitude)[:, None, :]
    a, b = x[..., : n // 2], x[..., n // 2 : n]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., n:]], dim=-1)


def latent_cache(h: torch.Tensor, w: dict, m: dict, eps: float, positions: torch.Tensor):
    """(latents [T, kv_rank], rotated shared key part [T, rot_dim]) that a layer with `dkv` makes."""
    R = m["kv_rank"]
    down = mm(h, w["dkv"])
    return rms_norm(down[:, :R], w["dkv.norm"], eps), rotate(down[:, None, R:], positions, m["rot"])[:, 0]


def latent_attention(h: torch.Tensor, w: dict, m: dict, cache, positions: torch.Tensor) -> torch.Tensor:
    """h [T, width]; cache = (latents, rotated key part) of this layer or of the layer it reads."""
    T = h.shape[0]
    H, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    latent, shared = cache
    q = mm(h, w["q"]).view(T, H, d + r)
    q_plain, q_turned = q[..., :d], rotate(q[..., d:], positions, m["rot"])
    k_plain = mm(latent, w["uk"]).view(T, H, d)
    v = mm(latent, w["uv"]).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihr,jr->hij", q_turned, shared)) * m["scale"]
    seen = positions[None, :] <= positions[:, None]
    scores = scores.masked_fill(~seen, -math.inf)
    # the sink: one more term of the denominator, without key or value
    sink = w["sink"].double()
    top = torch.maximum(scores.max(-1).values, sink[:, None])
    e = torch.exp(scores - top[..., None])
    weights = e / (e.sum(-1) + torch.exp(sink[:, None] - top))[..., None]
    out = torch.einsum("hij,jhv->ihv", weights, v)
    out = out * torch.sigmoid(mm(h, w["g"]))[..., None]  # one gate per head and token
    return mm(out.reshape(T, H * dv), w["o"])


def retention(h: torch.Tensor, w: dict, m: dict, eps: float, positions: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = rotate(mm(h, w["q"]).view(T, H, d), positions, m["rot"])
    k = rotate(mm(h, w["k"]).view(T, H, d), positions, m["rot"]) * d**-0.5
    v = mm(h, w["v"]).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        state = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            state = m["decay"][head] * state + torch.outer(k[t, head], v[t, head])
            out[t, head] = state.T @ q[t, head]
    out = rms_norm(out, None, eps).reshape(T, H * dv)
    z = mm(h, w["g"])
    return mm(out * (z * torch.sigmoid(z)), w["o"])


def clamped_feed_forward(h: torch.Tensor, w: dict, m: dict) -> torch.Tensor:
    limit = m["limit"]
    g = torch.clamp(mm(h, w["gate"]) + w["gate.b"], max=limit)
    u = torch.clamp(mm(h, w["up"]) + w["up.b"], -limit, limit)
    return mm(g * torch.sigmoid(1.702 * g) * (u + 1.0), w["down"]) + w["down.b"]


def token_input(x: torch.Tensor, rows: torch.Tensor, w: dict) -> torch.Tensor:
    """rows: the layer's columns of the shared table at the tokens, [T, side dim]."""
    return mm(gelu_tanh(mm(x, w["gate"])) * rows, w["proj"])


def _sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v.double() for k, v in weights.items() if k.startswith(prefix)}


def forward(config: dict, weights: dict, tokens, layer_outputs=None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of one whole sequence."""
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    positions = torch.arange(len(ids))
    eps = config["norm"]["eps"]
    side = config["token_side"]["dim"]
    x = weights["embed"].double()[ids]
    caches: dict = {}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        norms = {n: weights[p + n].double() for n in ("norm1", "norm1b", "norm2", "norm2b") if p + n in weights}
        h = rms_norm(x, norms["norm1"], eps)
        mix = _sub(weights, p + "mix.")
        if layer["type"] == "latent_attention":
            if "kv_from" not in m:
                caches[i] = latent_cache(h, mix, m, eps, positions)
            y = latent_attention(h, mix, m, caches[m.get("kv_from", i)], positions)
        else:
            y = retention(h, mix, m, eps, positions)
        x = x + rms_norm(y, norms["norm1b"], eps)
        if layer["mlp"] is not None:
            y = clamped_feed_forward(rms_norm(x, norms["norm2"], eps), _sub(weights, p + "mlp."), layer["mlp"])
            x = x + rms_norm(y, norms["norm2b"], eps)
        sw = _sub(weights, p + "side.")
        rows = weights["side.embed"].double()[ids][:, i * side : (i + 1) * side]
        x = x + rms_norm(token_input(x, rows, sw), sw["norm"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return _r(rms_norm(x, weights["final.norm"].double(), eps)) @ weights["head"].double().T
