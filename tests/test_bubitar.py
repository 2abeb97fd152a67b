"""The Bubitar decoder in the engine against the plain implementation (`plain_bubitar.py`).

Each mechanism alone (normed additions, the clamped gating, the GELU product with a multiplier, scaled
rotary tables, per-head products, the retention scan with its state rows, one-layer models of either
mixer), keys placed so that one far score stands out, a sink that decides, then whole models under every
way of cutting and batching over poisoned pages and reused slots, replays against unrecorded steps, and
greedy generation through the engine, the command line and the replay program.  The tests make their own
small configurations and weights (larger than an initialisation would be, so that attention is peaked
and the clamps bite); sizes differ from layer to layer, also where a model could make them equal.

`double` cases run everything above the kernels on the CPU stand-in; `hip` cases run the HIP kernels
(`-m gpu`) in float32 and bfloat16.
"""

from __future__ import annotations

import json
import math
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

import mini_llm_runtime_amd.models  # noqa: F401
import plain_bubitar as plain
import schedules
from helpers import make_runner, random_tokens
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.config import BubitarConfig, ConfigError
from mini_llm_runtime_amd.engine import ContinuousBatchEngine
from mini_llm_runtime_amd.models import build_model, config_from_dict
from mini_llm_runtime_amd.weights import save_state_dict

ROOT = Path(__file__).resolve().parents[1]


# ---- configurations -----------------------------------------------------------------------------------

def _rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def _latent(heads, dim, rot_dim, vdim, rank, scale, rot, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return ("latent_attention", m)


def _retention(heads, dim, vdim, decay, rot):
    return ("retention", {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": rot})


def _ff(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _model(vocab, width, eps, side, layers):
    return {
        "architecture": "Bubitar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "token_side": {"dim": side},
        "layers": [{"type": kind, "mixer": m, "mlp": f} for (kind, m), f in layers],
    }


_YARN = (4.0, 64, 8.0, 2.0)  # stretches the slow pairs already at these short lengths
CONFIGS = {
    # both mixers, a cache read two layers later by a layer with other head counts, a partial rotation in
    # the retention layer, a layer without feed-forward
    "A": _model(300, 64, 1e-6, 8, [
        (_latent(4, 16, 8, 24, 40, 0.25, _rot(10000.0, 8, _YARN)), _ff(96, 0.8)),
        (_retention(2, 32, 16, (0.9, 0.99), _rot(500.0, 16)), _ff(80, 2.5)),
        (_latent(2, 24, 8, 8, 40, 0.2, _rot(10000.0, 8, _YARN), kv_from=0), None),
        (_retention(4, 16, 16, (1.0, 0.5, 0.97, 0.8), _rot(10000.0, 16)), None),
    ]),
    # sizes that the matrix-core kernels refuse: a width of 72, heads of 10 + 6 dims of which 4 turn, values
    # of 12, an odd side dim, an odd vocabulary, retention heads of 20 x 12
    "B": _model(257, 72, 1e-5, 5, [
        (_retention(3, 20, 12, (0.95, 0.9, 0.999), _rot(777.0, 20)), _ff(52, 1.3)),
        (_latent(3, 10, 6, 12, 20, 0.3, _rot(3000.0, 4)), _ff(45, 0.6)),
    ]),
    # matrix-core sizes: a cached row of 96 + 32 = 128, eight heads on it; retention heads of 64 x 32
    "C": _model(512, 128, 1e-5, 16, [
        (_latent(8, 32, 32, 32, 96, 0.12, _rot(1e6, 32, (8.0, 128, 16.0, 1.5))), _ff(192, 1.0)),
        (_retention(4, 64, 32, (0.97, 0.99, 0.995, 0.999), _rot(1e6, 64)), _ff(160, 3.0)),
        (_latent(4, 64, 32, 16, 96, 0.1, _rot(1e6, 32, (8.0, 128, 16.0, 1.5)), kv_from=0), _ff(128, 1.0)),
    ]),
    # long requests: hundreds of keys (the decode kernel's partitions and their merge, several key tiles of
    # the prompt kernel), states that carry over hundreds of tokens
    "D": _model(200, 128, 1e-5, 12, [
        (_retention(2, 64, 64, (0.999, 0.98), _rot(10000.0, 32)), None),
        (_latent(4, 32, 16, 48, 64, 0.15, _rot(10000.0, 16, (8.0, 256, 32.0, 1.0))), _ff(96, 1.2)),
    ]),
    # one layer of each mixer and nothing else: what a mixer does is not blurred by the other
    "L": _model(128, 64, 1e-6, 4, [(_latent(2, 16, 16, 32, 32, 0.3, _rot(10000.0, 16, _YARN)), None)]),
    # a cached row wider than the matrix-core attention kernels take (272 + 16 = 288): the plain kernel runs it
    "W": _model(96, 64, 1e-6, 4, [(_latent(3, 16, 16, 24, 272, 0.2, _rot(10000.0, 16)), _ff(48, 1.5))]),
    "R": _model(128, 64, 1e-6, 4, [(_retention(2, 16, 32, (0.9, 0.995), _rot(10000.0, 8)), None)]),
}
BLOCK = {"A": 16, "B": 8, "C": 16, "D": 16, "L": 8, "R": 4, "W": 16}
LENGTHS = {
    "A": (1, 9, 50, 83, 37, 64), "B": (2, 19, 35, 66, 45), "C": (5, 17, 140, 70, 97), "D": (660, 341),
    "L": (1, 24, 75, 41, 130), "R": (1, 24, 75, 41, 130), "W": (3, 70, 41),
}


def make_weights(cfg: dict, seed: int) -> dict[str, torch.Tensor]:
    """bfloat16 tensors by the design's checkpoint names."""
    g = torch.Generator().manual_seed(seed)
    width, side = cfg["width"], cfg["token_side"]["dim"]

    def normal(*shape, std, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16)

    w = {
        "embed": normal(cfg["vocab"], width, std=1.0),
        "side.embed": normal(cfg["vocab"], len(cfg["layers"]) * side, std=1.0),
        "final.norm": normal(width, std=0.2, mean=1.0),
        "head": normal(cfg["vocab"], width, std=1.0 / math.sqrt(width)),
    }
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm1b"):
            w[p + n] = normal(width, std=0.2, mean=1.0)
        out = m["heads"] * m["vdim"]
        if layer["type"] == "retention":
            w[p + "mix.q"] = normal(m["heads"] * m["dim"], width, std=1.0 / math.sqrt(width))
            w[p + "mix.k"] = normal(m["heads"] * m["dim"], width, std=1.0 / math.sqrt(width))
            w[p + "mix.v"] = normal(out, width, std=1.0 / math.sqrt(width))
            w[p + "mix.g"] = normal(out, width, std=1.5 / math.sqrt(width))
        else:
            # queries and keys large enough for peaked attention, sinks that take a visible share
            w[p + "mix.q"] = normal(m["heads"] * (m["dim"] + m["rot_dim"]), width, std=2.0 / math.sqrt(width))
            if "kv_from" not in m:
                w[p + "mix.dkv"] = normal(m["kv_rank"] + m["rot_dim"], width, std=2.0 / math.sqrt(width))
                w[p + "mix.dkv.norm"] = normal(m["kv_rank"], std=0.2, mean=1.0)
            w[p + "mix.uk"] = normal(m["heads"] * m["dim"], m["kv_rank"], std=2.0 / math.sqrt(m["kv_rank"]))
            w[p + "mix.uv"] = normal(out, m["kv_rank"], std=1.0 / math.sqrt(m["kv_rank"]))
            w[p + "mix.sink"] = normal(m["heads"], std=1.5, mean=1.0)
            w[p + "mix.g"] = normal(m["heads"], width, std=1.5 / math.sqrt(width))
        w[p + "mix.o"] = normal(width, out, std=1.0 / math.sqrt(out))
        f = layer["mlp"]
        if f is not None:
            for n in ("norm2", "norm2b"):
                w[p + n] = normal(width, std=0.2, mean=1.0)
            w[p + "mlp.gate"] = normal(f["ff"], width, std=1.5 / math.sqrt(width))
            w[p + "mlp.up"] = normal(f["ff"], width, std=1.5 / math.sqrt(width))
            w[p + "mlp.down"] = normal(width, f["ff"], std=1.0 / math.sqrt(f["ff"]))
            w[p + "mlp.gate.b"] = normal(f["ff"], std=0.3)
            w[p + "mlp.up.b"] = normal(f["ff"], std=0.3)
            w[p + "mlp.down.b"] = normal(width, std=0.3)
        w[p + "side.gate"] = normal(side, width, std=1.0 / math.sqrt(width))
        w[p + "side.proj"] = normal(width, side, std=1.0 / math.sqrt(side))
        w[p + "side.norm"] = normal(width, std=0.2, mean=1.0)
    return w


def write_model(tmp_path, name: str, cfg: dict, weights: dict) -> Path:
    folder = Path(tmp_path) / name
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_state_dict(folder / "model.safetensors", weights)
    return folder


def make_dir(tmp_path, which: str, seed: int = 3) -> tuple[Path, dict, dict]:
    cfg = CONFIGS[which]
    weights = make_weights(cfg, seed)
    return write_model(tmp_path, f"bubitar{which}", cfg, weights), cfg, weights


def _ops(backend: str, dtype: torch.dtype):
    if backend == "double":
        return TorchOps(dtype, "cpu")
    from mini_llm_runtime_amd.kernels.ops import HipOps

    return HipOps(dtype, "cuda")


CASES = [
    pytest.param("double", torch.float32, id="double-f32"),
    pytest.param("hip", torch.float32, id="hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip", torch.bfloat16, id="hip-bf16", marks=pytest.mark.gpu),
]
GPU_CASES = [
    pytest.param(torch.float32, id="f32", marks=pytest.mark.gpu),
    pytest.param(torch.bfloat16, id="bf16", marks=pytest.mark.gpu),
]


def _compare(got, requests, weights, cfg, dtype, f32_bound=1e-4, row_bound=6e-2, together=2.5e-2):
    """float32: every value within 1e-4 of the logits' size.  bfloat16: all rows together within 2.5 %
    (relative L2); every row within 6 %, but for a few (one in twenty, and as many as rounding alone puts
    beyond 6 %) that may be off by up to 4 times what rounding alone does to the worst row of their request
    (the plain implementation with its products rounded to bfloat16).  A sublayer's output passes a norm before it is added, so where that output is
    near zero, or where a sink and one or two keys share the weight, every rounding moves the row by a
    percent, in the plain implementation as in the engine, and the worst row of hundreds is one where
    they all push the same way: the same rows stand out under every schedule.  A wrong key, page, slot or
    state changes a row by half and more, and most rows."""
    assert got, "no logits came back"
    num = den = 0.0
    loose = rows = loose_alone = 0
    for rid, toks in requests.items():
        ref = plain.forward(cfg, weights, toks)
        size = float(ref.pow(2).mean().sqrt())
        if dtype != torch.float32:
            with plain.rounded():
                coarse = plain.forward(cfg, weights, toks)
            alone = (coarse - ref).pow(2).sum(-1).sqrt() / ref.pow(2).sum(-1).sqrt()
            loose_alone += int((alone >= row_bound).sum())
        for pos in range(len(toks)):
            row = got[(rid, pos)].double()
            assert torch.isfinite(row).all(), f"{rid}:{pos} is not finite"
            diff = row - ref[pos]
            if dtype == torch.float32:
                assert float(diff.abs().max()) < f32_bound * size, f"{rid}:{pos}: off by {float(diff.abs().max()):.3e}"
                continue
            rows += 1
            rel = float(diff.pow(2).sum().sqrt() / ref[pos].pow(2).sum().sqrt())
            if rel >= row_bound:
                loose += 1
                assert rel < 4.0 * float(alone.max()), f"{rid}:{pos}: relative error {rel:.3e}, rounding alone up to {float(alone.max()):.3e}"
                continue
            num += float(diff.pow(2).sum())
            den += float(ref[pos].pow(2).sum())
    if dtype != torch.float32:
        # (as many as rounding alone puts beyond the bound, and a few)
        assert loose <= 0.05 * rows + 1 + 1.5 * loose_alone, f"{loose} of {rows} rows are off by more than {row_bound}, {loose_alone} by rounding alone"
        assert (num / den) ** 0.5 < together, f"relative error of all rows {(num / den) ** 0.5:.3e}"


def _requests(which: str) -> dict[str, list[int]]:
    vocab = CONFIGS[which]["vocab"]
    return {f"r{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate(LENGTHS[which])}


# ---- configuration and model --------------------------------------------------------------------------

def test_config_reads_every_layer_by_itself():
    c = config_from_dict(CONFIGS["A"])
    assert isinstance(c, BubitarConfig)
    assert [l.mixer.kind for l in c.layers] == ["latent_attention", "retention", "latent_attention", "retention"]
    assert c.layers[2].mixer.kv_from == 0 and c.layers[0].mixer.kv_from is None
    assert c.layers[0].mixer.rot.scaling.factor == 4.0 and c.layers[1].mixer.rot.scaling is None
    assert c.layers[1].mixer.decay == (0.9, 0.99) and c.layers[1].mlp.limit == 2.5 and c.layers[3].mlp is None
    assert c.token_side_dim == 8
    assert BubitarConfig.from_dict(c.to_dict()) == c


@pytest.mark.parametrize(
    "change",
    [
        lambda c: c["layers"][0]["mixer"].pop("kv_rank"),
        lambda c: c["layers"][0].update(type="convolution"),
        lambda c: c["layers"][1]["mixer"].update(decay=[0.9]),  # one decay for two heads
        lambda c: c["layers"][1]["mixer"]["rot"].update(dims=40),  # more than a head has
        lambda c: c["layers"][2]["mixer"].update(kv_from=1),  # a retention layer has no latents
        lambda c: c["layers"][2]["mixer"].update(kv_rank=48),  # another rank than the cache it reads
        lambda c: c["layers"][0]["mixer"].update(kv_from=2),  # a later layer
        lambda c: c["layers"][0]["mlp"].update(kind="moe"),
        lambda c: c.pop("token_side"),
    ],
)
def test_config_refuses_what_does_not_fit(change):
    cfg = json.loads(json.dumps(CONFIGS["A"]))
    change(cfg)
    with pytest.raises(ConfigError):
        config_from_dict(cfg)


def test_model_is_built_from_the_framework_parts():
    from mini_llm_runtime_amd.cache import PagedKVSpec, SlotStateSpec

    model = build_model(config_from_dict(CONFIGS["A"]))
    kinds = [(type(l).__name__, type(l.mixer).__name__, type(l.feed_forward).__name__) for l in model.layers]
    assert kinds == [
        ("SandwichNormBlock", "LatentAttention", "ClampedGLU"), ("SandwichNormBlock", "Retention", "ClampedGLU"),
        ("SandwichNormBlock", "LatentAttention", "NoneType"), ("SandwichNormBlock", "Retention", "NoneType"),
    ]
    assert model.replayable and model.splittable
    specs = model.site_cache_specs()
    assert specs[0] == PagedKVSpec(1, 48) and specs[2] is None  # 40 + 8 in one row; the third layer reads the first's
    assert specs[1] == SlotStateSpec((2, 32, 16), "float32") and specs[3] == SlotStateSpec((4, 16, 16), "float32")
    assert model.cache_site_of(2) == 0
    names = set(model.param_specs())
    assert "layers.2.mixer.latent_norm_weight" not in names and "layers.0.mixer.latent_norm_weight" in names
    assert model.param_specs()["layers.1.token_input.table"].shape == (300, 8)


def test_scaled_rotation_frequencies():
    from mini_llm_runtime_amd.parts import build_part
    from mini_llm_runtime_amd.parts.spec import PartSpec

    for rot in (_rot(10000.0, 8, _YARN), _rot(1e6, 32, (8.0, 128, 16.0, 1.5)), _rot(10000.0, 16, (8.0, 256, 32.0, 1.0)),
                _rot(500.0, 16)):
        scaling = rot.get("scaling")
        part = build_part("position", PartSpec("rotary", {"head_dim": rot["dims"], "theta": rot["base"], "scaling": scaling}))
        f, amplitude = plain.rotary_frequencies(rot)
        torch.testing.assert_close(torch.from_numpy(part._inv_freq_host), f, rtol=1e-14, atol=0)
        assert abs(part.amplitude - amplitude) < 1e-15
        if scaling:  # the fastest pair keeps its frequency, the slowest is stretched by the whole factor
            plain_f, _ = plain.rotary_frequencies({"base": rot["base"], "dims": rot["dims"]})
            assert float(f[0]) == float(plain_f[0]) and abs(float(f[-1] * scaling["factor"] / plain_f[-1]) - 1) < 1e-12


# ---- mechanisms alone, on the GPU ----------------------------------------------------------------------

def _tolerance(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("rows,size,slices", [(1, 64, 0), (7, 100, 3), (300, 192, 0), (3, 2048, 2), (5, 72, 1), (4, 70, 2), (2, 8196, 1), (8, 3584, 11), (70, 4096, 0)])
def test_normed_addition(dtype, rows, size, slices):
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(rows + size)
    x = torch.randn(rows, size, generator=g) * 3.0
    w = (1.0 + 0.3 * torch.randn(size, generator=g)).to(dtype)
    w_next = 1.0 + 0.3 * torch.randn(size, generator=g)  # a 32-bit weight beside one in the engine's dtype
    if slices:
        y = torch.randn(slices, rows, size, generator=g)
        total = y.double().sum(0)
    else:
        y = (torch.randn(rows, size, generator=g) * 5.0).to(dtype)
        total = y.double()
    added = x.double() + plain.rms_norm(total, w.double(), 1e-5)
    for kind in ("norm", "cast", "none"):
        stream = x.clone().cuda()
        got = ops.add_normed(
            stream, y.cuda(), w.cuda(), 1e-5, next_weight=w_next.cuda() if kind == "norm" else None, next_eps=1e-6,
            cast=kind == "cast",
        )
        torch.testing.assert_close(stream.cpu().double(), added, rtol=1e-5, atol=1e-5)  # the 32-bit sum
        if kind == "none":
            assert got is None
            continue
        want = plain.rms_norm(added, w_next.double(), 1e-6) if kind == "norm" else added
        assert got.dtype == dtype
        torch.testing.assert_close(got.double().cpu(), want, **_tolerance(dtype))


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("rows,inner,limit", [(1, 40, 1.0), (33, 52, 0.6), (300, 256, 2.5)])
def test_clamped_gating(dtype, rows, inner, limit):
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(rows + inner)
    sums = torch.randn(rows, 2 * inner, generator=g) * 2.0
    got = ops.glu_clamped(sums.cuda(), limit)
    gate = torch.clamp(sums[:, :inner].double(), max=limit)
    up = torch.clamp(sums[:, inner:].double(), -limit, limit)
    assert float((sums[:, :inner] < -limit).float().mean()) > 0.02  # the gate has no lower clamp: such values must pass
    torch.testing.assert_close(got.double().cpu(), gate * torch.sigmoid(1.702 * gate) * (up + 1.0), **_tolerance(dtype))


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("m,inner,k,limit", [(1, 40, 64, 1.0), (5, 26, 72, 0.6), (33, 128, 100, 2.5), (300, 256, 128, 1.0), (64, 640, 256, 1.5), (2048, 320, 512, 0.9)])
def test_clamped_gating_as_the_epilogue_of_its_product(dtype, m, inner, k, limit):
    """Gate and up rows woven in pairs, the biases with them; every product kernel that a shape may choose."""
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(m + inner + k)
    x = torch.randn(m, k, generator=g).to(dtype)
    wg = (torch.randn(inner, k, generator=g) * 2.0 / math.sqrt(k)).to(dtype)
    wu = (torch.randn(inner, k, generator=g) * 2.0 / math.sqrt(k)).to(dtype)
    bg, bu = torch.randn(inner, generator=g) * 0.5, torch.randn(inner, generator=g) * 0.5
    woven = torch.stack([wg.view(-1, 2, k), wu.view(-1, 2, k)], dim=1).reshape(2 * inner, k).contiguous()
    bias = torch.stack([bg.view(-1, 2), bu.view(-1, 2)], dim=1).reshape(2 * inner).contiguous()
    got = ops.linear(x.cuda(), woven.cuda(), bias.cuda(), clamped_glu=(limit, 1.702))
    gate = torch.clamp(x.double() @ wg.double().T + bg.double(), max=limit)
    up = torch.clamp(x.double() @ wu.double().T + bu.double(), -limit, limit)
    assert got.shape == (m, inner) and got.dtype == dtype
    torch.testing.assert_close(got.double().cpu(), gate * torch.sigmoid(1.702 * gate) * (up + 1.0), **_tolerance(dtype))


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("m,n,k", [(1, 8, 64), (5, 5, 72), (33, 16, 100), (300, 12, 128)])
def test_gelu_product_with_gathered_rows(dtype, m, n, k):
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(m * n + k)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = (torch.randn(n, k, generator=g) * 2.0 / math.sqrt(k)).to(dtype)
    table = torch.randn(50, n, generator=g).to(dtype)
    ids = torch.randint(0, 50, (m,), generator=g).to(torch.int32)
    rows = ops.embedding(table.cuda(), ids.cuda(), out_dtype=dtype)
    assert rows.dtype == dtype and torch.equal(rows.cpu(), table[ids.long()])
    got = ops.linear(x.cuda(), w.cuda(), None, activation="gelu_tanh", multiply=rows)
    want = plain.gelu_tanh(x.double() @ w.double().T) * table[ids.long()].double()
    torch.testing.assert_close(got.double().cpu(), want, **_tolerance(dtype))
    # the same with the rows gathered inside the product's epilogue
    inside = ops.linear(x.cuda(), w.cuda(), None, activation="gelu_tanh", multiply=table.cuda(), multiply_rows=ids.cuda())
    assert torch.equal(inside, got)


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("tokens,heads,n,k,stride", [(1, 2, 40, 16, 16), (70, 3, 20, 10, 10), (130, 8, 32, 96, 128), (9, 4, 100, 64, 80), (5, 2, 24, 40, 48), (300, 3, 70, 72, 72)])
def test_products_with_a_matrix_per_head(dtype, tokens, heads, n, k, stride):
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(tokens + heads)
    x = torch.randn(tokens, heads * stride, generator=g).to(dtype)
    w = (torch.randn(heads, n, k, generator=g) / math.sqrt(k)).to(dtype)
    scale = torch.rand(tokens, heads, generator=g)
    ref = torch.einsum("thk,hnk->thn", x.view(tokens, heads, stride)[..., :k].double(), w.double())
    got = ops.heads_linear(x.cuda(), w.cuda(), in_stride=stride, row_scale=scale.cuda())
    torch.testing.assert_close(got.double().cpu().view(tokens, heads, n), ref * scale.double()[..., None], **_tolerance(dtype))
    # into the leading columns of wider rows, the rest untouched
    wide = torch.full((tokens, heads * (n + 7)), 3.0).to(dtype).cuda()
    ops.heads_linear(x.cuda(), w.cuda(), in_stride=stride, out=wide, out_stride=n + 7)
    wide = wide.double().cpu().view(tokens, heads, n + 7)
    torch.testing.assert_close(wide[..., :n], ref, **_tolerance(dtype))
    assert bool((wide[..., n:] == 3.0).all())


@pytest.mark.gpu
@pytest.mark.parametrize("chunked", [False, True], ids=["by-token", "by-chunk"])
@pytest.mark.parametrize("heads,dim,vdim,rdims", [(2, 16, 32, 8), (3, 20, 12, 20), (4, 64, 48, 64), (1, 128, 16, 0), (2, 200, 20, 100)])
def test_retention_scan_and_its_state_rows(heads, dim, vdim, rdims, chunked):
    """Three entries of unequal length (one token, less than a chunk of 64, two chunks and a bit), two of
    which go on from a carried state; rows of other slots stay.  Token by token and in chunks."""
    ops = _ops("hip", torch.float32)
    g = torch.Generator().manual_seed(heads * dim + vdim)
    lens, starts = [5, 1, 150], [0, 40, 7]
    tokens = sum(lens)
    width = 2 * heads * dim + 2 * heads * vdim
    p = torch.randn(tokens, width, generator=g)
    decay = torch.tensor([0.9, 0.99, 1.0, 0.0][:heads])  # also a head that forgets at once
    rot = {"base": 100.0, "dims": rdims}
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)])
    bank = torch.randn(10, heads, dim, vdim, generator=g)  # stale values everywhere
    read, write = [0, 3, 4], [1, 2, 5]
    rotation = None
    if rdims:
        f, _ = plain.rotary_frequencies(rot)
        angle = positions.double()[:, None] * f[None, :]
        rotation = (angle.cos().float().cuda(), angle.sin().float().cuda(), rdims)
    state = bank.clone().cuda()
    cu = torch.tensor([0, 5, 6, 156], dtype=torch.int32)
    ctx = SimpleNamespace(num_entries=3, cu_q=cu.cuda(), q_starts=torch.tensor(starts, dtype=torch.int32).cuda())
    out = ops.retention_scan(
        p.cuda(), state, torch.tensor(read, dtype=torch.int32).cuda(), torch.tensor(write, dtype=torch.int32).cuda(), ctx,
        heads=heads, head_dim=dim, value_dim=vdim, decay=decay.cuda(), key_scale=dim**-0.5, rotation=rotation,
        chunked=chunked,
    )
    qk = heads * dim
    for r in range(3):
        a, b = int(cu[r]), int(cu[r + 1])
        rows = p[a:b].double()
        q = rows[:, :qk].view(-1, heads, dim)
        k = rows[:, qk : 2 * qk].view(-1, heads, dim)
        if rdims:
            q, k = plain.rotate(q, positions[a:b], rot), plain.rotate(k, positions[a:b], rot)
        v = rows[:, 2 * qk : 2 * qk + heads * vdim].view(-1, heads, vdim)
        s = bank[read[r]].double() if starts[r] > 0 else torch.zeros(heads, dim, vdim, dtype=torch.float64)
        for t in range(b - a):
            s = decay.double()[:, None, None] * s + (k[t] * dim**-0.5)[:, :, None] * v[t][:, None, :]
            want = torch.einsum("hdv,hd->hv", s, q[t]).reshape(-1)
            torch.testing.assert_close(out[a + t].double().cpu(), want, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(state[write[r]].double().cpu(), s, rtol=1e-4, atol=1e-4)
    for row in set(range(10)) - set(write):
        assert torch.equal(state[row].cpu(), bank[row]), f"row {row} was written"
    # the heads' norm and the gate
    gated = ops.retention_gate(out, p.cuda(), heads=heads, value_dim=vdim, gate_offset=2 * qk + heads * vdim, eps=1e-5)
    z = p[:, 2 * qk + heads * vdim :].double()
    want = plain.rms_norm(out.double().cpu().view(tokens, heads, vdim), None, 1e-5).reshape(tokens, -1) * (z * torch.sigmoid(z))
    torch.testing.assert_close(gated.double().cpu(), want, rtol=1e-4, atol=1e-4)


# ---- one far key, a sink that decides, a state that must not be lost -------------------------------------

def _needle_model(rank: int, dim: int, rot_dim: int, vdim: int, sink: float) -> tuple[dict, dict]:
    """One latent-attention layer with one head, made so that a query's weight sits on ONE key wherever
    it lies: token 1 marks a key, token 2 asks, every other token is filler.  The marked key's value goes
    into the logits, so they say whether that key was seen."""
    width = 16
    cfg = _model(8, width, 1e-6, 2, [(_latent(1, dim, rot_dim, vdim, rank, 1.0, _rot(10000.0, rot_dim)), None)])
    g = torch.Generator().manual_seed(rank + dim)
    w = {k: v.float() for k, v in make_weights(cfg, 5).items()}
    w["embed"] = torch.zeros(8, width)
    w["embed"][:, :8] = torch.eye(8) * 4.0
    w["l0.norm1"] = torch.ones(width)
    q = torch.zeros(dim + rot_dim, width)
    q[0, 2] = 8.0  # the unrotated query of token 2 ...
    dkv = torch.randn(rank + rot_dim, width, generator=g) * 0.05
    dkv[rank:] = 0.0  # no rotated key part: the place of the key must not matter
    dkv[0, 1] = 8.0  # ... meets the latent of token 1 through Wuk
    uk = torch.zeros(dim, rank)
    uk[0, 0] = 4.0
    w["l0.mix.q"], w["l0.mix.dkv"], w["l0.mix.uk"] = q, dkv, uk
    w["l0.mix.dkv.norm"] = torch.ones(rank)
    w["l0.mix.uv"] = torch.randn(vdim, rank, generator=g) * 0.5
    w["l0.mix.g"] = torch.zeros(1, width)
    w["l0.mix.sink"] = torch.tensor([sink])
    w["l0.mix.o"] = torch.randn(width, vdim, generator=g) * 0.5
    return cfg, {name: t.to(torch.bfloat16) for name, t in w.items()}


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("rank,dim,rot_dim,vdim,length,marked", [(24, 16, 8, 16, 70, 0), (48, 32, 16, 24, 200, 15), (96, 16, 32, 32, 700, 16), (40, 8, 8, 12, 131, 63)])
def test_one_far_key_among_many(tmp_path, backend, dtype, rank, dim, rot_dim, vdim, length, marked):
    """The marked key lies at the very first position, at a page's last and first slot, hundreds of keys
    back; queries at the end of a prompt, of a portion, and decoded alone."""
    if backend == "double" and length > 150:
        pytest.skip("the CPU stand-in is slow at this length")
    cfg, weights = _needle_model(rank, dim, rot_dim, vdim, sink=-2.0)
    folder = write_model(tmp_path, "needle", cfg, weights)
    cases = {}
    for name, token in (("marked", 1), ("unmarked", 3)):
        toks = [3 + (i % 5) for i in range(length)]
        toks[marked] = token
        toks[-1] = 2
        cases[name] = toks
    ops = _ops(backend, dtype)
    _, _, cache, runner = make_runner(folder, ops, block_size=16, num_blocks=2 * (length // 16 + 2), max_requests=2)
    cache.poison()
    for family in (schedules.whole, lambda r: schedules.bulk_then_tail(r, tail=5), schedules.portions):
        got = schedules.run_schedule(runner, cache, family(cases))
        for name, toks in cases.items():
            ref = plain.forward(cfg, weights, toks)[-1]
            row = got[(name, length - 1)].double()
            assert float((row - ref).abs().max()) < (1e-4 if dtype == torch.float32 else 0.08) * float(ref.abs().max())
        seen = got[("marked", length - 1)]
        assert float((seen - got[("unmarked", length - 1)]).abs().max()) > 0.3 * float(seen.abs().max())


@pytest.mark.parametrize("backend,dtype", CASES)
def test_sinks_that_take_most_of_one_head(tmp_path, backend, dtype):
    """Two heads, one of which loses most of its weight to its sink.  (A mixer's output is normed before
    it is added, so one head's sink alone would cancel: it is the balance between the heads that shows.)
    Left out, swapped between the heads, or counted once per partition of the keys, the logits differ."""
    length = 330
    cfg = _model(96, 32, 1e-6, 2, [(_latent(2, 16, 8, 16, 24, 0.2, _rot(10000.0, 8)), None)])
    toks = random_tokens(length, 96, 21)
    results = {}
    for sinks in ((25.0, -25.0), (-25.0, 25.0)):
        weights = make_weights(cfg, 13)
        weights["l0.mix.sink"] = torch.tensor(sinks).to(torch.bfloat16)
        ref = results[sinks] = plain.forward(cfg, weights, toks)[-1]
        if backend == "double" and sinks[0] < 0:
            continue
        folder = write_model(tmp_path, f"sink{int(sinks[0])}", cfg, weights)
        ops = _ops(backend, dtype)
        _, _, cache, runner = make_runner(folder, ops, block_size=16, num_blocks=length // 16 + 2, max_requests=1)
        for family in (schedules.whole, lambda r: schedules.bulk_then_tail(r, tail=3)):
            got = schedules.run_schedule(runner, cache, family({"a": toks}))
            row = got[("a", length - 1)].double()
            assert float((row - ref).abs().max()) < (1e-4 if dtype == torch.float32 else 0.08) * float(ref.abs().max())
    a, b = results.values()
    assert float((a - b).abs().max()) > 0.2 * float(a.abs().max())


@pytest.mark.parametrize("backend,dtype", CASES)
def test_a_state_that_remembers_the_first_token(tmp_path, backend, dtype):
    """A retention head that does not decay: the first token's key and value stay in the state for good, so
    a state lost between two steps, or a slot cleared too late, shows at every later position."""
    cfg = _model(64, 32, 1e-6, 2, [(_retention(2, 8, 16, (1.0, 0.9), _rot(10000.0, 4)), None)])
    weights = make_weights(cfg, 11)
    folder = write_model(tmp_path, "keeper", cfg, weights)
    a = random_tokens(90, 64, 1)
    b = [(a[0] + 1) % 64] + a[1:]  # differs in the first token only
    ref_a, ref_b = plain.forward(cfg, weights, a), plain.forward(cfg, weights, b)
    # the oracle remembers: clearly at the twentieth token (where a portion or the bulk's end may fall), still at the last
    assert float((ref_a[20] - ref_b[20]).abs().max()) > 0.1 * float(ref_a[20].abs().max())
    assert float((ref_a[-1] - ref_b[-1]).abs().max()) > 0.01 * float(ref_a[-1].abs().max())
    ops = _ops(backend, dtype)
    _, _, cache, runner = make_runner(folder, ops, block_size=8, num_blocks=1, max_requests=1)
    for family in (schedules.whole, lambda r: schedules.bulk_then_tail(r, tail=40), schedules.portions):
        for name, toks in (("a", a), ("b", b), ("a", a)):  # one slot, used again and again
            got = schedules.run_schedule(runner, cache, family({name: toks}))
            _compare(got, {name: toks}, weights, cfg, dtype)


# ---- whole models under every schedule -------------------------------------------------------------------

FAMILIES = {
    "whole": schedules.whole,
    "bulk_then_tail": lambda r: schedules.bulk_then_tail(r, tail=48),
    "portions": schedules.portions,
    "mixed": schedules.mixed,
    "mixed_two_slots": lambda r: schedules.mixed(r, max_live=2, seed=5, decode_tail=20),
}


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("which", list(CONFIGS))
def test_schedule_matches_plain(tmp_path, which, family, backend, dtype):
    if backend == "double" and (which == "D" or (which == "C" and family != "mixed")):
        pytest.skip("the CPU stand-in is slow at this size")
    folder, cfg, weights = make_dir(tmp_path, which)
    requests = _requests(which)
    steps = FAMILIES[family](requests)
    bs = BLOCK[which]
    _, model, cache, runner = make_runner(
        folder, _ops(backend, dtype), block_size=bs, num_blocks=max(1, schedules.pages_needed(steps, bs)),
        max_requests=schedules.most_live(steps),
    )
    cache.poison()
    for bank in cache.state_banks.values():  # stale states in every slot: a request must start from zeros
        bank.tensor.fill_(float("nan"))
    got = schedules.run_schedule(runner, cache, steps)
    _compare(got, requests, weights, cfg, dtype)
    cache.check_invariants()
    assert all(g.allocator.free_count == g.num_blocks for g in cache.groups), "pages were not given back"


def test_layer_outputs_match_plain(tmp_path):
    folder, cfg, weights = make_dir(tmp_path, "A")
    toks = random_tokens(31, cfg["vocab"], 8)
    _, _, cache, runner = make_runner(folder, _ops("double", torch.float32), block_size=16, num_blocks=4, max_requests=1)
    cache.create_request("a")
    from helpers import StepEntry

    out = runner.step([StepEntry.of("a", toks, [0, 17, 30])], capture_sites=True)
    layers = []
    plain.forward(cfg, weights, toks, layers)
    assert out.site_outputs.shape == (4, 3, cfg["width"])
    for i, x in enumerate(layers):
        torch.testing.assert_close(out.site_outputs[i].double(), x[[0, 17, 30]], rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", GPU_CASES)
def test_replayed_steps_equal_plain_steps(tmp_path, dtype):
    """Steps of a model with state slots and a shared cache are recorded and replayed; the replays give
    what the unrecorded steps give, bit for bit."""
    folder, cfg, _ = make_dir(tmp_path, "C")
    requests = {"a": random_tokens(90, cfg["vocab"], 1), "b": random_tokens(75, cfg["vocab"], 2)}
    steps = schedules.bulk_then_tail(requests, tail=40)
    results = []
    for use_graphs in (False, True):
        _, _, cache, runner = make_runner(folder, _ops("hip", dtype), block_size=16, num_blocks=16, max_requests=2)
        runner.use_graphs = use_graphs
        results.append(schedules.run_schedule(runner, cache, steps))
    plain_steps, replayed = results
    assert plain_steps.keys() == replayed.keys()
    for key in plain_steps:
        assert torch.equal(plain_steps[key], replayed[key]), key


# ---- generation through the engine ------------------------------------------------------------------------

@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_through_the_engine(tmp_path, which, backend, dtype):
    folder, cfg, weights = make_dir(tmp_path, which)
    ops = _ops(backend, dtype)
    engine = ContinuousBatchEngine.from_model_dir(
        folder, dtype=ops.dtype, ops=ops, block_size=BLOCK[which], num_blocks=40, max_running_requests=3,
        max_batch_tokens=24,
    )
    prompts = [random_tokens(n, cfg["vocab"], 9 + n) for n in (5, 30, 1, 17)]
    outs = engine.generate(prompts, max_new_tokens=40)  # long enough to pass page borders while decoding
    for prompt, tokens in zip(prompts, outs):
        assert len(tokens) == 40
        seq = list(prompt)
        for i, tok in enumerate(tokens):
            logits = plain.forward(cfg, weights, seq)[-1]
            best = int(torch.argmax(logits))
            if tok != best:
                # only rounding may choose between two nearly equal logits, and only in bfloat16
                assert dtype == torch.bfloat16, f"token {i}: {tok} != {best}"
                assert float(logits[best] - logits[tok]) < 6e-2 * float(logits.abs().max())
                break
            seq.append(tok)


# ---- the command line and the replay program --------------------------------------------------------------

def test_preset_and_random_model_writer(tmp_path):
    from helpers import read_weights
    from mini_llm_runtime_amd import cli
    from mini_llm_runtime_amd.config.presets import preset_names

    assert "bubitar-tiny" in preset_names()
    assert cli.main(["random-model", "--config", "bubitar-tiny", "--seed", "2", "--out", str(tmp_path / "m")]) == 0
    cfg, w = read_weights(tmp_path / "m")
    assert cfg["architecture"] == "Bubitar" and w["embed"].shape == (320, 96) and w["side.embed"].shape == (320, 24)
    assert w["l0.mix.dkv"].shape == (64, 96) and "l2.mix.dkv" not in w and "l2.norm2" not in w
    assert w["l1.mlp.gate.b"].shape == (128,) and w["l0.mix.sink"].shape == (4,)
    plain.forward(cfg, w, [1, 2, 3])  # the plain implementation reads the same folder


@pytest.mark.gpu
def test_generate_command_and_trace_replay(tmp_path, gpu_device):
    import subprocess
    import sys

    import numpy as np

    folder, cfg, weights = make_dir(tmp_path, "A")
    prompt = random_tokens(21, cfg["vocab"], 4)
    proc = subprocess.run(
        [sys.executable, "-m", "mini_llm_runtime_amd.cli", "generate", "--model", str(folder), "--dtype", "float32",
         "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "5"],
        cwd=ROOT, capture_output=True, text=True, timeout=300,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout.strip().splitlines()[-1])
    seq = list(prompt)
    for tok in out["generated_token_ids"]:
        assert tok == int(torch.argmax(plain.forward(cfg, weights, seq)[-1]))
        seq.append(tok)
    # the replay program: requests in portions beside each other, slots and pages used again
    toks = {"a": random_tokens(40, cfg["vocab"], 5), "b": random_tokens(27, cfg["vocab"], 6), "c": random_tokens(33, cfg["vocab"], 7)}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks["a"][:25], "want": [0, 24]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks["a"][25:27], "want": [1]}, {"id": "b", "tokens": toks["b"], "want": [26]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": toks["a"][27:], "want": [12]}, {"id": "c", "tokens": toks["c"][:32], "want": []}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "c", "tokens": toks["c"][32:], "want": [0]}], "end": ["c"]},
    ]
    proc = subprocess.run(
        [str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "bfloat16", "--out", str(tmp_path / "o"),
         "--max-tokens", "128", "--max-live", "2"],
        input="".join(json.dumps(s) + "\n" for s in steps), cwd=ROOT, capture_output=True, text=True, timeout=300,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    wanted = {0: [("a", 0), ("a", 24)], 1: [("a", 26), ("b", 26)], 2: [("a", 39)], 3: [("c", 32)]}
    for step, rows in wanted.items():
        got = torch.from_numpy(np.fromfile(tmp_path / "o" / f"{step}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"]))
        for row, (rid, pos) in zip(got, rows):
            ref = plain.forward(cfg, weights, toks[rid][: pos + 1])[-1]
            assert float((row.double() - ref).pow(2).sum().sqrt() / ref.pow(2).sum().sqrt()) < 6e-2, (step, rid, pos)
