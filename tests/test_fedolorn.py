"""The Fedolorn decoder in the engine against the plain implementation (`plain_fedolorn.py`).

Each mechanism alone (norm with offset weights, the products' activations and multiplier, the
chunked mask, value heads of their own width, the output gate, the routing, the grouped expert
products), then whole models under every way of cutting and batching, then greedy generation
through the engine.  The tests make their own small configurations and their own weights: larger
than an initialisation would be, so that attention is peaked and the router decides, and a key
read from the wrong place or a wrong expert shows.

`double` cases run everything above the kernels on the CPU stand-in; `hip` cases run the HIP
kernels (`-m gpu`) in float32 and bfloat16.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import pytest
import torch

import mini_llm_runtime_amd.models  # noqa: F401
import plain_fedolorn as plain
import schedules
from helpers import make_runner, random_tokens
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.config import ConfigError, FedolornConfig
from mini_llm_runtime_amd.engine import ContinuousBatchEngine
from mini_llm_runtime_amd.models import build_model, config_from_dict
from mini_llm_runtime_amd.weights import save_state_dict


# ---- configurations -----------------------------------------------------------------------------------

def _attention(heads, kv_heads, dim, vdim, scale, mask):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if mask is not None:
        m["mask"] = {"size": mask}
    return m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, scale, groups=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def _model(vocab, width, eps, emb_scale, layers):
    return {
        "architecture": "Fedolorn", "vocab": vocab, "width": width, "norm": {"eps": eps},
        "embedding": {"scale": emb_scale},
        "layers": [{"type": "attention", "mixer": a, "mlp": f} for a, f in layers],
    }


CONFIGS = {
    # value heads wider and narrower than key heads, a layer without feed-forward, groups of experts
    "P": _model(300, 64, 1e-6, 1.3, [
        (_attention(4, 2, 16, 32, 0.3, 24), _dense(96)),
        (_attention(2, 1, 32, 16, 0.21, 7), _moe(8, 2, 40, 1.7, (4, 2))),
        (_attention(4, 4, 16, 16, 0.25, 40), None),
    ]),
    # sizes that the matrix-core kernels refuse: a head size of 24, an inner size of 20, one expert a
    # group, one expert a token, a layer with the plain causal mask, an odd vocabulary
    "Q": _model(257, 72, 1e-5, 0.7, [
        (_attention(3, 3, 24, 24, 0.2, 5), _moe(6, 1, 20, 0.9, (6, 3))),
        (_attention(6, 2, 24, 24, 0.2, None), _dense(52)),
    ]),
    # a width that is no multiple of 8, every expert chosen, no groups, a chunk longer than any request
    "R": _model(211, 100, 3e-6, 1.0, [
        (_attention(5, 1, 20, 12, 0.22, 1000), _moe(4, 4, 36, 2.0, None)),
        (_attention(2, 2, 12, 20, 0.3, 3), _moe(4, 2, 28, 1.0, (2, 2))),
    ]),
    # matrix-core sizes: head size 64 with a group of four, 128 against 64, sixteen experts
    "S": _model(512, 128, 1e-5, 2.0, [
        (_attention(4, 1, 64, 64, 0.14, 32), _moe(16, 4, 64, 2.2, (4, 2))),
        (_attention(2, 2, 128, 64, 0.09, 48), _dense(256)),
        (_attention(8, 4, 32, 32, 0.18, 16), _moe(16, 3, 32, 1.5, (8, 3))),
    ]),
    # attention only: what the mask and the gate do is not blurred by a router's close calls
    "T": _model(128, 64, 1e-6, 1.0, [
        (_attention(4, 2, 32, 32, 0.35, 20), None),
        (_attention(2, 1, 48, 16, 0.3, 33), None),
    ]),
    # long requests: hundreds of keys in a chunk (the decode kernel's partitions and their merge, several
    # key tiles of the prompt kernel), a chunk edge deep inside a prompt and passed while decoding
    "U": _model(200, 128, 1e-5, 1.0, [
        (_attention(4, 2, 64, 64, 0.15, 320), _moe(8, 2, 32, 1.2, (2, 1))),
        (_attention(2, 1, 64, 32, 0.15, 512), None),
    ]),
}
BLOCK = {"P": 16, "Q": 8, "R": 4, "S": 16, "T": 8, "U": 16}
LENGTHS = {
    "P": (1, 9, 50, 83, 37, 64), "Q": (2, 19, 35, 66, 45), "R": (3, 30, 41, 58), "S": (5, 17, 140, 70, 97),
    "T": (1, 24, 75, 41, 130), "U": (660, 341),
}


def make_weights(cfg: dict, seed: int) -> dict[str, torch.Tensor]:
    """bfloat16 tensors by the design's checkpoint names."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]

    def normal(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

    w = {"embed": normal(cfg["vocab"], width, std=1.0), "final.norm": normal(width, std=0.2)}
    for i, layer in enumerate(cfg["layers"]):
        p, a = f"l{i}.", layer["mixer"]
        out = a["heads"] * a["vdim"]
        w[p + "norm1"] = normal(width, std=0.2)
        # queries and keys large enough for peaked attention
        w[p + "mix.q"] = normal(a["heads"] * a["dim"], width, std=2.0 / math.sqrt(width))
        w[p + "mix.k"] = normal(a["kv_heads"] * a["dim"], width, std=2.0 / math.sqrt(width))
        w[p + "mix.v"] = normal(a["kv_heads"] * a["vdim"], width, std=1.0 / math.sqrt(width))
        w[p + "mix.g"] = normal(out, width, std=1.5 / math.sqrt(width))
        w[p + "mix.o"] = normal(width, out, std=1.0 / math.sqrt(out))
        mlp = layer["mlp"]
        if mlp is None:
            continue
        w[p + "norm2"] = normal(width, std=0.2)
        if mlp["kind"] == "dense":
            w[p + "mlp.up"] = normal(mlp["ff"], width, std=1.0 / math.sqrt(width))
            w[p + "mlp.down"] = normal(width, mlp["ff"], std=1.0 / math.sqrt(mlp["ff"]))
        else:
            ff, r = mlp["expert"]["ff"], mlp["router"]
            w[p + "mlp.router"] = normal(r["experts"], width, std=3.0 / math.sqrt(width))
            w[p + "mlp.correction"] = normal(r["experts"], std=0.3)
            for e in range(r["experts"]):
                w[f"{p}mlp.e{e}.up"] = normal(ff, width, std=1.0 / math.sqrt(width))
                w[f"{p}mlp.e{e}.down"] = normal(width, ff, std=1.0 / math.sqrt(ff))
    return w


def make_dir(tmp_path, which: str, seed: int = 3) -> tuple[Path, dict, dict]:
    cfg = CONFIGS[which]
    folder = Path(tmp_path) / f"fedolorn{which}"
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    weights = make_weights(cfg, seed)
    save_state_dict(folder / "model.safetensors", weights)
    return folder, cfg, weights


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


def _has_router(cfg: dict) -> bool:
    return any(l["mlp"] is not None and l["mlp"]["kind"] == "moe" for l in cfg["layers"])


def _compare(got, requests, weights, cfg, dtype, f32_bound=1e-4, routed_rows_off=0.03, row_bound=6e-2, together=2.5e-2):
    """float32: every value within 1e-4 of the logits' size.  bfloat16: every row within 6 % (relative
    L2) and all rows together within 2.5 %; where a router decides, a token whose two candidate
    experts are nearly tied may go the other way after rounding, so up to 3 % of the rows may differ
    more (a wrong key, page or expert shows in far more rows than that)."""
    assert got, "no logits came back"
    rows = bad = 0
    num = den = 0.0
    for rid, toks in requests.items():
        ref = plain.forward(cfg, weights, toks)
        size = float(ref.pow(2).mean().sqrt())
        for pos in range(len(toks)):
            row = got[(rid, pos)].double()
            assert torch.isfinite(row).all(), f"{rid}:{pos} is not finite"
            diff = row - ref[pos]
            rows += 1
            if dtype == torch.float32:
                assert float(diff.abs().max()) < f32_bound * size, f"{rid}:{pos}: off by {float(diff.abs().max()):.3e}"
                continue
            rel = float(diff.pow(2).sum().sqrt() / ref[pos].pow(2).sum().sqrt())
            if rel > row_bound:
                bad += 1
                assert _has_router(cfg), f"{rid}:{pos}: relative error {rel:.3e}"
            else:
                num += float(diff.pow(2).sum())
                den += float(ref[pos].pow(2).sum())
    if dtype != torch.float32:
        assert bad <= routed_rows_off * rows, f"{bad} of {rows} rows are off"
        assert (num / den) ** 0.5 < together, f"relative error of all rows {(num / den) ** 0.5:.3e}"


def _requests(which: str) -> dict[str, list[int]]:
    vocab = CONFIGS[which]["vocab"]
    return {f"r{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate(LENGTHS[which])}


# ---- configuration and weights ------------------------------------------------------------------------

def test_config_reads_every_layer_by_itself():
    c = config_from_dict(CONFIGS["P"])
    assert isinstance(c, FedolornConfig)
    assert [l.mixer.vdim for l in c.layers] == [32, 16, 16]
    assert [l.mixer.mask_size for l in c.layers] == [24, 7, 40]
    assert c.layers[2].mlp is None and c.layers[1].mlp.groups_keep == 2 and c.layers[0].mlp.kind == "dense"
    assert FedolornConfig.from_dict(c.to_dict()) == c
    q = config_from_dict(CONFIGS["Q"])
    assert q.layers[1].mixer.mask_size is None
    r = config_from_dict(CONFIGS["R"])
    assert (r.layers[0].mlp.groups_count, r.layers[0].mlp.groups_keep) == (1, 1)


@pytest.mark.parametrize(
    "change",
    [
        lambda c: c["layers"][0]["mixer"].pop("vdim"),
        lambda c: c["layers"][0].update(type="recurrent"),
        lambda c: c["layers"][1]["mlp"]["router"].update(top=5),  # two groups of two hold four experts
        lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3),
        lambda c: c["layers"][0]["mixer"].update(heads=3),
        lambda c: c.pop("norm"),
    ],
)
def test_config_refuses_what_does_not_fit(change):
    cfg = json.loads(json.dumps(CONFIGS["P"]))
    change(cfg)
    with pytest.raises(ConfigError):
        config_from_dict(cfg)


def test_model_is_built_from_the_framework_parts():
    model = build_model(config_from_dict(CONFIGS["P"]))
    kinds = [(type(l.mixer).__name__, type(l.feed_forward).__name__) for l in model.layers]
    assert kinds == [("GQAAttention", "MLP"), ("GQAAttention", "RoutedExperts"), ("GQAAttention", "NoneType")]
    assert model.replayable and model.splittable
    # heads of two widths share one kernel head size, equal widths keep theirs
    assert [l.mixer.kernel_dim for l in model.layers] == [32, 32, 16]
    specs = model.site_cache_specs()
    assert (specs[0].num_kv_heads, specs[0].head_dim) == (2, 32)
    assert (specs[1].num_kv_heads, specs[1].head_dim) == (1, 32)
    assert (specs[2].num_kv_heads, specs[2].head_dim) == (4, 16)


# ---- mechanisms alone, on the GPU ----------------------------------------------------------------------

def _tolerance(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("m,n,k", [(1, 40, 64), (5, 96, 72), (33, 130, 100), (300, 256, 128), (64, 20, 36)])
def test_product_activations_and_multiplier(dtype, m, n, k):
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(m * n + k)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(dtype)
    other = torch.randn(m, n, generator=g).to(dtype)
    z = x.double() @ w.double().T
    for activation, multiply, ref in (
        ("relu2", None, plain.squared_relu(z)),
        ("sigmoid", other, torch.sigmoid(z) * other.double()),
        (None, other, z * other.double()),
    ):
        got = ops.linear(x.cuda(), w.cuda(), None, activation=activation, multiply=None if multiply is None else multiply.cuda())
        torch.testing.assert_close(got.double().cpu(), ref, **_tolerance(dtype))


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("rows,size", [(1, 64), (7, 100), (300, 192), (3, 2048)])
def test_norm_with_weights_stored_around_zero(dtype, rows, size):
    from types import SimpleNamespace

    from mini_llm_runtime_amd.parts import build_part
    from mini_llm_runtime_amd.parts.spec import PartSpec

    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(rows + size)
    norm = build_part("norm", PartSpec("rms_norm", {"size": size, "eps": 1e-5, "weight_offset": 1.0}))
    stored = (torch.randn(size, generator=g) * 0.3).to(torch.bfloat16)  # as a checkpoint holds it
    norm.bind({"weight": stored.to(dtype).cuda()}, dtype=dtype, device=torch.device("cuda"))
    assert norm.weight.dtype == torch.float32  # 1 + w does not fit bfloat16
    x = torch.randn(rows, size, generator=g) * 3.0
    delta = torch.randn(rows, size, generator=g).to(dtype)
    stream = x.clone().cuda()
    got = norm.forward(SimpleNamespace(ops=ops), stream, delta.cuda())
    want = plain.zero_centred_rms_norm(x.double() + delta.double(), stored.double(), 1e-5)
    torch.testing.assert_close(stream.cpu().double(), x.double() + delta.double(), rtol=1e-6, atol=1e-6)  # the 32-bit sum
    torch.testing.assert_close(got.double().cpu(), want, **_tolerance(dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("experts,top,groups,keep", [(8, 2, 4, 2), (6, 1, 6, 3), (4, 4, 1, 1), (16, 3, 8, 3), (64, 6, 8, 4), (12, 3, 2, 1), (5, 2, 1, 1)])
def test_routing_kernel(experts, top, groups, keep):
    ops = _ops("hip", torch.float32)
    g = torch.Generator().manual_seed(experts * 7 + top)
    tokens = 97
    h = torch.randn(tokens, 32, generator=g)
    router = torch.randn(experts, 32, generator=g) * 0.6
    correction = torch.randn(experts, generator=g) * 0.4  # also negative choice scores
    logits = h @ router.T
    ids, weights = ops.route_experts(logits.cuda(), correction.cuda(), top=top, groups=groups, keep_groups=keep, scale=1.7)
    want_ids, want_w = plain.route(
        h.double(), router.double(), correction.double(),
        {"experts": experts, "top": top, "scale": 1.7, "groups": {"count": groups, "keep": keep}},
    )
    got = {(t, int(e)): float(w) for t in range(tokens) for e, w in zip(ids[t].cpu(), weights[t].cpu())}
    want = {(t, int(e)): float(w) for t in range(tokens) for e, w in zip(want_ids[t], want_w[t])}
    assert set(got) == set(want)
    for key in want:
        assert abs(got[key] - want[key]) < 1e-5


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("tokens,hidden,inner,experts,top", [(1, 64, 40, 8, 2), (7, 72, 20, 6, 1), (50, 100, 36, 4, 4), (200, 128, 64, 16, 4), (19, 64, 24, 5, 3), (300, 64, 40, 4, 2), (130, 200, 136, 3, 1), (9, 1024, 512, 4, 2), (21, 1032, 520, 3, 2)])
def test_grouped_expert_products(dtype, tokens, hidden, inner, experts, top):
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(tokens + experts)
    h = torch.randn(tokens, hidden, generator=g).to(dtype)
    up = (torch.randn(experts * inner, hidden, generator=g) / math.sqrt(hidden)).to(dtype)
    down = (torch.randn(experts * hidden, inner, generator=g) / math.sqrt(inner)).to(dtype)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    if tokens > 40 and experts - 2 >= top - 1:
        ids[:40, 0] = 1  # one expert with several tiles of rows
        ids[:40, 1:] = torch.stack([(torch.randperm(experts - 2, generator=g)[: top - 1] + 2) for _ in range(40)]).to(torch.int32)
    weights = torch.rand(tokens, top, generator=g) + 0.1
    out = ops.expert_products(h.cuda(), up.cuda(), down.cuda(), ids.cuda(), weights.cuda(), experts=experts, activation="relu2")
    assert out.shape == (top, tokens, hidden) and out.dtype == torch.float32
    ref = torch.zeros(tokens, hidden, dtype=torch.float64)
    for t in range(tokens):
        for j in range(top):
            e = int(ids[t, j])
            a = plain.squared_relu(up[e * inner : (e + 1) * inner].double() @ h[t].double())
            if dtype == torch.bfloat16:
                a = a.to(torch.bfloat16).double()
            ref[t] += float(weights[t, j]) * (down[e * hidden : (e + 1) * hidden].double() @ a)
    torch.testing.assert_close(out.sum(0).double().cpu(), ref, **_tolerance(dtype))


def _needle_model(mask: int, dim: int, vdim: int) -> tuple[dict, dict]:
    """One attention layer, one head, made so that every query's weight sits on ONE key, the first one
    it may see: token 1 marks keys, token 2 is the query, every other token is filler.  Value and
    output weights carry the marked key's value into the logits, so the logits say whether that key
    was seen: one position too early or too late and they change completely."""
    width = 16
    cfg = _model(8, width, 1e-6, 1.0, [(_attention(1, 1, dim, vdim, 1.0, mask), None)])
    g = torch.Generator().manual_seed(mask)
    w = make_weights(cfg, 5)
    w["embed"] = torch.zeros(8, width)
    w["embed"][:, :8] = torch.eye(8) * 4.0
    w["l0.norm1"] = torch.zeros(width)
    w["final.norm"] = torch.zeros(width)
    q = torch.zeros(dim, width)
    k = torch.zeros(dim, width)
    q[0, 2] = 6.0  # queries of token 2 ...
    k[0, 1] = 6.0  # ... meet keys of token 1 (norm makes the entries about 4 / rms)
    w["l0.mix.q"], w["l0.mix.k"] = q, k
    w["l0.mix.v"] = torch.randn(vdim, width, generator=g) * 0.5
    w["l0.mix.g"] = torch.zeros(vdim, width)
    w["l0.mix.o"] = torch.randn(width, vdim, generator=g) * 0.5
    return cfg, {name: t.to(torch.bfloat16) for name, t in w.items()}


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("mask,dim,vdim", [(16, 16, 16), (37, 32, 16), (64, 16, 48), (5, 24, 24), (300, 64, 64)])
def test_one_key_just_inside_and_just_outside_the_chunk(tmp_path, backend, dtype, mask, dim, vdim):
    if backend == "double" and mask > 100:
        pytest.skip("the CPU stand-in is slow at this length")
    cfg, weights = _needle_model(mask, dim, vdim)
    folder = Path(tmp_path) / "needle"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    save_state_dict(folder / "model.safetensors", weights)
    # a marked key as the first position of a chunk, as the last position of the one before, and far
    # back inside a chunk; queries at the end of a prompt and decoded alone
    length = 2 * mask + max(3, mask // 2) + 1
    start = (length - 1) - (length - 1) % mask  # first position of the last query's chunk
    cases = {}
    for name, marked in (("first", start), ("before", start - 1), ("second", start + 1)):
        toks = [3 + (i % 5) for i in range(length)]
        toks[marked] = 1
        toks[-1] = 2
        cases[name] = toks
    ops = _ops(backend, dtype)
    _, _, cache, runner = make_runner(folder, ops, block_size=8, num_blocks=4 * (length // 8 + 2), max_requests=4)
    cache.poison()
    for family in (schedules.whole, lambda r: schedules.bulk_then_tail(r, tail=mask + 3), schedules.portions):
        got = schedules.run_schedule(runner, cache, family(cases))
        for name, toks in cases.items():
            ref = plain.forward(cfg, weights, toks)[-1]
            row = got[(name, length - 1)].double()
            assert float((row - ref).abs().max()) < (1e-4 if dtype == torch.float32 else 0.08) * float(ref.abs().max())
        # the marked key matters when it is seen and only then
        seen = got[("first", length - 1)]
        assert float((seen - got[("before", length - 1)]).abs().max()) > 0.3 * float(seen.abs().max())


# ---- whole models under every schedule -------------------------------------------------------------------

FAMILIES = {
    "whole": schedules.whole,
    "bulk_then_tail": lambda r: schedules.bulk_then_tail(r, tail=48),
    "portions": schedules.portions,
    "mixed": schedules.mixed,
}


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("which", list(CONFIGS))
def test_schedule_matches_plain(tmp_path, which, family, backend, dtype):
    if backend == "double" and (which == "U" or (which == "S" and family != "mixed")):
        pytest.skip("the CPU stand-in is slow at this size")
    folder, cfg, weights = make_dir(tmp_path, which)
    requests = _requests(which)
    steps = FAMILIES[family](requests)
    bs = BLOCK[which]
    _, model, cache, runner = make_runner(
        folder, _ops(backend, dtype), block_size=bs, num_blocks=schedules.pages_needed(steps, bs), max_requests=4
    )
    cache.poison()
    got = schedules.run_schedule(runner, cache, steps)
    _compare(got, requests, weights, cfg, dtype)
    cache.check_invariants()
    assert all(g.allocator.free_count == g.num_blocks for g in cache.groups), "pages were not given back"


@pytest.mark.parametrize("dtype", GPU_CASES)
def test_replayed_steps_equal_plain_steps(tmp_path, dtype):
    """Steps of a model with routed experts are recorded and replayed; the replays give what the
    unrecorded steps give, bit for bit (nothing on the host depends on the routing)."""
    folder, cfg, _ = make_dir(tmp_path, "S")
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
@pytest.mark.parametrize("which", ["P", "T"])
def test_greedy_generation_through_the_engine(tmp_path, which, backend, dtype):
    folder, cfg, weights = make_dir(tmp_path, which)
    ops = _ops(backend, dtype)
    engine = ContinuousBatchEngine.from_model_dir(
        folder, dtype=ops.dtype, ops=ops, block_size=BLOCK[which], num_blocks=40, max_running_requests=3,
        max_batch_tokens=24,
    )
    prompts = [random_tokens(n, cfg["vocab"], 9 + n) for n in (5, 30, 1, 17)]
    outs = engine.generate(prompts, max_new_tokens=12)
    for prompt, tokens in zip(prompts, outs):
        assert len(tokens) == 12
        seq = list(prompt)
        for i, tok in enumerate(tokens):
            logits = plain.forward(cfg, weights, seq)[-1]
            best = int(torch.argmax(logits))
            if tok != best:
                # only rounding may choose between two nearly equal logits, and only in bfloat16
                assert dtype == torch.bfloat16, f"token {i}: {tok} != {best}"
                assert float(logits[best] - logits[tok]) < 3e-2 * float(logits.abs().max())
                break
            seq.append(tok)


# ---- the command line and the replay program --------------------------------------------------------------

ROOT = Path(__file__).resolve().parents[1]


def test_preset_and_random_model_writer(tmp_path):
    from helpers import read_weights
    from mini_llm_runtime_amd import cli
    from mini_llm_runtime_amd.config.presets import preset_names

    assert "fedolorn-tiny" in preset_names()
    assert cli.main(["random-model", "--config", "fedolorn-tiny", "--seed", "2", "--out", str(tmp_path / "m")]) == 0
    cfg, w = read_weights(tmp_path / "m")
    assert cfg["architecture"] == "Fedolorn" and w["embed"].shape == (384, 96)
    assert w["l1.mlp.e7.down"].shape == (96, 48) and w["l1.mlp.correction"].shape == (8,) and "l2.norm2" not in w
    assert float(w["l0.norm1"].float().abs().max()) < 0.5  # stored around zero
    plain.forward(cfg, w, [1, 2, 3])  # the plain implementation reads the same folder


@pytest.mark.gpu
def test_generate_command_and_trace_replay(tmp_path, gpu_device):
    import subprocess
    import sys

    import numpy as np

    folder, cfg, weights = make_dir(tmp_path, "P")
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
    # the replay program: two requests in portions beside each other, slots and pages used again
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


# ---- pages of runs that every later query has left behind ------------------------------------------------

def test_chunked_sites_give_pages_back():
    from mini_llm_runtime_amd.cache import PagedKVSpec
    from mini_llm_runtime_amd.cache.manager import CacheManager

    spec = PagedKVSpec(2, 16, chunk=8)
    assert [spec.first_live_position(n) for n in (0, 7, 8, 15, 16, 23)] == [0, 0, 8, 8, 16, 16] and spec.live_span() == 7
    with pytest.raises(ValueError):
        PagedKVSpec(2, 16, window=4, chunk=8)
    cache = CacheManager([spec], block_size=4, num_blocks=8, max_requests=2, dtype=torch.float32, device=torch.device("cpu"))
    assert cache.lifetime_blocks(1000, 6) == [blocks(7 + 6, 4) + 1]
    request = cache.create_request("a")
    fed = 0
    for n in (5, 6, 6, 6, 3):  # 26 tokens through a pool that holds whole requests of 32 at most
        cache.begin_step([("a", n)])
        passed = cache.commit_step()
        fed += n
        live = [b for b in request.tables[0] if b >= 0]
        assert len(live) == blocks(fed, 4) - (fed - fed % 8) // 4
        cache.check_invariants()
        if fed >= 8:
            assert all(b == -1 for b in request.tables[0][: (fed - fed % 8) // 4])
    assert passed == {"a": {0: passed["a"][0]}} and len(passed["a"][0]) == 2  # 24 tokens behind: the run 16..23 went
    cache.release_request("a")
    assert cache.groups[0].allocator.free_count == 8


def blocks(tokens: int, size: int) -> int:
    return -(-tokens // size)


CONFIGS["V"] = _model(160, 64, 1e-6, 1.2, [
    (_attention(4, 2, 16, 16, 0.3, 16), _dense(80)),
    (_attention(2, 2, 32, 32, 0.2, 16), None),
])


@pytest.mark.parametrize("backend,dtype", CASES)
def test_generation_in_a_pool_smaller_than_a_request(tmp_path, backend, dtype):
    """A chunked model's request needs the pages of one run and of a step, not of its whole length: 75
    tokens (19 pages of 4) go through a pool of 9 pages, whose pages are used again and again."""
    folder, cfg, weights = make_dir(tmp_path, "V")
    ops = _ops(backend, dtype)
    engine = ContinuousBatchEngine.from_model_dir(
        folder, dtype=ops.dtype, ops=ops, block_size=4, num_blocks=9, max_running_requests=1, max_batch_tokens=8,
    )
    prompt = random_tokens(45, cfg["vocab"], 3)
    tokens = engine.generate([prompt], max_new_tokens=30)[0]
    assert len(tokens) == 30
    seq = list(prompt)
    for i, tok in enumerate(tokens):
        logits = plain.forward(cfg, weights, seq)[-1]
        best = int(torch.argmax(logits))
        if tok != best:
            assert dtype == torch.bfloat16, f"token {i}: {tok} != {best}"
            assert float(logits[best] - logits[tok]) < 3e-2 * float(logits.abs().max())
            break
        seq.append(tok)
