"""Drawn Bubitar configurations: every size, constant, layer order and option drawn anew, random weights,
a drawn schedule and page size, the engine against the plain implementation.  A model of this design that
nobody has looked at must run without a change of code; this is the nearest a test gets.

float32: 1e-3 of the logits' size (chosen models stay below 1e-4; drawn ones of five layers are more often
ill-conditioned: every sublayer's output is normed before it is added, so an output near zero turns the 32-bit
rounding of a cancelling sum into thousandths).  Two draws are left out because they make the norm behind a
sublayer a sign function: decays of 0 and 0.5 (see `draw_config`) and a token input of one dimension.  bfloat16: the bounds of `test_bubitar._compare` (all rows together, single
rows against what rounding alone does), a little wider together, because drawn models are more often
ill-conditioned than chosen ones (a layer whose only sublayer output is near zero before its norm)."""

from __future__ import annotations

import json
import random
from pathlib import Path

import pytest
import torch

import mini_llm_runtime_amd.models  # noqa: F401
import schedules
from helpers import make_runner, random_tokens
from mini_llm_runtime_amd.weights import save_state_dict
from test_bubitar import FAMILIES, _compare, _ff, _latent, _model, _ops, _retention, _rot, make_weights


def _draw_rot(rng: random.Random, most: int) -> dict:
    dims = rng.choice([d for d in (2, 4, 8, 16, 32, 64, most) if d <= most and d % 2 == 0])
    scaling = None
    if rng.random() < 0.5:
        scaling = (rng.choice([2.0, 4.0, 8.0, 32.0]), rng.choice([16, 64, 256, 4096]), rng.choice([4.0, 8.0, 32.0]), rng.choice([0.5, 1.0, 2.0]))
    return _rot(rng.choice([100.0, 10000.0, 1e6]), dims, scaling)


def draw_config(seed: int) -> dict:
    rng = random.Random(seed)
    width = rng.choice([48, 64, 70, 72, 96, 100, 128, 160, 192, 256])
    layers = []
    owners: list[int] = []  # latent layers that make a cache of their own
    for i in range(rng.randint(1, 5)):
        mlp = None if rng.random() < 0.25 else _ff(rng.choice([24, 40, 45, 64, 136, 320]), rng.choice([0.5, 1.0, 2.0, 7.0]))
        if rng.random() < 0.5:
            heads = rng.choice([1, 2, 3, 4, 6, 8])
            dim = rng.choice([8, 16, 20, 32, 48, 64, 128, 136])
            vdim = rng.choice([dim, 8, 12, 16, 32, 40, 64, 96])
            # (a head that forgets at once or nearly so is o = (q . k) v of the last token, and the head's norm
            # makes sign(q . k) of it: no yardstick where q . k is near zero; the kernels' own test has such heads)
            decay = [rng.choice([0.8, 0.9, 0.97, 0.99, 0.999, 1.0]) for _ in range(heads)]
            mixer = _retention(heads, dim, vdim, decay, _draw_rot(rng, dim - dim % 2))
        else:
            heads = rng.choice([1, 2, 3, 4, 6, 8, 12, 20])
            dim = rng.choice([8, 10, 16, 24, 32, 64])
            vdim = rng.choice([dim, 8, 12, 16, 32, 48])
            scale = round(rng.uniform(0.08, 0.3), 3)
            if owners and rng.random() < 0.5:
                source = rng.choice(owners)
                other = layers[source][0][1]
                mixer = _latent(heads, dim, other["rot_dim"], vdim, other["kv_rank"], scale, other["rot"], kv_from=source)
            else:
                rot_dim = rng.choice([2, 4, 6, 8, 16, 32, 64])
                rank = rng.choice([8, 20, 24, 40, 64, 96, 128, 192])
                mixer = _latent(heads, dim, rot_dim, vdim, rank, scale, _draw_rot(rng, rot_dim))
                owners.append(i)
        layers.append((mixer, mlp))
    return _model(rng.randint(50, 600), width, rng.choice([1e-5, 1e-6]), rng.choice([3, 4, 5, 8, 16, 24]), layers)


def _run(tmp_path, seed: int, backend: str, dtype: torch.dtype) -> None:
    cfg = draw_config(seed)
    rng = random.Random(1000 + seed)
    folder = Path(tmp_path) / f"drawn{seed}"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    weights = make_weights(cfg, seed)
    save_state_dict(folder / "model.safetensors", weights)
    longest = 200 if backend == "hip" else 50
    requests = {f"r{i}": random_tokens(rng.randint(1, longest), cfg["vocab"], seed * 10 + i) for i in range(rng.randint(2, 4))}
    family = rng.choice(sorted(FAMILIES))
    steps = FAMILIES[family](requests)
    bs = rng.choice([4, 8, 16, 32])
    _, _, cache, runner = make_runner(
        folder, _ops(backend, dtype), block_size=bs, num_blocks=max(1, schedules.pages_needed(steps, bs)),
        max_requests=schedules.most_live(steps),
    )
    cache.poison()
    for bank in cache.state_banks.values():
        bank.tensor.fill_(float("nan"))
    got = schedules.run_schedule(runner, cache, steps)
    try:
        _compare(got, requests, weights, cfg, dtype, f32_bound=1e-3, together=3.5e-2)
    except AssertionError as e:
        raise AssertionError(f"{e}\nconfiguration {seed}: {json.dumps(cfg)}; {family}, pages of {bs}") from None
    cache.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_drawn_configuration_on_the_stand_in(tmp_path, seed):
    _run(tmp_path, seed, "double", torch.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(32))
def test_drawn_configuration(tmp_path, seed):
    _run(tmp_path, seed, "hip", torch.float32 if seed % 2 else torch.bfloat16)
