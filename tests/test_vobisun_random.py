"""Drawn Vobisun configurations: every size, constant, layer count, loop and option drawn anew, random weights,
a drawn schedule and page size, the engine against the plain implementation.  A model of this design that
nobody has looked at must run without a change of code; this is the nearest a test gets.

The bounds are those of `test_vobisun._compare`, the float32 one a little wider (drawn models of many layer
runs add up more 32-bit roundings than the chosen ones).  108 more from the same generator ran once on the GPU in both
dtypes: float32 passed all; bfloat16 missed the bound in seven, each time from a request's first token on, where a
recurrent head's q . k was within a rounding of zero (`test_vobisun._first_token_is_a_coin_flip`; the stand-in on the
CPU, which shares no kernel, gave the same rows to three digits)."""

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
from test_vobisun import FAMILIES, _compare, _layer, _left, _model, _ops, _right, make_weights


def draw_config(seed: int) -> tuple[dict, list[int]]:
    rng = random.Random(seed)
    width = rng.choice([48, 64, 70, 72, 96, 100, 128, 160, 192, 256])
    layers, ranks = [], []
    for _ in range(rng.randint(1, 4)):
        kv_heads = rng.choice([1, 1, 2, 3, 4])
        heads = kv_heads * rng.choice([1, 2, 4, 6])
        dim = rng.choice([8, 10, 16, 24, 32, 48, 64, 96, 128])
        vdim = rng.choice([dim, 8, 12, 16, 32, 40, 64, 96])
        rot_dims = rng.choice([d for d in (2, 4, 6, 8, 16, 32, 64, dim - dim % 2) if d <= dim])
        factor = rng.choice([None, None, 1.0, 2.0, 4.0, 32.0])
        left = _left(
            heads, kv_heads, dim, vdim, rng.choice([1, 2, 5, 8, 16, 17, 33, 64, 100]), rng.choice([1, 2, 3, 4, 8, 16, 20, 32]),
            rot_dims, factor, round(rng.uniform(0.08, 0.3), 3), rng.choice([100.0, 10000.0, 1e6]),
        )
        right = _right(rng.choice([1, 2, 3, 4, 6, 8]), rng.choice([8, 16, 20, 32, 48, 64, 128]), rng.choice([8, 12, 16, 32, 64, 96]), rng.choice([1.0, 2.0, 8.0, 16.0, 64.0]))
        ff = None if rng.random() < 0.25 else rng.choice([24, 40, 45, 64, 136, 320])
        layers.append(_layer(left, right, ff, round(rng.uniform(0.3, 1.5), 2), round(rng.uniform(0.3, 1.5), 2)))
        ranks.append(rng.choice([1, 3, 8, 16, 24, 40]))
    loop = None
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        stop = rng.randint(start, len(layers))
        loop = (start, stop, rng.randint(1, 3))
    cfg = _model(rng.randint(50, 600), width, rng.choice([1e-5, 1e-6]), rng.choice([1.0, 4.0, 16.0]), rng.randint(1, 5), layers, loop)
    return cfg, ranks


def _run(tmp_path, seed: int, backend: str, dtype: torch.dtype) -> None:
    cfg, ranks = draw_config(seed)
    rng = random.Random(1000 + seed)
    folder = Path(tmp_path) / f"drawn{seed}"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    weights = make_weights(cfg, seed, ranks)
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
        _compare(got, requests, weights, cfg, dtype, f32_bound=5e-4, together=3.5e-2)
    except AssertionError as e:
        raise AssertionError(f"{e}\nconfiguration {seed}: {json.dumps(cfg)}; ranks {ranks}; {family}, pages of {bs}") from None
    cache.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_drawn_configuration_on_the_stand_in(tmp_path, seed):
    _run(tmp_path, seed, "double", torch.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("seed", range(32))
def test_drawn_configuration(tmp_path, seed, dtype):
    """Both dtypes on every drawn model: requests whose first token is a coin flip are left out in bfloat16 (see
    `_compare`), never in float32."""
    _run(tmp_path, seed, "hip", dtype)
