"""Mepupel models drawn at random (layer order, every size, windows and kept counts, routers, factors)
replayed through the step function in mixed batches against the plain implementation, in both dtypes.
The sizes are the kind a real checkpoint has (multiples of 8 or 16 mostly, some not)."""

import random

import pytest

from mepupel_util import (attention, dense, every_expert, experts, latent, mamba, model_json, oracle_with_margins,
                          random_weights, tokens, write_folder)
from replay_util import mixed, tail_one_by_one, whole
from rorosun_util import run_steps
from test_gpu_mepupel import check_rows

pytestmark = pytest.mark.gpu


def draw_mlp(rng):
    kind = rng.choice(["dense", "moe", "moe", None])
    if kind is None:
        return None
    if kind == "dense":
        return dense(rng.choice([24, 48, 80, 128]))
    count = rng.choice([1, 2, 3, 4])
    size = rng.choice([1, 2, 3, 4])
    n = count * size
    keep = rng.randint(1, count)
    top = rng.randint(1, min(4, keep * size))
    return experts(n, top, rng.choice([16, 24, 40, 64]), rng.choice([None, 0.5, 1.0, 2.5]),
                   rng.choice([None, (count, keep)]), rng.choice([None, 16, 56]))


def draw_model(seed):
    rng = random.Random(seed)
    width = rng.choice([48, 64, 96, 128, 160, 200])
    layers, latents = [], []
    for i in range(rng.randint(3, 7)):
        kind = rng.choice(["mamba2", "attention", "latent", "latent"])
        mlp = draw_mlp(rng)
        if kind == "mamba2":
            groups = rng.choice([1, 2, 4])
            heads = groups * rng.choice([1, 2, 3])
            vdim = rng.choice([8, 16, 24, 32, 64])
            parts = rng.choice([d for d in (1, 2, 4, heads) if (heads * vdim) % d == 0])
            layers.append(mamba(heads, vdim, rng.choice([8, 16, 48, 64, 100]), groups, rng.choice([2, 3, 4, 4, 5]), parts, mlp))
        elif kind == "attention":
            kv = rng.choice([1, 2, 3])
            heads = kv * rng.choice([1, 2, 4, 5, 8])
            dim = rng.choice([16, 32, 48, 64, 96, 128])
            vdim = rng.choice([dim, dim, 32, 80])
            rot = rng.choice([0, dim, dim // 2, 8])
            yarn = rng.choice([None, (rng.choice([2.0, 8.0, 16.0]), rng.choice([32.0, 256.0, 2048.0]), rng.choice([8.0, 32.0]), rng.choice([1.0, 2.0]))])
            window = rng.choice([None, 1, 7, 16, 33, 64, 100])
            keep = 0 if window is None else rng.choice([0, 1, 4, 16, 40])
            layers.append(attention(heads, kv, dim, vdim, rot, rng.choice([None, 0.2, 0.05]), rng.choice([1e4, 5e5]), yarn, window, keep, mlp))
        else:
            source = rng.choice([None] + latents)
            if source is None:
                rank = rng.choice([16, 32, 40, 64, 128, 200])
                latents.append(i)
            else:
                rank = layers[source]["mixer"]["kv_rank"]
            dim = rng.choice([8, 16, 32, 64])
            layers.append(latent(rng.choice([1, 2, 4, 6, 12]), dim, rng.choice([dim, 16, 48]), rank, rng.choice([8, 24, 80, 96]),
                                 rng.choice([None, 0.3]), source, mlp))
    return model_json(layers, vocab=rng.choice([97, 256, 640]), width=width, eps=rng.choice([1e-5, 1e-6]),
                      mult=rng.choice([None, 0.5, 0.22, 1.0]))


@pytest.mark.parametrize("seed", range(12))
def test_random_models_in_mixed_batches(tmp_path, seed):
    from tokamak_amd.engine.runner import ModelRunner

    cfg = draw_model(1000 + seed)
    w = random_weights(cfg, seed)
    requests = {f"r{i}": tokens(cfg["vocab"], n, 7 * seed + i) for i, n in enumerate([3, 130, 47, 1, 81, 20])}
    steps, peak = mixed(requests, seed=seed)
    for dtype, model in (("float32", cfg), ("bfloat16", every_expert(cfg))):
        folder = write_folder(tmp_path / dtype, model, w)
        both = {rid: oracle_with_margins(model, w, toks) for rid, toks in requests.items()}
        expected = {rid: b[0] for rid, b in both.items()}
        runner = ModelRunner.from_folder(folder, dtype=dtype, page_size=16, kv_pool_tokens=max(peak, 16), max_requests=4)
        check_rows(steps, run_steps(runner, steps), expected, dtype, (seed, cfg))
        for plan in (whole({"r1": requests["r1"]}), tail_one_by_one("r4", requests["r4"], tail=40)):
            check_rows(plan, run_steps(runner, plan), expected, dtype, (seed, cfg))
        runner.manager.check()
        assert all(runner.manager.num_free_pages(g) == runner.manager.num_pages(g) for g in range(runner.num_groups))
