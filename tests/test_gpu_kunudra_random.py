"""Kunudra configurations drawn by seed: sizes, head counts, windows, caps, which layers share values,
experts, constants, layer order and page size all vary; each is run whole and under a mixed schedule
(four live requests, pools used again) and held against the plain model, in both engines (bfloat16 with
steadily chosen experts: see `tiny_kunudra.make_weights`)."""

import numpy as np
import pytest

import plain_kunudra as pk
import replay_util as ru
import tiny_kunudra as tk

pytestmark = pytest.mark.gpu
SEEDS = list(range(12))
CHAOTIC_SHARE = 0.03  # of the largest |logit|: a yardstick whose 99th percentile lies beyond this says nothing


def draw(seed: int):
    rng = np.random.default_rng(2000 + seed)
    pick = lambda values: values[int(rng.integers(0, len(values)))]  # noqa: E731
    width = pick([40, 48, 72, 90, 96, 128, 200, 256])
    shared_width = pick([16, 24, 32, 64])  # kv_heads * vdim of every layer that shares values

    def mlp():
        kind = pick(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return tk.dense(pick([32, 70, 96, 256]))
        experts, identity = pick([1, 2, 3, 5, 8, 16]), pick([None, 0, 1, 3])
        top = int(rng.integers(1, experts + (identity or 0) + 1))
        return tk.moe(pick([16, 26, 32, 64, 96]), experts, min(top, 6), identity=identity,
                      scale=pick([None, 0.5, 1.0, 2.5]), shared=pick([None, None, 24, 64]))

    layers = []
    for _ in range(int(rng.integers(1, 6))):
        window = pick([None, 1, 2, 3, 9, 15, 16, 17, 31, 32, 33, 50, 64, 80, 500])
        if rng.random() < 0.55:
            heads = pick([1, 2, 3, 4, 6, 8])
            kv_heads = pick([d for d in (1, 2, 3, 4, 6, 8) if heads % d == 0])
            dim = pick([8, 16, 32, 32, 40, 64, 64, 96])
            sharing = rng.random() < 0.6 and shared_width % kv_heads == 0 and (shared_width // kv_heads) % 2 == 0
            vdim = shared_width // kv_heads if sharing else pick([dim, dim, 8, 24, 64])
            layers.append(tk.attention(heads, pick([kv_heads, kv_heads, None]) if kv_heads == heads else kv_heads, dim, vdim,
                                       float(rng.uniform(0.1, 1.2)), window=window, softcap=pick([None, 1.5, 10.0, 50.0]),
                                       v_mix=sharing, mlp=mlp()))
        else:
            heads, dim, rot = pick([1, 2, 3, 4, 8]), pick([4, 8, 16, 32, 48, 64]), pick([2, 4, 8, 16, 32, 64])
            layers.append(tk.latent(heads, dim, rot, pick([4, 8, 16, 32, 64]), pick([8, 12, 32, 64, 128]), pick([6, 16, 24, 80]),
                                    float(rng.uniform(0.1, 1.0)), float(pick([10.0, 1000.0, 20000.0])), window=window, mlp=mlp()))
    pairs = pick([None, (7, 3, 1), (97, 31, 5), (1021, 255, 16)])
    cfg = tk.config(int(rng.integers(60, 400)), width, layers, eps=float(pick([1e-6, 1e-5, 1e-4])),
                    alpha=pick([None, 1.0, 1.5, 3.0]), pairs=pairs)
    return cfg, pick([4, 8, 16, 16, 32])


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    made = {}

    def get(seed, dtype):
        if (seed, dtype) not in made:
            cfg, block = draw(seed)
            weights = tk.make_weights(cfg, seed=seed, steady_choice=dtype == "bfloat16")
            folder = tk.write_model_dir(tmp_path_factory.mktemp("random") / f"{seed}-{dtype}", cfg, weights)
            lengths = (71, 3, 38, 1, 55)
            requests = {f"q{i}": tk.random_tokens(cfg, n, seed=seed * 10 + i) for i, n in enumerate(lengths)}
            wide = {k: v.astype(np.float64) for k, v in weights.items()}
            oracles = {}
            for rid, t in requests.items():
                exact = pk.logits(cfg, wide, t)
                oracles[rid] = ru.Oracle(exact, pk.logits(cfg, wide, t, store=pk.bf16_round))
                pk.ANGLE_TYPE = np.float32  # (a float32 engine's angles: see plain_kunudra)
                try:
                    as_float32 = pk.logits(cfg, wide, t, store=lambda a: np.asarray(a, dtype=np.float32).astype(np.float64))
                finally:
                    pk.ANGLE_TYPE = np.float64
                oracles[rid].moved_by_float32 = float(np.abs(as_float32 - exact).max())
            made[seed, dtype] = (cfg, block, folder, requests, oracles)
        return made[seed, dtype]

    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("family", ["whole", "mixed"])
@pytest.mark.parametrize("seed", SEEDS)
def test_a_configuration_drawn_by_seed(models, seed, family, dtype):
    from mini_infer_amd.engine import ModelRunner

    cfg, block, folder, requests, oracles = models(seed, dtype)
    schedule = ru.schedule_whole(requests) if family == "whole" else ru.schedule_mixed(requests, seed=seed, max_live=4, tail=9)
    pages = ru.peak_pages(requests, schedule, block)
    runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=pages, block_size=block, max_concurrent=4)
    got = ru.run_schedule(runner, requests, schedule)
    what = f"seed {seed} ({[layer['type'] for layer in cfg['layers']]}, width {cfg['width']}, pages of {block})"
    for rid in requests:
        if dtype == "bfloat16" and oracles[rid].yard_p99 > CHAOTIC_SHARE * float(np.abs(oracles[rid].exact).max()):
            continue  # (bfloat16 storage alone scatters this configuration's logits: nothing to hold an engine against)
        # float32: 1e-4, or twice as far as float32 storage and angles alone move this input's logits; bfloat16:
        # three times the yardstick's largest error (requests of 1 and 3 tokens make it the largest of few draws,
        # and latent attention over the cache rounds two rows more than the plain model's whole-sequence form)
        ru.assert_close(got[rid], oracles[rid], dtype, f"{what} {family} {rid}",
                        fp32_tol=max(ru.FP32_TOL, 2.0 * oracles[rid].moved_by_float32), bf16_max_factor=3.0)
    runner.cache.check()
    assert runner.cache.states.num_free == 4 and runner.num_free_blocks() == pages
