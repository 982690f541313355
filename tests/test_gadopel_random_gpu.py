"""Gadopel models drawn at random - layer order, sizes, head counts, windows, kept positions,
rotation widths, loops, missing feed-forwards - stepped through a random mixed schedule on a small
pool and compared with the plain implementation, in both number formats."""
import numpy as np
import pytest

import gadopel_util as U
import replay_util as R
from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions

pytestmark = pytest.mark.gpu


def random_config(seed: int) -> dict:
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(len(xs)))]
    width = pick(64, 72, 96, 100, 128, 160, 256)
    layers = []
    for _ in range(int(rng.integers(2, 6))):
        ff = pick(None, 48, 104, 192, 256)
        if rng.random() < 0.4:
            rank, rot = pick((24, 4), (40, 8), (64, 32), (64, 64), (128, 32), (96, 16), (128, 64), (200, 24))
            layers.append(U.latent_layer(pick(1, 2, 3, 5, 8, 18), pick(8, 16, 24, 32, 64), rot, pick(8, 16, 24, 32, 48),
                                         rank, base=float(pick(100.0, 10000.0, 300000.0)), scale=pick(0.08, 0.125, 0.2), ff=ff))
        else:
            kv = pick(1, 2, 3, 4)
            dim = pick(16, 20, 32, 48, 64, 128)
            rot = pick(dim, dim // 2 // 2 * 2, 4)
            mask = {"size": pick(1, 5, 16, 33, 100), "keep_first": pick(0, 1, 7, 16, 40)} if rng.random() < 0.75 else None
            scaling = pick(None, U.YARN, {"factor": 2.0, "original": 16, "fast": 3.0, "slow": 0.5})
            layers.append(U.attention_layer(kv * pick(1, 2, 4, 8), kv, dim, pick(dim, 16, 32, 64), rot,
                                            base=float(pick(500.0, 10000.0, 1e6)), scale=pick(0.1, 0.125, 0.25),
                                            mask=mask, scaling=scaling, ff=ff))
    cfg = {"architecture": "Gadopel", "vocab": pick(64, 101, 256, 333), "width": width,
           "norm": {"eps": pick(1e-6, 1e-5)}, "layers": layers}
    if rng.random() < 0.7:
        a = int(rng.integers(0, len(layers)))
        b = int(rng.integers(a + 1, len(layers) + 1))
        cfg["loop"] = {"start": a, "stop": b, "times": int(rng.integers(1, 4))}
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_models_under_random_schedules(seed, dtype, tmp_path, gpu):
    cfg = random_config(1000 + seed)
    folder, state = U.write_model(str(tmp_path / "m"), cfg, seed, gain=0.8)
    rng = np.random.default_rng(seed)
    lengths = [int(n) for n in rng.integers(1, 140, size=7)]
    reqs = {f"q{i}": U.prompt(cfg, n, 13 * i + seed) for i, n in enumerate(lengths)}
    steps = R.mixed(reqs, seed=seed, max_live=4, chunk_sizes=(2, 3, 7, 16, 40))
    eng = Engine(folder, EngineOptions(dtype=dtype, page_size=16, cache_tokens=R.max_live_tokens(steps, unit=16),
                                       max_seqs=4, max_seq_len=160, max_batch_tokens=1024))
    rows = U.run_steps(eng, steps)
    assert len(rows) == sum(lengths)
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs), dtype, f"model {cfg}")
    eng.cache.check()
    assert eng.cache.free_seats == 4 and all(g.free_pages() == g.num_pages for g in eng.cache.groups)
