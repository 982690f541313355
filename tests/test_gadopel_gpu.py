"""The Gadopel decoder in the engine against the plain implementation (``plain_gadopel``).

Small configurations of their own (``gadopel_util``: other sizes, head counts, layer orders,
windows and loops than any served model), seeded weights with spread-out attention and sinks of a
few units.  Every schedule - whole prompts, token-by-token decoding, portions down to two tokens,
mixed batches on a pool so small that pages and seats come back - must give the logits of the
plain whole-sequence forward pass, in both number formats.
"""
import numpy as np
import pytest
import torch

import gadopel_util as U
import plain_gadopel as plain
import replay_util as R
from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions
from kv_cache_optimization_for_llm_amd.engine.runner import LLM, ServeOptions

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    base = tmp_path_factory.mktemp("gadopel")
    return {name: (cfg, *U.write_model(str(base / name), cfg, seed)) for name, (cfg, seed) in U.CONFIGS.items()}


def engine_for(folder, dtype, **kw):
    opts = dict(dtype=dtype, page_size=16, cache_tokens=1024, max_seqs=4, max_seq_len=512, max_batch_tokens=1024)
    opts.update(kw)
    return Engine(folder, EngineOptions(**opts))


REQUESTS = {"P": [1, 2, 9, 40, 77], "Q": [3, 33, 70], "R": [1, 18, 50, 131], "S": [1, 5, 47, 150]}


def requests_for(name, cfg):
    return {f"{name}{i}": U.prompt(cfg, n, 100 * i + n) for i, n in enumerate(REQUESTS[name])}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_whole_prompts_and_the_first_tokens(name, dtype, models, gpu):
    cfg, folder, state = models[name]
    reqs = requests_for(name, cfg)
    eng = engine_for(folder, dtype)
    rows = U.run_steps(eng, R.whole(reqs))
    assert len(rows) == sum(len(t) for t in reqs.values())
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs), dtype, "whole")
    eng.cache.check()
    assert eng.cache.free_seats == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_prefill_against_token_by_token_decoding(name, dtype, models, gpu):
    """Most of a request in one step, the rest one token at a time: long enough that every window
    passes over decoded tokens and leaves the kept first positions behind."""
    cfg, folder, state = models[name]
    reqs = {k: v for k, v in requests_for(name, cfg).items() if len(v) > 30}
    eng = engine_for(folder, dtype)
    rows = U.run_steps(eng, R.tail_decoded(reqs, tail=45))
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs), dtype, "decode")
    # and a request decoded from its very first token on
    first = {"solo": U.prompt(cfg, 60, 9)}
    rows = U.run_steps(eng, R.tail_decoded(first, tail=59))
    U.assert_rows(rows, U.expected_rows(cfg, state, first), dtype, "decode from the first token")
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(2,), (7, 16, 5, 2, 33, 3, 64, 2), (17, 1, 1, 30)])
@pytest.mark.parametrize("name", ["P", "R", "S"])
def test_portions_of_any_size(name, sizes, dtype, models, gpu):
    cfg, folder, state = models[name]
    reqs = {k: v for k, v in requests_for(name, cfg).items() if len(v) > 8}
    eng = engine_for(folder, dtype, page_size=8 if name == "P" else 16)
    rows = U.run_steps(eng, R.chunked(reqs, sizes))
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs), dtype, f"portions {sizes}")
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, seed", [("P", 0), ("Q", 1), ("R", 2), ("R", 3), ("S", 4), ("S", 5)])
def test_mixed_batches_on_a_small_pool_reuse_pages_and_seats(name, seed, dtype, models, gpu):
    cfg, folder, state = models[name]
    lengths = [40, 3, 90, 25, 61, 2, 130, 47, 33]
    reqs = {f"m{i}": U.prompt(cfg, n, 7 * i + seed) for i, n in enumerate(lengths)}
    steps = R.mixed(reqs, seed=seed, max_live=3)
    pool = R.max_live_tokens(steps, unit=16)
    eng = engine_for(folder, dtype, cache_tokens=pool, max_seqs=3, max_seq_len=192)
    rows = U.run_steps(eng, steps)
    assert len(rows) == sum(lengths)
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs), dtype, "mixed")
    eng.cache.check()
    stats = eng.cache.stats()
    assert stats["pages_reused"] > 0 and stats["running"] == 0
    assert all(g.free_pages() == g.num_pages for g in eng.cache.groups)


def test_a_request_alone_and_in_a_batch_give_the_same_32_bit_logits(models, gpu):
    """fp32 logits of a (request, position) do not depend on the cut, the batch or the pages."""
    cfg, folder, state = models["R"]
    reqs = {f"b{i}": U.prompt(cfg, n, 50 + i) for i, n in enumerate([70, 21, 44])}
    eng = engine_for(folder, "float32")
    alone = U.run_steps(eng, R.whole(reqs))
    together = U.run_steps(eng, R.mixed(reqs, seed=4, max_live=3, chunk_sizes=(2, 3, 16, 9)))
    assert alone.keys() == together.keys()
    for key in alone:
        np.testing.assert_array_equal(alone[key], together[key], err_msg=str(key))


def test_window_pages_are_given_back_and_the_kept_ones_stay(models, gpu):
    cfg, folder, state = models["R"]
    eng = engine_for(folder, "float32", cache_tokens=256)
    toks = U.prompt(cfg, 200, 77)
    reqs = {"w": toks}
    rows = U.run_steps(eng, [{"step": 0, "entries": [{"id": "w", "tokens": toks[:150], "want": [149]}], "end": []}])
    seat = eng.seat_of("w")
    by_window = {g.spec.window: g for g in eng.cache.groups if g.spec.kind == "window"}
    assert sorted(by_window) == [16, 33]
    g = by_window[33]                       # 17 kept positions: blocks 0 and 1 stay; the window starts in block 7
    row = g.table_host[seat]
    assert (row[:2] >= 0).all() and (row[2:7] == -1).all() and (row[7:10] >= 0).all()
    g = by_window[16]                       # 16 kept positions: block 0 stays
    row = g.table_host[seat]
    assert row[0] >= 0 and (row[1:8] == -1).all() and (row[8:10] >= 0).all()
    more = U.run_steps(eng, [{"step": 1, "entries": [{"id": "w", "tokens": toks[150:], "want": [0, 49]}], "end": ["w"]}])
    exp = U.expected_rows(cfg, state, reqs)
    U.assert_rows(rows, exp, "float32")
    got = {("w", 150 + p): v for (_, p), v in more.items()}
    U.assert_rows(got, exp, "float32")
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_trace_runner_replays_a_mixed_schedule(dtype, models, tmp_path, gpu):
    cfg, folder, state = models["P"]
    reqs = {f"t{i}": U.prompt(cfg, n, 11 + i) for i, n in enumerate([30, 2, 75, 18, 52])}
    steps = R.mixed(reqs, seed=5, max_live=4)
    rows = R.run_trace(folder, dtype, steps, R.max_live_tokens(steps), str(tmp_path / "out"), cfg["vocab"])
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs), dtype, "trace")
    assert R.cache_stats(str(tmp_path / "out"))["pages_reused"] > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "R", "S"])
def test_greedy_generation_through_the_entry_point(name, dtype, models, gpu):
    cfg, folder, state = models[name]
    prompts = [U.prompt(cfg, n, 3 + n) for n in (1, 12, 37, 64, 5, 90)]
    llm = LLM(folder, EngineOptions(dtype=dtype, max_seqs=3, max_seq_len=160, cache_tokens=480),
              ServeOptions(chunk_size=16, max_batch_tokens=48))
    got, reasons = llm.generate(prompts, max_new_tokens=24, ignore_eos=True, return_reasons=True)
    assert reasons == ["length"] * len(prompts)
    for p, g in zip(prompts, got):
        assert len(g) == 24
        logits = plain.forward(cfg, state, list(p) + list(g)).numpy()
        for i, tok in enumerate(g):
            row = logits[len(p) + i - 1]
            slack = (1e-3 if dtype == "float32" else 6e-2) * (row.max() - row.mean())
            assert row[tok] >= row.max() - slack, f"token {i}: {tok} is not the best ({int(row.argmax())})"
    llm.engine.cache.check()
    assert llm.engine.cache.free_seats == 3


@pytest.mark.parametrize("name", ["R", "S"])
def test_decode_steps_from_graphs_equal_eager_steps(name, models, gpu):
    """A bf16 decode step replayed from its HIP graph gives bit for bit what the eager step gives."""
    cfg, folder, state = models[name]
    reqs = {f"g{i}": U.prompt(cfg, n, 31 + i) for i, n in enumerate([48, 80])}
    steps = R.tail_decoded(reqs, tail=20)
    eager = U.run_steps(engine_for(folder, "bfloat16", use_graphs=False), steps)
    eng = engine_for(folder, "bfloat16")
    assert eng.graphs is not None
    replayed = U.run_steps(eng, steps)
    assert eng.graphs.replays > 0
    for key in eager:
        np.testing.assert_array_equal(eager[key], replayed[key], err_msg=str(key))


def test_portion_steps_from_graphs_equal_eager_steps(models, gpu, monkeypatch):
    """Steps with prompt portions whose shape comes back run from a graph of their own: the same
    portions of two requests beside each other, four times over, eagerly and replayed.  (A graph
    cuts the keys into ranges by its context bucket, an eager step by the context it sees: the
    eager steps are given the bucket too, and then a replay is bit for bit the eager step.)"""
    import kv_cache_optimization_for_llm_amd.engine.engine as engine_module
    from kv_cache_optimization_for_llm_amd.engine.graphs import context_bucket
    plain_build = engine_module.build_batch

    def build_with_bucket(*args, **kwargs):
        batch = plain_build(*args, **kwargs)
        batch.max_context = context_bucket(batch.max_context)
        return batch
    monkeypatch.setattr(engine_module, "build_batch", build_with_bucket)
    cfg, folder, state = models["S"]
    steps, n = [], 0
    for rep in range(4):
        reqs = {f"a{rep}": U.prompt(cfg, 96, 60 + rep), f"b{rep}": U.prompt(cfg, 96, 70 + rep)}
        for lo in range(0, 96, 24):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[lo:lo + 24], "want": [0, 23]}
                                                  for rid, toks in reqs.items()],
                          "end": list(reqs) if lo == 72 else []})
            n += 1
    eager = U.run_steps(engine_for(folder, "bfloat16", use_graphs=False), steps)
    eng = engine_for(folder, "bfloat16")
    replayed = U.run_steps(eng, steps)
    assert eng.portion_graphs is not None and eng.portion_graphs.replays > 0
    for key in eager:
        np.testing.assert_array_equal(eager[key], replayed[key], err_msg=str(key))
    reqs = {f"{c}{rep}": U.prompt(cfg, 96, (60 if c == "a" else 70) + rep) for rep in range(4) for c in "ab"}
    U.assert_rows(replayed, U.expected_rows(cfg, state, reqs), "bfloat16", "replayed portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_contiguous_cache_mode_gives_the_logits_of_the_plain_model(dtype, models, gpu):
    """The buddy-allocated cache under the same kernels: portions, then decoding, two requests a step."""
    cfg, folder, state = models["S"]
    reqs = {f"c{i}": U.prompt(cfg, n, 90 + i) for i, n in enumerate([70, 33, 121])}
    eng = engine_for(folder, dtype, cache_mode="contiguous", cache_tokens=4 * 128, max_seq_len=128)
    rows = U.run_steps(eng, R.mixed(reqs, seed=9, max_live=3))
    U.assert_rows(rows, U.expected_rows(cfg, state, reqs), dtype, "contiguous")
    eng.cache.check()


def test_the_serving_process_serves_the_model_in_both_cache_modes(models, tmp_path, gpu):
    """``cli.client`` starts ``cli.serve`` on the model folder: every sequence emits its budget and
    the paged and the contiguous cache emit the same ids."""
    import json
    import os
    import subprocess
    import sys
    cfg, folder, state = models["R"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    results = {}
    for mode in ("paged", "contiguous"):
        out = tmp_path / f"{mode}.json"
        env = dict(os.environ, IGNORE_EOS="1", ORCA_POLICY="oracle", PYTHONPATH=root)
        cmd = [sys.executable, "-m", "kv_cache_optimization_for_llm_amd.cli.client", folder, "5", "--prompt-len", "37",
               "--max-new-tokens", "10", "--num-seqs", "2", "--out", str(out), "--", "--dtype", "float32",
               "--cache-mode", mode, "--max-seqs", "4", "--max-seq-len", "64", "--cache-tokens", "384",
               "--chunk-size", "8", "--max-batch-tokens", "24"]
        proc = subprocess.run(cmd, env=env, cwd=root, capture_output=True, text=True, timeout=280)
        assert proc.returncode == 0, proc.stdout + proc.stderr
        results[mode] = json.load(open(out))
    for r in results.values():
        assert r["status"] == "ok" and r["sequences_done"] == 10 and r["tokens"] == 100
        assert r["count_mismatches"] == 0 and r["budget_mismatches"] == 0 and r["errors"] == []
    assert results["paged"]["checksums"] == results["contiguous"]["checksums"]


def test_the_sweep_command_runs_a_configuration_file_of_this_architecture(models, tmp_path, gpu):
    import json
    import os
    from kv_cache_optimization_for_llm_amd.cli import sweep
    cfg, folder, state = models["S"]
    out = tmp_path / "sweep.jsonl"
    assert sweep.main(["--shapes", os.path.join(folder, "config.json"), "--batches", "3", "--cache-modes", "paged",
                       "--prompt-len", "40", "--prompt-min", "5", "--workload", "mixed", "--new-tokens", "9",
                       "--max-seqs", "2", "--out", str(out)]) == 0
    line, = [json.loads(l) for l in out.read_text().splitlines()]
    assert line["requests_done"] == 3 and line["tokens_emitted"] == 27 and line["finish_reasons"] == {"length": 3}
    assert line["layers"] == 4 and line["pages_reused"] > 0
