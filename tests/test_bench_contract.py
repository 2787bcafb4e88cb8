"""bench.py's command line and its one-line JSON, as far as they can be checked without a GPU:
more than one GPU is refused with a message, the byte count behind `roofline.achieved` is the
stated formula, and (on the GPU) the default run prints one JSON object with the agreed keys."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert r.stdout.strip() == ""
    assert "one GPU" in r.stderr


def test_algorithmic_bytes_formula():
    sys.path.insert(0, ROOT)
    import bench
    rows, kv_dim, q_dim = 32768, 512, 4096
    # K and V once in bf16, q in and context out in f32, one block-table entry per page, the new row
    assert bench.algorithmic_bytes(rows, kv_dim, q_dim, False) == 2 * rows * kv_dim * 2 + 2 * q_dim * 4 + 2048 * 4
    assert bench.algorithmic_bytes(rows, kv_dim, q_dim, True) - bench.algorithmic_bytes(rows, kv_dim, q_dim, False) \
        == 2 * kv_dim * 2
    assert bench.HBM_PEAK_GBPS == 8000.0


@pytest.mark.gpu
def test_default_run_prints_one_json_line_with_the_agreed_keys():
    r = subprocess.run([sys.executable, BENCH, "--steps", "16", "--warmup", "2", "--cpu-seconds", "1"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 16 and d["warmup"] == 2 and d["higher_is_better"] is False
    assert d["unit"] == "us/token" and d["vs_baseline"] is None and d["data"] == "synthetic"
    assert "workload" in d["config"] and "configs[2]" in d["config"]["workload"]
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["unit"] == "GB/s" and rf["peak"] == 8000.0
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3
    assert abs(rf["achieved"] - rf["bytes_per_launch"] / rf["avg_launch_us"] / 1e3) / rf["achieved"] < 1e-2
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["unit"] == "us/token" and cb["cores"] >= 1 and cb["value"] > 0
    assert d["ceiling"]["read_only_launch_us"] > 0
    assert d["ceiling"]["read_then_merge_launch_pair_us"] >= d["ceiling"]["read_only_launch_us"]
    assert d["ceiling"]["read_store_then_merge_launch_pair_us"] > 0
    # the timed kernels produced a context: checked against float64 attention inside the run
    assert 0 <= d["checked_max_abs"] <= 1e-4
    # the restore leg carries the reference's state clone beside it
    assert d["restore"]["cpu_baseline"]["kind"] == "port" and d["restore"]["cpu_baseline"]["value"] > 0
    # the reference's own SDPA length sweep
    sweep = d["sdpa_sweep"]["rows"]
    assert sorted({r["len"] for r in sweep}) == [1024, 4096, 16384, 32768] and {r["element"] for r in sweep} == {"f32", "bf16"}
    assert all(r["us_per_call"] > 0 and r["gbps_effective"] > 0 and r["host_call_ms_per_call"] > 0 for r in sweep)
    # the further legs of the default run: configs[4] at batch 4 and the f32 element
    legs = d["legs"]
    for key, dtype in (("configs4_batch4", "bf16"), ("configs2_f32_element", "f32")):
        leg = legs[key]
        assert leg["dtype"] == dtype and leg["unit"] == "us/token" and leg["value"] > 0
        assert 0 <= leg["checked_max_abs"] <= 1e-4
        lrf = leg["roofline"]
        assert lrf["bound"] == "hbm" and abs(lrf["frac"] - lrf["achieved"] / lrf["peak"]) < 1e-3
    assert legs["configs4_batch4"]["config"]["batch"] == 4 and "configs[4]" in legs["configs4_batch4"]["config"]["workload"]


@pytest.mark.gpu
def test_config3_report_counts_the_reused_tokens_the_reference_algorithm_reuses():
    """`bench.py --config 3` reports, per request, what `saragossa serve` returns as
    x-saragossa-prompt-tokens / x-saragossa-reused-prefix-tokens (src/serve/state.rs:59-80) and
    bench-serve sums up (src/bench_serve.rs:249-289). The reused-token figures must be those of
    the reference's own prefill_prompt_state over the same request stream with the same pool."""
    sys.path.insert(0, ROOT)
    import numpy as np

    import bench
    from oracle import prefix_cache as pc
    r = subprocess.run([sys.executable, BENCH, "--config", "3", "--no-cpu-baseline"], capture_output=True,
                       text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    d = json.loads([l for l in r.stdout.splitlines() if l.strip()][-1])
    rep = d["serve_report"]
    assert rep["summary"]["requested"] == rep["summary"]["succeeded"] == 16 and rep["summary"]["failed"] == 0

    class Sim(pc.PromptDecoder):
        class S:
            def __init__(self, n): self.n = n
            def clone(self): return Sim.S(self.n)
        def prefill_uncached(self, tokens): return Sim.S(len(tokens))
        def extend(self, state, tokens): state.n += len(tokens)

    shared, hist, turn = bench.config3_traffic(np)
    bt, pool_blocks = 16, d["config"]["pool_blocks"]
    ocache = pc.BlockAwarePrefixCache(bt, 10 ** 6, state_bytes=lambda s, m: 1)
    over = lambda extra: len(ocache.entries) + extra > pool_blocks
    stream = [np.concatenate([shared, h]) for h in hist] + \
             [np.concatenate([shared, h, t]) for h, t in zip(hist, turn)]
    want = []
    for tokens in stream:
        _, reused = pc.prefill_prompt_state(ocache, Sim(), [int(t) for t in tokens], None, over)
        want.append((len(tokens), reused))
    got = [(q["prompt_tokens"], q["reused_prefix_tokens"]) for q in rep["requests"]]
    assert got == want
    assert rep["summary"]["reused_prefix_tokens"] == sum(w[1] for w in want) == d["reused_tokens"]
    assert rep["summary"]["prompt_tokens"] == sum(w[0] for w in want)
    assert all(q["restore_us"] > 0 for q in rep["requests"] if q["reused_prefix_tokens"])
    # the decode phase of every request on the KV side (bench-serve's decode_tok_s, generated_tokens)
    assert all(q["generated_tokens"] == 128 and q["decode_kv_tok_s"] > 0 for q in rep["requests"])
    assert rep["summary"]["decode_kv_tok_s_mean"] > 0
