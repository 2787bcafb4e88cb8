#!/usr/bin/env python3
"""KV-path decode benchmark on one MI355X.

Workload (BASELINE.json configs[2]): a Qwen3.6-35B-A3B-style hybrid at 32k context.
10 full-attention layers with 16 query heads, 2 KV heads, head_dim 256, bf16 KV in
16-token pages behind random block tables, pre-filled with 32768 rows of N(0,1).
One step = one decoded token: for each of the 10 layers, append one fresh K/V row
and run paged GQA decode attention with a fresh query. Inputs are resident in HBM
when the timed region starts.

Prints ONE JSON line. `value` is microseconds per token over the 10 KV layers.
`roofline` covers the decode attention kernel alone: algorithmic bytes per launch
(K and V of one layer read once, query in, context out, block table) over the
kernel's average duration measured with HIP events around every launch in a
separate pass after the timed region. `cpu_baseline` times the CPU oracle (a C
restatement of the reference's CPU path) on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak

# BASELINE.json configs that are decode workloads. Each entry: groups of identical layers
# (count, q_heads, kv_heads, head_dim, cached rows, sliding window). The default, and the
# configuration the metric is quoted on, is configs[2].
WORKLOADS = {
    1: dict(name="configs[1]: 36 layers q32/kv8/hd128 (Qwen3-4B KV shapes), %d cached rows",
            groups=[(36, 32, 8, 128, 2048, 0)]),
    2: dict(name="configs[2]: 10 full-attention layers q16/kv2/hd256, %d cached rows",
            groups=[(10, 16, 2, 256, 32768, 0)]),
    4: dict(name="configs[4]: 8 global layers q16/kv8/hd256 at %d rows + 40 local layers with a "
                 "1024-row ring",
            groups=[(8, 16, 8, 256, 65536, 0), (40, 16, 8, 256, 65536, 1024)]),
}


# HBM bytes one attention launch (split + merge) moves, from the hardware counters
# FETCH_SIZE and WRITE_SIZE collected with rocprofv3 --pmc over this same program and scaled
# by what the counters read for a copy of known size (the method and the raw readings are in
# profiles/decode_split_kernel_config2.md). Not measurable from inside this process, so it is
# a recorded figure, present only for the workload it was taken on.
MEASURED_TRAFFIC_BYTES = {2: 70160 * 1024}


# What the matrix pipes sustain for the prefill kernel's product stream when nothing else is in
# the kernel: 16x16x32 bf16 products with every operand in registers, on random operand values
# (the clock under the matrix pipes drops when operand bits toggle), measured with a
# stand-alone product-stream program on one MI355X in a stream of launches, like the prefill
# leg's `us` (1732 with the launches one at a time; 1580 on the box of an earlier recording).
# A recorded figure, like the traffic above; the published peak stays the roofline's `peak`.
MFMA_STREAM_RANDOM_TFLOPS = 1783.0

def algorithmic_bytes(rows: int, kv_dim: int, q_dim: int, with_append: bool, elem_bytes: int = 2) -> int:
    """Bytes one layer's decode step has to move: K and V once (in the cache's element: 2 bytes
    for bf16, 4 for f32), q in and ctx out (f32), the block table, and the appended row when the
    append is counted."""
    b = 2 * rows * kv_dim * elem_bytes + 2 * q_dim * 4 + (rows + 15) // 16 * 4
    if with_append:
        b += 2 * kv_dim * elem_bytes
    return b


def native_remember():
    """The same 256 one-block remembers from a plain C host (tests/native/kv_c_remember.c, built
    by __graft_entry__.build()): what the call costs without an interpreter around it. None
    when the program has not been built."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "native", "kv_c_remember")
    if not os.path.exists(exe):
        return None
    try:
        run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
        if run.returncode != 0:
            return {"error": (run.stderr or run.stdout)[-200:]}
        return json.loads(run.stdout.strip().splitlines()[-1])
    except Exception as exc:  # a report field, never a reason to lose the bench line
        return {"error": str(exc)[:200]}


def bench_restore(skv, torch, np, state, stream, element="bf16"):
    """Prefix block restore (BASELINE.json configs[3] shapes): the 4096-token shared prefix,
    256 hash blocks of 16 tokens over 36 layers of Qwen3-4B KV (8 kv heads, head_dim 128), is
    matched by chained hash and gathered from the hot cache's page pool into a fresh
    session's paged cache. Timed with HIP events from before the host-side hash walk to the
    end of the last copy kernel; payload = bytes restored, traffic = read + write."""
    from saragossa_amd import BlockHash
    qh, kvh, hd, nl, n_tok, bt = 32, 8, 128, 36, 4096, 16
    dev = torch.device("cuda:0")
    f32 = element == "f32"
    esize = 4 if f32 else 2

    def make(seed):
        out = []
        for i in range(nl):
            kv = (state.full_attention_f32 if f32 else state.full_attention_bf16)(n_tok + 16, qh, kvh, hd)
            kv.set_block_table(np.random.default_rng(seed * 100 + i).permutation(kv.pages())
                               .astype(np.int32))
            out.append(kv)
        return out

    src = make(1)
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    for kv in src:
        k = torch.randn(n_tok, kvh * hd, device=dev, generator=gen)
        v = torch.randn(n_tok, kvh * hd, device=dev, generator=gen)
        kv.encode_append_batch(stream, k.data_ptr(), v.data_ptr(), n_tok)
        torch.cuda.synchronize()
    hot = skv.HotCache(state, bt, 10 ** 6, n_tok // bt + 8, src)
    tokens = np.random.default_rng(3).integers(0, 151936, size=n_tok).astype(np.uint64)
    root = BlockHash.root()
    # One remember per block boundary, the reference's own call pattern
    # (remember_prefix_block, src/serve/state.rs:613-639): 256 calls, each a hash step and a
    # one-page copy launch, host-bound. Median of five passes with the interpreter's cyclic
    # collector held off: a full collection in the middle of a pass (tens of milliseconds with
    # torch loaded) is the interpreter's pause, not the library's.
    import gc
    one_by_one = []
    for _ in range(5):
        while hot.evict_lru_block() is not None:
            pass
        torch.cuda.synchronize()
        gc.collect()
        gc.disable()
        try:
            h = root
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for b in range(n_tok // bt):
                h = BlockHash.chain(h, tokens[b * bt:(b + 1) * bt])
                hot.remember_prefix_block(root, h, (b + 1) * bt, src, stream=stream)
            e1.record()
            torch.cuda.synchronize()
        finally:
            gc.enable()
        one_by_one.append(e0.elapsed_time(e1) * 1e3)
    snap_us = sorted(one_by_one)[len(one_by_one) // 2]
    # the same 256 blocks remembered by one call (a chunked prefill crosses many boundaries)
    while hot.evict_lru_block() is not None:
        pass
    hashes, h = [], root
    for b in range(n_tok // bt):
        h = BlockHash.chain(h, tokens[b * bt:(b + 1) * bt])
        hashes.append(h)
    samples = []
    for _ in range(5):  # median: the first call also pays for cold code and a cold index
        while hot.evict_lru_block() is not None:
            pass
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        kept = hot.remember_prefix_blocks(root, hashes, bt, src, stream=stream)
        e1.record()
        torch.cuda.synchronize()
        assert kept == n_tok // bt
        samples.append(e0.elapsed_time(e1) * 1e3)
    snap_range_us = sorted(samples)[len(samples) // 2]
    dst = make(2)
    times = []
    for it in range(13):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        reused, _ = hot.match_restore(root, tokens, dst, stream=stream)
        e1.record()
        torch.cuda.synchronize()
        if it >= 3:
            times.append(e0.elapsed_time(e1) * 1e3)
    assert reused == n_tok
    # the same restore eight times in a row between two events, as a server under load issues
    # them: the host's hash walk for one restore then runs while the GPU still copies the last
    # (informational; `us` stays the single restore on an idle stream, what one request waits for)
    streamed = []
    for it in range(6):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(8):
            hot.match_restore(root, tokens, dst, stream=stream)
        e1.record()
        torch.cuda.synchronize()
        if it >= 1:
            streamed.append(e0.elapsed_time(e1) * 1e3 / 8)
    streamed.sort()
    us_stream = streamed[len(streamed) // 2]
    same = all(np.array_equal(a.read_rows_f32(0, 96)[0], b.read_rows_f32(0, 96)[0]) and
               np.array_equal(a.read_rows_f32(n_tok - 40, 40)[1], b.read_rows_f32(n_tok - 40, 40)[1])
               for a, b in zip(src[::7], dst[::7]))
    if not same:
        raise RuntimeError("restore: restored rows differ from the snapshotted rows")
    times.sort()
    us = times[len(times) // 2]
    payload = n_tok * nl * 2 * kvh * hd * esize
    out = {"workload": "configs[3]: restore of a 4096-token prefix, 256 blocks x 36 layers, "
                       "kv8/hd128 %s (hash walk on the host included)" % element,
           "payload_mib": round(payload / 2 ** 20, 1), "us": round(us, 1),
           "payload_gbps": round(payload / us / 1e3, 1),
           "traffic_gbps": round(2 * payload / us / 1e3, 1),
           "frac_of_hbm_peak": round(2 * payload / us / 1e3 / HBM_PEAK_GBPS, 4),
           "us_in_a_stream_of_8": round(us_stream, 1),
           "frac_of_hbm_peak_in_a_stream_of_8": round(2 * payload / us_stream / 1e3 / HBM_PEAK_GBPS, 4),
           "snapshot_256_blocks_one_by_one_us": round(snap_us, 1),
           "snapshot_256_blocks_one_by_one_passes_us": [round(t, 1) for t in one_by_one],
           "snapshot_256_blocks_one_by_one_native": native_remember(),
           "snapshot_256_blocks_one_call_us": round(snap_range_us, 1),
           "snapshot_traffic_gbps": round(2 * payload / snap_range_us / 1e3, 1)}
    for kv in src + dst:
        kv.close()
    hot.close()
    return out


def bench_sdpa_sweep(skv, torch, np, state, stream, iters=100):
    """The reference's own SDPA micro-benchmark (attention_decode_bench,
    src/decode_resident/tests.rs:1494-1541): decode attention alone at q16/kv2/hd256 over 1024,
    4096, 16384 and 32768 cached rows of its arithmetic test data, ms per call and effective GB/s
    over the K and V bytes read once. The reference times its synchronous host call on an f32
    cache (greedy policy); here each length is timed on both elements, as device launches back
    to back (HIP events) and, like the reference, as the synchronous host call (query in, context
    out over PCIe, a stream synchronisation per call)."""
    qh, kvh, hd = 16, 2, 256
    kv_dim, q_dim = kvh * hd, qh * hd
    dev = torch.device("cuda:0")
    q_host = ((np.arange(q_dim) % 89).astype(np.float32) - 44.0) * np.float32(0.01)
    q = torch.from_numpy(q_host).to(dev)
    out = torch.empty(q_dim, device=dev, dtype=torch.float32)
    rows = []
    for n in (1024, 4096, 16384, 32768):
        idx = torch.arange(n * kv_dim, device=dev, dtype=torch.int64)
        k = (((idx % 101).to(torch.float32) - 50.0) * 0.01).view(n, kv_dim)
        v = (((idx % 97).to(torch.float32) - 48.0) * 0.01).view(n, kv_dim)
        for element, esize in (("f32", 4), ("bf16", 2)):
            kv = (state.full_attention_f32 if element == "f32" else state.full_attention_bf16)(n, qh, kvh, hd)
            kv.encode_append_batch(stream, k.data_ptr(), v.data_ptr(), n)
            for _ in range(5):
                kv.encode_attention_decode(stream, q.data_ptr(), out.data_ptr())
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(iters):
                kv.encode_attention_decode(stream, q.data_ptr(), out.data_ptr())
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / iters
            t0 = time.perf_counter()
            for _ in range(iters):
                kv.attention_decode(q_host)
            host_ms = (time.perf_counter() - t0) * 1e3 / iters
            nbytes = n * kv_dim * esize * 2
            rows.append({"len": n, "element": element, "us_per_call": round(us, 2),
                         "gbps_effective": round(nbytes / us / 1e3, 1),
                         "host_call_ms_per_call": round(host_ms, 4),
                         "host_call_gbps_effective": round(nbytes / host_ms / 1e6, 1)})
            kv.close()
        del idx, k, v
    return {"workload": "attention_decode_bench of the reference (src/decode_resident/tests.rs:1494-1541): "
                        "q16/kv2/hd256, decode attention alone, %d calls per length" % iters,
            "rows": rows}


def bench_prefill(skv, torch, np, state, stream, element="bf16"):
    """Chunked prefill over the cache (cached_attention_prefill_rows as one launch): a
    512-row chunk appended and attended causally over the rows already cached, at the KV
    shapes of configs[2] (after 32768 rows) and configs[1] (the last chunk of its 2048-token
    prompt). The one matrix-core-bound kernel of the path: flops = 4 * keys * q_dim over the
    (query, key) pairs attended; the kernel issues twice that on the matrix cores because
    queries and probabilities are split into two bf16 terms. With the f32 element the products
    run once, on the f32 matrix instruction."""
    dev = torch.device("cuda:0")
    f32 = element == "f32"
    out = []
    for name, (qh, kvh, hd), base, chunk in (("configs[2] shape q16/kv2/hd256", (16, 2, 256), 32768, 512),
                                            ("configs[1] shape q32/kv8/hd128", (32, 8, 128), 1536, 512)):
        kv_dim, q_dim = kvh * hd, qh * hd
        kv = (state.full_attention_f32 if f32 else state.full_attention_bf16)(base + chunk + 16, qh, kvh, hd)
        kv.set_block_table(np.random.default_rng(7).permutation(kv.pages()).astype(np.int32))
        gen = torch.Generator(device=dev)
        gen.manual_seed(7)
        k0 = torch.randn(base, kv_dim, device=dev, generator=gen)
        v0 = torch.randn(base, kv_dim, device=dev, generator=gen)
        kv.encode_append_batch(stream, k0.data_ptr(), v0.data_ptr(), base)
        q = torch.randn(chunk, q_dim, device=dev, generator=gen)
        k = torch.randn(chunk, kv_dim, device=dev, generator=gen)
        v = torch.randn(chunk, kv_dim, device=dev, generator=gen)
        o = torch.empty(chunk, q_dim, device=dev)
        def call():
            kv.truncate(base)  # host bookkeeping only
            kv.encode_prefill_rows(stream, q.data_ptr(), k.data_ptr(), v.data_ptr(), chunk, o.data_ptr())

        def timed(calls):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(calls):
                call()
            e1.record()
            return e0, e1

        # (a) one call at a time on a GPU that has just been idle, the way the kernel traces
        # under profiles/ see it
        single = []
        for it in range(8):
            torch.cuda.synchronize()
            e0, e1 = timed(1)
            torch.cuda.synchronize()
            if it >= 3:
                single.append(e0.elapsed_time(e1) * 1e3)
        single.sort()
        # (b) a stream of calls, like the chunks of a long prompt: this matrix-core-bound kernel
        # keeps getting faster for some 40 ms of uninterrupted work (the device's clock
        # management; the HBM-bound decode launches show no such drift), so about 70 ms of calls
        # run untimed first, then 12 groups of four calls back to back
        warm = max(16, min(int(70e3 / max(single[len(single) // 2], 1.0)), 2000))
        for _ in range(warm):
            call()
        groups = [timed(4) for _ in range(12)]
        torch.cuda.synchronize()
        ts = sorted(e0.elapsed_time(e1) * 1e3 / 4 for e0, e1 in groups)
        us = ts[len(ts) // 2]
        keys = sum(base + i + 1 for i in range(chunk))
        flops = 4 * keys * q_dim
        row = {"workload": "%s, %s element: %d-row chunk over %d cached rows (append + attention + merge; a stream of calls, four per event pair, after 70 ms of them)"
                           % (name, element, chunk, base),
               "us": round(us, 1), "us_single_call_from_idle": round(single[len(single) // 2], 1),
               "algorithmic_tflops": round(flops / us / 1e6, 1)}
        if f32:
            row["frac_of_f32_mfma_peak"] = round(flops / us / 1e6 / 157.3, 4)
        else:
            row["mfma_tflops_issued"] = round(2 * flops / us / 1e6, 1)
            row["frac_of_bf16_mfma_peak"] = round(2 * flops / us / 1e6 / 2500.0, 4)
            row["issued_vs_recorded_product_stream"] = round(2 * flops / us / 1e6 / MFMA_STREAM_RANDOM_TFLOPS, 4)
        out.append(row)
        kv.close()
    return out


def bench_end_to_end(skv, torch, np, state):
    """BASELINE.json configs[1] end to end: the random-init Qwen3-4B-shaped decoder of the
    parity test (tests/config1_hip.py, which never touches the CPU oracle) with its KV path on the library; 2048-token prompt in
    512-row chunks, then greedy steps. Everything outside the KV path (embedding, projections,
    MLP, norms, lm_head) is plain torch fp32 and only there to drive the KV path at its real
    place in a decoder: the tok/s is dominated by those fp32 matrix products."""
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests"))
    from config1_hip import Config, HipKvPre, Weights, forward
    cfg = Config()
    n_prompt, n_new, chunk = 2048, 64, 512
    with torch.no_grad():
        w = Weights(cfg, seed=1)
        prompt = [int(t) for t in np.random.default_rng(1).integers(0, cfg.vocab, size=n_prompt)]
        kv = HipKvPre(cfg, n_prompt + n_new + 8, state)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        position, logits = 0, None
        for i in range(0, n_prompt, chunk):
            logits = forward(cfg, w, kv, prompt[i:i + chunk], position)
            position += chunk
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ids = []
        for _ in range(n_new):
            tok = int(torch.argmax(logits))
            ids.append(tok)
            logits = forward(cfg, w, kv, [tok], position)
            position += 1
        torch.cuda.synchronize()
        t2 = time.perf_counter()
    return {"workload": "configs[1] end to end: 36 layers, 2048-token prompt in 512-row chunks, %d greedy "
                        "steps; KV path (q/k norm + rotation, append, attention) on the library, the rest "
                        "torch fp32" % n_new,
            "prefill_tok_per_s": round(n_prompt / (t1 - t0), 1),
            "decode_tok_per_s": round(n_new / (t2 - t1), 1),
            "decode_ms_per_token": round((t2 - t1) * 1e3 / n_new, 3),
            "distinct_ids": len(set(ids))}


class _TimedHot:
    """HotCache with HIP events around the calls the serve path makes, so that the restore and
    snapshot legs of a turn can be told apart afterwards."""

    def __init__(self, hot, torch):
        self._hot, self._torch = hot, torch
        self.restore_ev, self.snap_ev = [], []

    def __getattr__(self, name):
        return getattr(self._hot, name)

    def _timed(self, bucket, fn, *a, **kw):
        e0 = self._torch.cuda.Event(enable_timing=True)
        e1 = self._torch.cuda.Event(enable_timing=True)
        e0.record()
        r = fn(*a, **kw)
        e1.record()
        bucket.append((e0, e1, r))
        return r

    def match_restore(self, *a, **kw):
        return self._timed(self.restore_ev, self._hot.match_restore, *a, **kw)

    def remember_prefix_block(self, *a, **kw):
        return self._timed(self.snap_ev, self._hot.remember_prefix_block, *a, **kw)

    def remember_prefix_blocks(self, *a, **kw):
        return self._timed(self.snap_ev, self._hot.remember_prefix_blocks, *a, **kw)


def _percentile(values, q):
    """percentile of bench-serve's summary (src/bench_serve.rs:284-285): nearest rank on the sorted values."""
    if not values:
        return 0.0
    v = sorted(values)
    return v[min(len(v) - 1, max(0, int(round(q * (len(v) - 1)))))]


def config3_traffic(np):
    """The seeded request stream of BASELINE.json configs[3]: 8 sessions share a 4096-token
    prefix, each sends prefix + history (256..1024 tokens), then the same plus a 512-token turn."""
    n_sessions, vocab = 8, 151936
    rng = np.random.default_rng(3)
    shared = rng.integers(0, vocab, size=4096)
    hist = [rng.integers(0, vocab, size=int(rng.integers(256, 1025))) for _ in range(n_sessions)]
    turn = [rng.integers(0, vocab, size=512) for _ in range(n_sessions)]
    return shared, hist, turn


def restore_cpu_baseline(np, seconds):
    """The reference's CPU path at the prefix-cache boundary: remember_prefix_block clones the whole
    f32 prompt state (src/serve/state.rs:613-639) and match_prefix clones the hit's state
    (src/serve/cache.rs:121-151). The oracle's state clone is a deep copy of [n, kv_dim] f32 K and
    V per layer; timed here for the 4096-token boundary of configs[3] (36 layers, kv8/hd128), a
    bounded sample scaled to the 36 layers."""
    import oracle
    qh, kvh, hd, nl, n = 32, 8, 128, 36, 4096
    kv_dim = kvh * hd
    k = np.ones((n, kv_dim), np.float32)
    caches = []
    for _ in range(4):
        c = oracle.LayerKvCache("f32")
        c.append_batch(k, k, oracle.layout(qh, kvh, hd))
        caches.append(c)
    c0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - c0 < seconds:
        for c in caches:
            c.clone()
        reps += 1
    dt = (time.perf_counter() - c0) / reps / len(caches) * nl
    payload_f32 = n * kv_dim * 4 * 2 * nl
    return {"value": round(payload_f32 / dt / 1e9, 2), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "deep copy of one layer's f32 K/V at 4096 rows, %d x 4 copies timed, scaled to %d "
                      "layers: %.1f ms per cloned 4096-token state (the reference clones one per block "
                      "boundary and one per hit)" % (reps, nl, dt * 1e3)}


def bench_config3(args, skv, torch, np, state, stream):
    """BASELINE.json configs[3]: 8 sessions share a 4096-token prefix, each adds a 256..1024
    token history and then a 512-token turn; 16-token hash blocks over 36 layers of Qwen3-4B
    KV; the page pool holds 60 % of the distinct blocks the traffic produces, so the LRU
    evicts. Every turn runs the serve-side boundary algorithm (match + restore of the hit,
    chunked append of the rest, snapshot of the new blocks) and then checks every row of every
    layer against its re-derived value, bit for bit."""
    qh, kvh, hd, nl, bt, n_sessions, vocab = 32, 8, 128, 36, 16, 8, 151936
    kv_dim = kvh * hd
    dev = torch.device("cuda:0")
    shared, hist, turn = config3_traffic(np)
    base = len(shared) // bt
    demand = base + sum((len(shared) + len(h) + len(t)) // bt - base for h, t in zip(hist, turn))
    pool_blocks = int(demand * 0.6)

    def rows_of(layer, tokens, which):
        """K (which=0) or V (which=1) rows of a prompt: a function of the layer, the position
        and the tokens up to it, so equal prefixes give equal rows and nothing else does."""
        t = torch.from_numpy(np.asarray(tokens, dtype=np.int64)).to(dev)
        c = torch.cumsum(t * 2654435761 % 1000003, 0)
        pos = torch.arange(t.numel(), device=dev, dtype=torch.int64)
        d = torch.arange(kv_dim, device=dev, dtype=torch.int64)
        x = (pos[:, None] * 7919 + c[:, None] * 104729 + d[None, :] * 31 + layer * 1299709 + which * 15485863)
        x = (x * 6364136223846793005 + 1442695040888963407) >> 40
        return ((x & 0xffff).to(torch.float32) / 65536.0 - 0.5) * 4.0

    def make_layers(cap, seed):
        out = []
        for i in range(nl):
            kv = state.full_attention_bf16(cap, qh, kvh, hd)
            kv.set_block_table(np.random.default_rng(seed * 100 + i).permutation(kv.pages()).astype(np.int32))
            out.append(kv)
        return out

    proto = make_layers(16, 0)
    hot = _TimedHot(skv.HotCache(state, bt, 10 ** 6, pool_blocks, proto), torch)
    model = skv.LoadedModelKv(hot, enabled=True)
    block_payload = nl * 2 * bt * kv_dim * 2
    tot = dict(restore_us=0.0, restored_blocks=0, snap_us=0.0, snap_blocks=0, append_us=0.0,
               appended_rows=0, reused=0, prompt=0, hits=0, turns=0)
    gk = torch.empty(5700, kv_dim, device=dev, dtype=torch.int16)
    gv = torch.empty(5700, kv_dim, device=dev, dtype=torch.int16)

    # One set of caches serves every turn, emptied in between: a server leases its KV buffers
    # from an arena (DecodeResidentState::full_attention, src/decode_resident/attention.rs:26-108)
    # rather than allocating per request, and copies into memory that was never touched since
    # its allocation run at about half the rate.
    n_decode = 128   # generated tokens per request (DEFAULT_MAX_TOKENS, src/bench_serve.rs:34)
    max_tokens = len(shared) + 1024 + 512 + 16 + n_decode
    layers = make_layers(max_tokens, 1)
    dq = torch.randn(nl, qh * hd, device=dev, dtype=torch.float32)
    dk = torch.randn(nl, kv_dim, device=dev, dtype=torch.float32)
    dv = torch.randn(nl, kv_dim, device=dev, dtype=torch.float32)
    dout = torch.empty(nl, qh * hd, device=dev, dtype=torch.float32)

    def run_turn(tokens, seed):
        n = len(tokens)
        for kv in layers:
            kv.truncate(0)
        ks = [rows_of(i, tokens, 0) for i in range(nl)]
        vs = [rows_of(i, tokens, 1) for i in range(nl)]
        torch.cuda.synchronize()
        app_ev = []

        def prefill_rows(first, last):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for i, kv in enumerate(layers):
                kv.encode_append_batch(stream, ks[i][first].data_ptr(), vs[i][first].data_ptr(), last - first)
            e1.record()
            app_ev.append((e0, e1, last - first))

        hot.restore_ev.clear()
        hot.snap_ev.clear()
        reused = model.prefill_prompt_state(tokens, None, layers, prefill_rows, stream=stream,
                                            blocks_per_chunk=32)   # 512-row prefill chunks
        torch.cuda.synchronize()
        for e0, e1, r in hot.restore_ev:
            if r[0]:
                tot["restore_us"] += e0.elapsed_time(e1) * 1e3
                tot["restored_blocks"] += r[0] // bt
        for e0, e1, r in hot.snap_ev:
            tot["snap_us"] += e0.elapsed_time(e1) * 1e3
            tot["snap_blocks"] += int(r)
        for e0, e1, rows in app_ev:
            tot["append_us"] += e0.elapsed_time(e1) * 1e3
            tot["appended_rows"] += rows
        tot["reused"] += reused
        tot["prompt"] += n
        tot["hits"] += 1 if reused else 0
        tot["turns"] += 1
        # one line per request, the figures `saragossa serve` returns as x-saragossa-* headers
        # (ServedCompletion::metric_headers, src/serve/state.rs:59-80) and bench-serve collects
        # per request (src/bench_serve.rs:249-289), restricted to what the KV side does
        r_us = sum(e0.elapsed_time(e1) * 1e3 for e0, e1, r in hot.restore_ev if r[0])
        s_us = sum(e0.elapsed_time(e1) * 1e3 for e0, e1, r in hot.snap_ev)
        a_us = sum(e0.elapsed_time(e1) * 1e3 for e0, e1, rows in app_ev)
        requests.append({"index": len(requests), "ok": True, "prompt_tokens": n,
                         "reused_prefix_tokens": int(reused), "prefill_kv_us": round(r_us + s_us + a_us, 1),
                         "restore_us": round(r_us, 1), "snapshot_us": round(s_us, 1),
                         "append_us": round(a_us, 1), "appended_rows": sum(rows for _, _, rows in app_ev)})
        # bit-exact contents after the turn: restored and appended rows alike
        for i, kv in enumerate(layers):
            if kv.len() != n:
                raise RuntimeError("config 3: layer %d holds %d rows, expected %d" % (i, kv.len(), n))
            kv.encode_gather(stream, 0, n, gk.data_ptr(), gv.data_ptr())
            wk = ks[i].to(torch.bfloat16).view(torch.int16)
            wv = vs[i].to(torch.bfloat16).view(torch.int16)
            if not (torch.equal(gk[:n], wk) and torch.equal(gv[:n], wv)):
                raise RuntimeError("config 3: cache contents differ from the re-derived rows "
                                   "(layer %d, %d reused tokens)" % (i, reused))
        # the request's decode phase on the KV side: n_decode tokens, each one fused append +
        # attention step per layer over the prompt just restored and appended (decode_tok_s of
        # bench-serve's RequestReport, src/bench_serve.rs:292-305, without the model around it)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n_decode):
            for i, kv in enumerate(layers):
                kv.encode_decode_step(stream, dk[i].data_ptr(), 0, dv[i].data_ptr(), 0, dq[i].data_ptr(),
                                      dout[i].data_ptr())
        e1.record()
        torch.cuda.synchronize()
        requests[-1]["generated_tokens"] = n_decode
        requests[-1]["decode_kv_tok_s"] = round(n_decode / (e0.elapsed_time(e1) * 1e-3), 1)
        return reused

    requests = []
    t0 = time.perf_counter()
    for s_ in range(n_sessions):
        run_turn(np.concatenate([shared, hist[s_]]), 10 + s_)
    for s_ in range(n_sessions):
        run_turn(np.concatenate([shared, hist[s_], turn[s_]]), 30 + s_)
    wall = time.perf_counter() - t0
    restore_traffic = 2 * tot["restored_blocks"] * block_payload
    snap_traffic = 2 * tot["snap_blocks"] * block_payload
    r_gbps = restore_traffic / max(tot["restore_us"], 1e-9) / 1e3
    s_gbps = snap_traffic / max(tot["snap_us"], 1e-9) / 1e3
    result = {
        "metric": "prefix block restore GB/s (multi-turn hot cache, match + gather of the hit blocks)",
        "value": round(restore_traffic / 2 / max(tot["restore_us"], 1e-9) / 1e3, 1),
        "unit": "GB/s", "n_gpus": 1, "steps": tot["turns"], "warmup": 0,
        "ms_per_step": round(wall * 1e3 / tot["turns"], 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
        "config": {"workload": "configs[3]: 8 sessions x 2 turns, shared 4096-token prefix, histories of "
                               "256..1024 tokens, 512-token turns, 16-token hash blocks, 36 layers kv8/hd128 "
                               "bf16, pool = 60 %% of %d distinct blocks" % demand,
                   "pool_blocks": pool_blocks, "block_bytes": block_payload},
        "turns_with_hit": tot["hits"], "reused_tokens": tot["reused"], "prompt_tokens": tot["prompt"],
        "evictions": hot.evictions(), "skipped": hot.skipped(), "cached_blocks": len(hot._hot),
        "restore": {"blocks": tot["restored_blocks"], "us": round(tot["restore_us"], 1),
                    "traffic_gbps": round(r_gbps, 1)},
        "snapshot": {"blocks": tot["snap_blocks"], "us": round(tot["snap_us"], 1),
                     "traffic_gbps": round(s_gbps, 1)},
        "append": {"rows": tot["appended_rows"], "us": round(tot["append_us"], 1),
                   "us_per_row_all_layers": round(tot["append_us"] / max(tot["appended_rows"], 1), 3)},
        "contents": "bit-exact after every turn (every row of every layer re-derived and compared)",
        "serve_report": {
            "summary": {"requested": len(requests), "succeeded": sum(r["ok"] for r in requests),
                        "failed": sum(not r["ok"] for r in requests), "concurrency": 1,
                        "prefill_kv_p50_us": round(_percentile([r["prefill_kv_us"] for r in requests], 0.50), 1),
                        "prefill_kv_p95_us": round(_percentile([r["prefill_kv_us"] for r in requests], 0.95), 1),
                        "decode_kv_tok_s_mean": round(sum(r["decode_kv_tok_s"] for r in requests) / len(requests), 1),
                        "prompt_tokens": tot["prompt"], "reused_prefix_tokens": tot["reused"],
                        "total_ms": round(wall * 1e3, 1)},
            "requests": requests},
        "roofline": {"bound": "hbm", "kernel": "page_copy_kernel (restore of the hit blocks, host hash walk included)",
                     "achieved": round(r_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(r_gbps / HBM_PEAK_GBPS, 4), "traffic": None},
    }
    hot.close()
    for kv in proto + layers:
        kv.close()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = restore_cpu_baseline(np, min(args.cpu_seconds, 10.0))
    print(json.dumps(result))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--config", type=int, default=2, choices=sorted(WORKLOADS) + [3])
    ap.add_argument("--context", type=int, default=0, help="override the cached rows")
    ap.add_argument("--batch", type=int, default=1,
                    help="independent sequences decoded together (configs[4] also asks for 4)")
    ap.add_argument("--element", choices=["bf16", "f32"], default="bf16",
                    help="element of the decode leg's caches (f32 is the reference's choice for greedy decoding)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-restore", action="store_true")
    ap.add_argument("--no-legs", action="store_true",
                    help="default run only: skip the configs[4] batch-4 and f32-element legs and the SDPA length sweep")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--end-to-end", action="store_true",
                    help="with --config 1: also run the whole random-init decoder and report tok/s")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; every figure is one MI355X's throughput "
              "(--gpus must be 1)", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    import saragossa_amd as skv

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the KV path has no CPU fallback", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.config == 3:
        return bench_config3(args, skv, torch, np, skv.DecodeResidentState(0),
                             torch.cuda.current_stream().cuda_stream)
    if args.batch < 1:
        print("bench.py: --batch must be at least 1", file=sys.stderr)
        return 2
    state = skv.DecodeResidentState(0)
    result = decode_bench(args, skv, torch, np, state, main_leg=True)
    if args.config == 2 and args.batch == 1 and args.element == "bf16" and not args.context and not args.no_legs:
        # Further legs of the default run, each timed like the headline and reported with its own
        # roofline object: BASELINE configs[4] at batch 4 (one launch pair per layer covers the
        # four sequences) and configs[2] on the cache's f32 element (the reference's choice for
        # greedy decoding). Fewer steps than the headline: they only have to be steady.
        import argparse as _ap
        legs = {}
        for key, over in (("configs4_batch4", dict(config=4, batch=4, element="bf16", steps=min(args.steps, 32), warmup=4)),
                          ("configs2_f32_element", dict(config=2, batch=1, element="f32", steps=min(args.steps, 64), warmup=4))):
            ns = _ap.Namespace(**vars(args))
            for k, v in over.items():
                setattr(ns, k, v)
            ns.no_cpu_baseline = True
            leg = decode_bench(ns, skv, torch, np, state, main_leg=False)
            legs[key] = {k: leg[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step", "dtype", "config",
                                             "tok_per_s", "hbm_gbps", "hbm_frac", "roofline", "checked_max_abs")
                         if k in leg}
            if "ceiling" in leg:
                legs[key]["ceiling"] = leg["ceiling"]
        result["legs"] = legs
    print(json.dumps(result))
    return 0


def decode_bench(args, skv, torch, np, state, main_leg):
    """One decode workload (args.config, args.batch, args.element): builds the caches, times
    args.steps steps after args.warmup, checks the last context against float64 softmax
    attention, times the attention launches with HIP events, and returns the result object.
    The restore, recurrent-state, prefill and CPU legs only run for the main leg."""
    import ctypes as C
    dev = torch.device("cuda:0")
    ELEM_BYTES = 4 if args.element == "f32" else 2

    def algorithmic(rows, kv_dim_, q_dim_, with_append):
        return algorithmic_bytes(rows, kv_dim_, q_dim_, with_append, ELEM_BYTES)

    wl = WORKLOADS[args.config]
    no_cpu = args.no_cpu_baseline or not main_leg
    no_restore = args.no_restore or not main_leg
    if len(wl["groups"]) > 1:
        no_cpu = True   # the CPU sample is scaled by identical layers only
    groups = [(n, qh_, kvh_, hd_, args.context or ctx_, w_) for n, qh_, kvh_, hd_, ctx_, w_ in wl["groups"]]
    qh, kvh, hd = groups[0][1:4]     # all groups of a workload share the head shape
    kv_dim, q_dim = kvh * hd, qh * hd
    ctx_rows = groups[0][4]
    layers_n = sum(g[0] for g in groups)
    total_steps = args.warmup + args.steps

    gen = torch.Generator(device=dev)
    gen.manual_seed(args.config)
    rng = np.random.default_rng(args.config)
    stream = torch.cuda.current_stream().cuda_stream
    B = args.batch
    if B > 1:
        no_cpu = True   # the CPU sample is one sequence
    layers = []       # one handle per (layer, sequence), layer-major
    layer_rows = []   # rows each layer attends per step (for the byte count)
    host_kv = []      # first layer's f32 rows, kept for the CPU baseline
    for n, _, _, _, rows, window in groups:
        for _ in range(n):
            for _ in range(B):   # every sequence owns its pages and its block table
                kv = state.full_attention_with_element(rows + 3 * total_steps + 8, qh, kvh, hd,
                                                       skv.DTYPE_F32 if args.element == "f32" else skv.DTYPE_BF16,
                                                       window)
                kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
                fill = min(rows, window) if window else rows   # a ring only keeps its window
                k = torch.randn(fill, kv_dim, device=dev, dtype=torch.float32, generator=gen)
                v = torch.randn(fill, kv_dim, device=dev, dtype=torch.float32, generator=gen)
                kv.encode_append_batch(stream, k.data_ptr(), v.data_ptr(), fill)
                torch.cuda.synchronize()
                if not layers and not no_cpu:
                    host_kv = [k.cpu().numpy(), v.cpu().numpy()]
                del k, v
                layers.append(kv)
            layer_rows.append(fill)

    # the ring layers between two global layers share a geometry: a caller that holds the q/k/v of
    # several of them at once can step them in one launch pair (informational leg, see below)
    grouped_leg = B == 1 and any(g[5] for g in groups) and any(not g[5] for g in groups)
    n_pass = (3 if grouped_leg else 2) * total_steps  # timed pass + per-kernel pass (+ grouped pass)
    n_units = layers_n * B   # (layer, sequence) pairs, layer-major
    q_all = torch.randn(n_pass, n_units, q_dim, device=dev, dtype=torch.float32, generator=gen)
    k_all = torch.randn(n_pass, n_units, kv_dim, device=dev, dtype=torch.float32, generator=gen)
    v_all = torch.randn(n_pass, n_units, kv_dim, device=dev, dtype=torch.float32, generator=gen)
    out = torch.empty(n_units, q_dim, device=dev, dtype=torch.float32)
    torch.cuda.synchronize()

    lib = skv.lib()
    PtrArr = C.c_void_p * n_units
    layer_arr = PtrArr(*[l._h.value for l in layers])
    out_arr = PtrArr(*[out[i].data_ptr() for i in range(n_units)])

    def ptrs(t, step):
        base, stride = t[step].data_ptr(), t.stride(1) * 4
        return PtrArr(*[base + i * stride for i in range(n_units)])

    step_ptrs = [(ptrs(k_all, s), ptrs(v_all, s), ptrs(q_all, s)) for s in range(n_pass)]
    vpp = C.POINTER(C.c_void_p)

    def at(arr, li):   # the B pointers of layer li inside a layer-major array
        return C.cast(C.byref(arr, li * B * C.sizeof(C.c_void_p)), vpp)

    def run_step(s):
        kp, vp, qp = step_ptrs[s]
        if B == 1:
            rc = lib.skv_decode_step_layers_device(layer_arr, layers_n, stream, kp, vp, qp, out_arr)
            if rc:
                raise RuntimeError(lib.skv_last_error().decode())
            return
        for li in range(layers_n):   # one launch pair per layer covers the B sequences
            rc = lib.skv_decode_step_batch_device(at(layer_arr, li), B, stream, at(kp, li), at(vp, li),
                                                  at(qp, li), at(out_arr, li))
            if rc:
                raise RuntimeError(lib.skv_last_error().decode())

    for s in range(args.warmup):
        run_step(s)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.warmup, total_steps):
        run_step(s)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    step_us = ms_per_step * 1e3
    # Proof that the timed kernels did the work: the context the last timed step left for layer 0
    # (sequence 0), against textbook softmax attention in float64 (torch, on the device) over the
    # rows read back from that layer's cache; shares nothing with the library's kernels or the
    # CPU oracle.
    kv0 = layers[0]
    gk, gv = kv0.read_rows_f32()
    n0 = gk.shape[0]
    Kd = torch.from_numpy(gk).to(dev).double().view(n0, kvh, hd)
    Vd = torch.from_numpy(gv).to(dev).double().view(n0, kvh, hd)
    qd = q_all[total_steps - 1, 0].double().view(kvh, qh // kvh, hd)
    prob = torch.softmax(torch.einsum("kgd,nkd->kgn", qd, Kd) / hd ** 0.5, dim=-1)
    ref = torch.einsum("kgn,nkd->kgd", prob, Vd).reshape(-1)
    checked_max_abs = float((out[0].double() - ref).abs().max())
    del Kd, Vd, prob, ref, gk, gv
    if not checked_max_abs <= 1e-4:
        raise RuntimeError("bench: the last timed step's context of layer 0 differs from float64 softmax "
                           "attention over the cached rows by %.3e (> 1e-4)" % checked_max_abs)
    us_per_token = step_us / B   # a step yields one token per sequence
    mid = args.warmup + args.steps // 2
    step_bytes = B * sum(algorithmic(min(r + mid, w) if w else r + mid, kv_dim, q_dim, True)
                         for r, w in zip(layer_rows, [g[5] for g in groups for _ in range(g[0])]))

    # ---- per-kernel pass on the launch stream: the ten appends of a token first, then HIP
    # events around the ten attention launches (one per layer) so that the cost of recording
    # an event is spread over ten launches
    # (with a batch the launch is the fused step of the B sequences of one layer)
    evs = []
    for s in range(total_steps, total_steps + args.steps):
        kp, vp, qp = step_ptrs[s]
        if B == 1:
            for li, kv in enumerate(layers):
                kv.encode_append_kv(stream, kp[li], vp[li])
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        if B == 1:
            for li, kv in enumerate(layers):
                ws = max(kv.len() - kv.window(), 0) if kv.window() else 0
                kv.encode_attention_decode_windowed(stream, qp[li], out_arr[li], ws)
        else:
            run_step(s)
        e1.record()
        evs.append((e0, e1))
    torch.cuda.synchronize()
    kern_ms = sorted(e0.elapsed_time(e1) / layers_n for e0, e1 in evs)
    kern_avg_us = sum(kern_ms) / len(kern_ms) * 1e3
    kern_med_us = kern_ms[len(kern_ms) // 2] * 1e3

    # ---- what the hardware allows at this size: a launch per layer that only fetches the same
    # K and V pages (same grid, same access pattern, nothing computed, nothing merged), and an
    # empty launch; timed the same way, ten launches between two events
    ceiling = None
    if B == 1:
        def timed_launches(fn, per_pair):
            pairs = []
            for _ in range(max(args.steps // 2, 20)):
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                pairs.append((e0, e1))
            torch.cuda.synchronize()
            ts = sorted(a.elapsed_time(b) * 1e3 / per_pair for a, b in pairs[3:])
            return ts[len(ts) // 2]

        def read_all():
            for kv in layers:
                kv.encode_probe_read_pages(stream)

        def empty_all():
            for _ in layers:
                state.encode_probe_empty_launch(stream)

        def read_then_merge_all():
            # the launch pair of a layer with nothing multiplied: the read-only launch, then the
            # merge launch of a decode step over the partials the last attention call left
            for li, kv in enumerate(layers):
                kv.encode_probe_read_pages(stream)
                kv.encode_probe_merge(stream, out_arr[li])

        def read_store_then_merge_all():
            # the same pair when the first launch also leaves a split partial per workgroup, as
            # any split-K launch must before a merge can run
            for li, kv in enumerate(layers):
                kv.encode_probe_read_store_pages(stream)
                kv.encode_probe_merge(stream, out_arr[li])

        read_us = timed_launches(read_all, layers_n)
        empty_us = timed_launches(empty_all, layers_n)
        pair_us = timed_launches(read_then_merge_all, layers_n)
        pair_store_us = timed_launches(read_store_then_merge_all, layers_n)
        kv_bytes = sum(2 * min(kv.len(), kv.window() or kv.len()) * kv_dim * ELEM_BYTES for kv in layers) // layers_n
        ceiling = {"read_only_launch_us": round(read_us, 2),
                   "read_only_gbps": round(kv_bytes / read_us / 1e3, 1),
                   "read_only_frac_of_peak": round(kv_bytes / read_us / 1e3 / HBM_PEAK_GBPS, 4),
                   "empty_launch_us": round(empty_us, 2),
                   "attention_vs_read_only": round(read_us / kern_avg_us, 3),
                   "read_then_merge_launch_pair_us": round(pair_us, 2),
                   "attention_vs_read_then_merge": round(pair_us / kern_avg_us, 3),
                   "read_store_then_merge_launch_pair_us": round(pair_store_us, 2),
                   "attention_vs_read_store_then_merge": round(pair_store_us / kern_avg_us, 3),
                   "note": "a launch per layer that only fetches the cached K/V pages with the decode "
                           "kernel's grid and access pattern (no products, no partials, no merge); "
                           "read_then_merge: that launch followed by the merge launch of a decode step, "
                           "the pair of dependent launches an attention call cannot be cheaper than; "
                           "read_store_then_merge: the same with a split partial of the decode kernel's size "
                           "written by every workgroup of the first launch"}
    grouped = None
    if grouped_leg:
        # Informational, never `value`: the same token with the ring layers stepped five at a time
        # through skv_decode_step_batch_device (handles of one geometry and window, here layers
        # instead of sequences), the global layers one by one as before. Only a caller that holds
        # the q/k/v of those five layers at once can do this; a decoder whose layer l+1 consumes
        # layer l's output cannot, which is why the headline figure does not.
        windows = [g[5] for g in groups for _ in range(g[0])]
        ring_ix = [i for i, w in enumerate(windows) if w]
        glob_ix = [i for i, w in enumerate(windows) if not w]
        per_call = 5
        n_glob = len(glob_ix)
        GArr = C.c_void_p * n_glob

        def pick(arr, ix):
            return (C.c_void_p * len(ix))(*[arr[i] for i in ix])

        glob_layers = pick(layer_arr, glob_ix)
        glob_out = pick(out_arr, glob_ix)
        ring_calls = [ring_ix[i:i + per_call] for i in range(0, len(ring_ix), per_call)]
        ring_layers = [pick(layer_arr, ix) for ix in ring_calls]
        ring_out = [pick(out_arr, ix) for ix in ring_calls]

        def run_grouped(st):
            kp, vp, qp = step_ptrs[st]
            rc = lib.skv_decode_step_layers_device(glob_layers, n_glob, stream, pick(kp, glob_ix), pick(vp, glob_ix),
                                                   pick(qp, glob_ix), glob_out)
            if rc:
                raise RuntimeError(lib.skv_last_error().decode())
            for ix, la, oa in zip(ring_calls, ring_layers, ring_out):
                rc = lib.skv_decode_step_batch_device(la, len(ix), stream, pick(kp, ix), pick(vp, ix), pick(qp, ix), oa)
                if rc:
                    raise RuntimeError(lib.skv_last_error().decode())

        base_step = 2 * total_steps
        for st in range(base_step, base_step + args.warmup):
            run_grouped(st)
        torch.cuda.synchronize()
        g0 = time.perf_counter()
        for st in range(base_step + args.warmup, base_step + total_steps):
            run_grouped(st)
        torch.cuda.synchronize()
        g_us = (time.perf_counter() - g0) * 1e6 / args.steps
        g_mid = base_step + args.warmup + args.steps // 2
        g_bytes = sum(algorithmic(min(r + g_mid, w) if w else r + g_mid, kv_dim, q_dim, True)
                      for r, w in zip(layer_rows, windows))
        grouped = {"us_per_token": round(g_us, 2), "hbm_frac": round(g_bytes / g_us / 1e3 / HBM_PEAK_GBPS, 4),
                   "ring_layers_per_launch_pair": per_call,
                   "note": "informational, not `value`: the ring layers stepped five per launch pair through "
                           "skv_decode_step_batch_device, which needs the q/k/v of those layers at once; a "
                           "decoder whose next layer consumes this layer's output cannot call it that way"}

    # the dominant launch is a layer of the first group; with mixed groups the event pairs span
    # all layers, so bytes are summed over the layers and divided by the same time
    late = total_steps + args.steps // 2
    all_bytes = B * sum(algorithmic(min(r + late, w) if w else r + late, kv_dim, q_dim, B > 1)
                        for r, w in zip(layer_rows, [g[5] for g in groups for _ in range(g[0])]))
    launch_bytes = all_bytes // layers_n
    achieved = launch_bytes / (kern_avg_us * 1e-6) / 1e9
    cpu_inputs = None
    if not no_cpu:
        cpu_inputs = (k_all[:, 0].cpu().numpy(), v_all[:, 0].cpu().numpy(), q_all[:, 0].cpu().numpy())
    for kv in layers:
        kv.close()
    del layers, q_all, k_all, v_all
    torch.cuda.empty_cache()

    restore = None if (no_restore or args.config != 2) else bench_restore(skv, torch, np, state, stream, args.element)
    if restore is not None and not no_cpu:
        restore["cpu_baseline"] = restore_cpu_baseline(np, min(args.cpu_seconds, 10.0))
    recurrent = None
    if args.config == 2 and not no_restore:
        # configs[2]'s 30 linear-attention layers: their recurrent state (conv 96 KiB + ssm 2 MiB
        # each, f32) is snapshotted and restored as flat device-to-device copies
        sizes = [96 * 1024, 2 * 1024 * 1024] * 30
        bufs = [torch.randn(n // 4, device=dev, dtype=torch.float32, generator=gen) for n in sizes]
        want = [b.clone() for b in bufs]
        ptrs_ = [b.data_ptr() for b in bufs]
        ts, tr = [], []
        for it in range(12):
            e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            e0.record()
            snap = skv.state_snapshot(state, ptrs_, sizes, stream=stream)
            e1.record()
            for b in bufs:
                b.zero_()
            torch.cuda.synchronize()
            e1b = torch.cuda.Event(enable_timing=True)
            e1b.record()
            skv.state_restore(state, snap, ptrs_, sizes, stream=stream)
            e2.record()
            torch.cuda.synchronize()
            if it >= 2:
                ts.append(e0.elapsed_time(e1) * 1e3)
                tr.append(e1b.elapsed_time(e2) * 1e3)
            snap.close()
        if not all(torch.equal(a, b) for a, b in zip(bufs, want)):
            raise RuntimeError("recurrent state: restored bytes differ from the snapshotted bytes")
        ts.sort()
        tr.sort()
        tot_b = sum(sizes)
        recurrent = {"workload": "snapshot / restore of 30 recurrent states (96 KiB + 2 MiB each)",
                     "payload_mib": round(tot_b / 2 ** 20, 1),
                     "snapshot_us": round(ts[len(ts) // 2], 1), "restore_us": round(tr[len(tr) // 2], 1),
                     "snapshot_traffic_gbps": round(2 * tot_b / ts[len(ts) // 2] / 1e3, 1),
                     "restore_traffic_gbps": round(2 * tot_b / tr[len(tr) // 2] / 1e3, 1)}
        del bufs, want

    traffic = MEASURED_TRAFFIC_BYTES.get(args.config) if not args.context and B == 1 and args.element == "bf16" else None
    result = {
        "metric": "KV-path decode us/token @32k ctx (append + paged GQA SDPA, 10 KV layers)"
                  if args.config == 2 else "KV-path decode us/token (append + paged GQA SDPA)",
        "value": round(us_per_token, 2),
        "unit": "us/token",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.element,
        "data": "synthetic",
        "config": {"workload": (wl["name"] % ctx_rows) + ", %s KV in 16-token pages, batch %d, "
                               "1 token per sequence per step" % (args.element, B),
                   "context": ctx_rows, "layers": layers_n, "page_rows": 16, "batch": B},
        "tok_per_s": round(1e6 / us_per_token, 1),
        "hbm_gbps": round(step_bytes / (step_us * 1e-6) / 1e9, 1),
        "hbm_frac": round(step_bytes / (step_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "checked_max_abs": checked_max_abs,
        "checked": "context of layer 0 after the last timed step vs float64 softmax attention (torch) over "
                   "the rows read back from its cache; the run fails above 1e-4",
        "roofline": {"bound": "hbm", "kernel": ("f32_split_kernel<%d> + decode_merge_wave_kernel (one attention launch per "
                                                "sequence, average over the layers)" if args.element == "f32" else
                                                "decode_split_kernel<%d,8> + decode_merge_wave_kernel (one attention launch, "
                                                "average over the layers)" if B == 1 else
                                                "decode_split_batch_kernel<%d,8> + decode_merge_wave_batch_kernel (one launch pair "
                                                "per layer covers the batch, average over the layers)")
                                               % (128 if hd <= 128 else 256),
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "traffic_source": None if traffic is None else
                     "recorded figure, not observed by this run: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE over "
                     "this same command, scaled by a copy of known size (profiles/decode_split_kernel_config2.md)",
                     "bytes_per_launch": launch_bytes,
                     "avg_launch_us": round(kern_avg_us, 2), "median_launch_us": round(kern_med_us, 2),
                     "p10_launch_us": round(kern_ms[len(kern_ms) // 10] * 1e3, 2),
                     "p90_launch_us": round(kern_ms[len(kern_ms) * 9 // 10] * 1e3, 2)},
    }
    if ceiling is not None:
        result["ceiling"] = ceiling
    if grouped is not None:
        result["ring_layers_batched"] = grouped
    if restore is not None:
        result["restore"] = restore
    if recurrent is not None:
        result["recurrent_state"] = recurrent
    if args.config == 1 and args.end_to_end and main_leg:
        result["end_to_end"] = bench_end_to_end(skv, torch, np, state)
    if args.config == 2 and not no_restore:
        result["prefill"] = bench_prefill(skv, torch, np, state, stream, args.element)
        if not args.no_legs and args.element == "bf16":
            result["sdpa_sweep"] = bench_sdpa_sweep(skv, torch, np, state, stream)

    if not no_cpu:
        import oracle
        threads = oracle.default_threads(qh)
        lay = oracle.layout(qh, kvh, hd)
        cache = oracle.LayerKvCache("f32")
        cache.append_batch(host_kv[0], host_kv[1], lay)
        kq, vq, qq = cpu_inputs
        n_calls, t_cpu = 0, 0.0
        budget = args.cpu_seconds
        while t_cpu < budget and n_calls < 4096:
            i = n_calls % kq.shape[0]  # the synthetic rows again once they run out
            c0 = time.perf_counter()
            oracle.decode_step(cache, kq[i], vq[i], qq[i], lay, threads)
            t_cpu += time.perf_counter() - c0
            n_calls += 1
        cpu_us_per_token = t_cpu / n_calls * layers_n * 1e6
        result["cpu_baseline"] = {
            "value": round(cpu_us_per_token, 1), "unit": "us/token", "cores": threads,
            "kind": "port",
            "sample": "%d layer-steps of append + cached_attention_one on layer 0 (f32 cache, "
                      "%d rows) timed and scaled by %d layers; host has %d cores"
                      % (n_calls, ctx_rows, layers_n, os.cpu_count() or 0)}
    return result


if __name__ == "__main__":
    sys.exit(main())
