"""Device-side entry points (raw device pointers + stream), against the CPU oracle:
encode_append_kv / encode_attention_decode (src/decode_resident/tests.rs:1657-1716,
1930-2018) and the fused per-token step, on full and ring-buffer layers."""
import numpy as np
import pytest

import oracle
import saragossa_amd as skv

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def test_encode_append_kv_device_matches_cpu(state):
    # src/decode_resident/tests.rs:1930-2018: device append == host append, same RNE rounding
    q_heads, kv_heads, head_dim = 16, 2, 256
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(11)
    host = state.full_attention_bf16(8, q_heads, kv_heads, head_dim)
    devl = state.full_attention_bf16(8, q_heads, kv_heads, head_dim)
    rows_k = rng.standard_normal((5, kv_dim), dtype=np.float32) * 3
    rows_v = rng.standard_normal((5, kv_dim), dtype=np.float32) * 3
    # device rows sit inside a larger buffer at a byte offset, like the fused QKV output
    pad = 24
    buf = _dev(np.concatenate([np.zeros(pad, np.float32), rows_k.reshape(-1), rows_v.reshape(-1)]))
    for r in range(5):
        host.append_row(rows_k[r], rows_v[r])
        k_off = (pad + r * kv_dim) * 4
        v_off = (pad + 5 * kv_dim + r * kv_dim) * 4
        devl.encode_append_kv_with_offsets(_stream(), buf.data_ptr(), k_off, buf.data_ptr(), v_off)
    assert devl.len() == 5
    torch.cuda.synchronize()
    hk, hv = host.read_rows()
    dk, dv = devl.read_rows()
    assert np.array_equal(hk, dk) and np.array_equal(hv, dv)
    assert np.array_equal(dk, oracle.f32_to_bf16_bits(rows_k))
    # overflow is an error, never a silent wrap (tests.rs:505-525)
    for _ in range(3):
        devl.encode_append_kv(_stream(), buf.data_ptr(), buf.data_ptr())
    with pytest.raises(skv.DimensionError):
        devl.encode_append_kv(_stream(), buf.data_ptr(), buf.data_ptr())
    assert devl.len() == 8


def test_resident_device_append_then_read_same_stream(state):
    # src/decode_resident/tests.rs:1664-1716: append then attention queued back to back
    q_heads, kv_heads, head_dim, n = 16, 2, 256, 40
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(12)
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    q = rng.standard_normal(q_heads * head_dim, dtype=np.float32)
    kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
    kv.seed(keys[:-1], values[:-1], n - 1)
    kd, vd, qd = _dev(keys[-1]), _dev(values[-1]), _dev(q)
    out = torch.empty(q_heads * head_dim, device="cuda", dtype=torch.float32)
    kv.encode_append_kv(_stream(), kd.data_ptr(), vd.data_ptr())
    kv.encode_attention_decode(_stream(), qd.data_ptr(), out.data_ptr())
    got = out.cpu().numpy()
    lay = oracle.layout(q_heads, kv_heads, head_dim)
    cache = oracle.LayerKvCache("bf16r")
    cache.append_batch(keys, values, lay)
    want = oracle.cached_attention_one(q, cache, lay)
    assert np.abs(got - want).max() <= 1e-4


@pytest.mark.parametrize("dims,window,start,steps", [
    ((16, 2, 256), 0, 700, 40),      # full cache, split-K, appended row crosses a page boundary
    ((32, 8, 128), 0, 5, 40),        # short cache, single split
    ((16, 8, 256), 64, 10, 200),     # ring layer: fills, wraps several times
    ((8, 2, 64), 48, 0, 120),        # ring from empty, window multiple of 16
    ((4, 2, 16), 20, 3, 70),         # window not a multiple of 16 (ring rounds up to 32 rows)
    ((8, 2, 512), 0, 600, 20),       # head_dim 512, split-K
    ((4, 2, 512), 32, 5, 60),        # head_dim 512 on a ring
])
def test_fused_decode_steps_match_oracle(state, dims, window, start, steps):
    """Token by token: the fused append+attention step equals LayerKvCache::append +
    cached_attention_one with the layer's sliding window; contents stay bit-exact."""
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(start + steps)
    cap = start + steps
    kv = state.full_attention_bf16(cap, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    if start:
        k0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        v0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        kv.seed(k0, v0, start)
        cache.append_batch(k0, v0, lay)
    ks = rng.standard_normal((steps, kv_dim), dtype=np.float32)
    vs = rng.standard_normal((steps, kv_dim), dtype=np.float32)
    qs = rng.standard_normal((steps, q_dim), dtype=np.float32)
    kd, vd, qd = _dev(ks), _dev(vs), _dev(qs)
    out = torch.empty(steps, q_dim, device="cuda", dtype=torch.float32)
    for t in range(steps):
        kv.encode_decode_step(_stream(), kd.data_ptr(), t * kv_dim * 4, vd.data_ptr(),
                              t * kv_dim * 4, qd[t].data_ptr(), out[t].data_ptr())
    got = out.cpu().numpy()
    worst = 0.0
    for t in range(steps):
        want = oracle.decode_step(cache, ks[t], vs[t], qs[t], lay)
        worst = max(worst, float(np.abs(got[t] - want).max()))
    assert worst <= 1e-4, worst
    assert kv.len() == len(cache) == cap
    # contents: the rows the layer still holds are bit-exact
    first = 0 if window == 0 else max(0, cap - (window + 15) // 16 * 16)
    gk, gv = kv.read_rows_f32(first, cap - first)
    assert np.array_equal(gk, cache.keys()[first:]) and np.array_equal(gv, cache.values()[first:])
    with pytest.raises(skv.DimensionError):
        kv.encode_decode_step(_stream(), kd.data_ptr(), 0, vd.data_ptr(), 0, qd.data_ptr(),
                              out.data_ptr())


def test_ring_layer_host_api(state):
    """Ring-buffer KV for a sliding layer equals the reference's full KV + window_start
    (src/decoder/resident/types.rs:13-18), and rows that left the ring are errors."""
    q_heads, kv_heads, head_dim, window = 8, 4, 128, 32
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(5)
    n = 100
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    kv = state.full_attention_bf16(128, q_heads, kv_heads, head_dim, window=window)
    assert kv.pages() == (window + 32) // 16 and kv.window() == window   # the window plus 32 rows of slack
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    kv.seed(keys[:70], values[:70], 70)      # a seed longer than the ring keeps its tail
    cache.append_batch(keys[:70], values[:70], lay)
    for r in range(70, n):
        kv.append_row(keys[r], values[r])
        cache.append(keys[r][None], values[r][None], lay)
        q = rng.standard_normal(q_heads * head_dim, dtype=np.float32)
        ws = skv.flags.window_start(r, window)
        assert ws == oracle.window_start(r, window) == r + 1 - window
        got = kv.attention_decode_windowed(q, ws)
        want = oracle.cached_attention_one(q, cache, lay)
        assert np.abs(got - want).max() <= 1e-4
    with pytest.raises(skv.DimensionError):
        kv.attention_decode_windowed(q, n - window - 33)  # older than the ring holds
    with pytest.raises(skv.DimensionError):
        kv.read_rows(0, 4)
    gk, _ = kv.read_rows_f32(n - window, window)
    assert np.array_equal(gk, cache.keys()[n - window:])


@pytest.mark.parametrize("dims,window,starts,steps", [
    ((16, 8, 256), 0, [4100, 33, 900, 0], 24),     # config 4's global shape: long, short (one split), empty
    ((16, 8, 256), 64, [500, 0, 70, 63], 40),      # ring layers at different fill levels and wraps
    ((32, 8, 128), 0, [260, 2000], 20),            # two sequences, Qwen3-4B shape
    ((8, 2, 64), 0, list(range(100, 1900, 100)), 6),  # 18 sequences: more than one launch's worth
    ((8, 2, 512), 0, [700, 20, 3000], 8),          # head_dim 512
])
def test_decode_step_batch_matches_oracle(state, dims, window, starts, steps):
    """A batch of independent sequences through skv_decode_step_batch_device: every sequence
    gets what its own append + cached_attention_one gives (same bound as the single-sequence
    step), contents stay bit-exact, and the batch agrees with single-sequence calls."""
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(len(starts) * 1000 + steps)
    n = len(starts)
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    seqs, twins, caches = [], [], []
    for start in starts:
        cap = start + steps
        kv = state.full_attention_bf16(cap, q_heads, kv_heads, head_dim, window=window)
        kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
        twin = state.full_attention_bf16(cap, q_heads, kv_heads, head_dim, window=window)
        cache = oracle.LayerKvCache("bf16r")
        if start:
            k0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
            v0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
            kv.seed(k0, v0, start)
            twin.seed(k0, v0, start)
            cache.append_batch(k0, v0, lay)
        seqs.append(kv)
        twins.append(twin)
        caches.append(cache)
    ks = rng.standard_normal((steps, n, kv_dim), dtype=np.float32)
    vs = rng.standard_normal((steps, n, kv_dim), dtype=np.float32)
    qs = rng.standard_normal((steps, n, q_dim), dtype=np.float32)
    kd, vd, qd = _dev(ks), _dev(vs), _dev(qs)
    out = torch.empty(steps, n, q_dim, device="cuda", dtype=torch.float32)
    single = torch.empty(steps, n, q_dim, device="cuda", dtype=torch.float32)
    for t in range(steps):
        skv.encode_decode_step_batch(
            seqs, _stream(), [kd[t, i].data_ptr() for i in range(n)],
            [vd[t, i].data_ptr() for i in range(n)], [qd[t, i].data_ptr() for i in range(n)],
            [out[t, i].data_ptr() for i in range(n)])
        for i in range(n):
            twins[i].encode_decode_step(_stream(), kd[t, i].data_ptr(), 0, vd[t, i].data_ptr(), 0,
                                        qd[t, i].data_ptr(), single[t, i].data_ptr())
    got, one = out.cpu().numpy(), single.cpu().numpy()
    # the two differ only in how many splits the context was cut into
    assert np.abs(got - one).max() <= 2e-6
    worst = 0.0
    for i in range(n):
        for t in range(steps):
            want = oracle.decode_step(caches[i], ks[t, i], vs[t, i], qs[t, i], lay)
            worst = max(worst, float(np.abs(got[t, i] - want).max()))
    assert worst <= 1e-4, worst
    for i, start in enumerate(starts):
        cap = start + steps
        assert seqs[i].len() == cap
        first = 0 if window == 0 else max(0, cap - (window + 15) // 16 * 16)
        gk, gv = seqs[i].read_rows_f32(first, cap - first)
        assert np.array_equal(gk, caches[i].keys()[first:])
        assert np.array_equal(gv, caches[i].values()[first:])


def test_decode_step_batch_errors(state):
    """Mixed geometries, a repeated handle and a full sequence are errors, and a failed call
    leaves every sequence as it was."""
    a = state.full_attention_bf16(40, 8, 2, 64)
    b = state.full_attention_bf16(40, 8, 2, 64)
    c = state.full_attention_bf16(40, 8, 4, 64)
    full = state.full_attention_bf16(4, 8, 2, 64)
    z = np.zeros((4, 2 * 64), np.float32)
    full.seed(z, z, 4)
    buf = torch.zeros(8 * 64, device="cuda", dtype=torch.float32)
    p = buf.data_ptr()
    with pytest.raises(skv.DimensionError):
        skv.encode_decode_step_batch([a, c], _stream(), [p, p], [p, p], [p, p], [p, p])
    with pytest.raises(skv.DimensionError):
        skv.encode_decode_step_batch([a, a], _stream(), [p, p], [p, p], [p, p], [p, p])
    with pytest.raises(skv.DimensionError):
        skv.encode_decode_step_batch([a, b, full], _stream(), [p] * 3, [p] * 3, [p] * 3, [p] * 3)
    with pytest.raises(skv.DeviceError):
        skv.encode_decode_step_batch([a, b], _stream(), [p, 0], [p, p], [p, p], [p, p])
    assert a.len() == 0 and b.len() == 0 and full.len() == 4
    out = torch.empty(2, 8 * 64, device="cuda", dtype=torch.float32)
    skv.encode_decode_step_batch([a, b], _stream(), [p, p], [p, p], [p, p],
                                 [out[0].data_ptr(), out[1].data_ptr()])
    torch.cuda.synchronize()
    assert a.len() == 1 and b.len() == 1
    assert np.array_equal(out.cpu().numpy(), np.zeros((2, 8 * 64), np.float32))  # one key: out == its V row


def test_prefill_chunk_device_with_unaligned_query_pointer(state):
    """The chunk's q rows may start at any 4-byte offset of a larger buffer: the kernel then
    takes the 4-byte query loads."""
    q_heads, kv_heads, head_dim, start, chunk = 16, 2, 128, 200, 40
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(77)
    lay = oracle.layout(q_heads, kv_heads, head_dim)
    results = []
    for pad in (0, 1, 3):
        kv = state.full_attention_bf16(start + chunk, q_heads, kv_heads, head_dim)
        cache = oracle.LayerKvCache("bf16r")
        r2 = np.random.default_rng(78)
        k0 = r2.standard_normal((start, kv_dim), dtype=np.float32)
        v0 = r2.standard_normal((start, kv_dim), dtype=np.float32)
        kv.seed(k0, v0, start)
        cache.append_batch(k0, v0, lay)
        q = r2.standard_normal((chunk, q_dim), dtype=np.float32)
        k = r2.standard_normal((chunk, kv_dim), dtype=np.float32)
        v = r2.standard_normal((chunk, kv_dim), dtype=np.float32)
        buf = _dev(np.concatenate([np.zeros(pad, np.float32), q.reshape(-1)]))
        kd, vd = _dev(k), _dev(v)
        out = torch.empty(chunk, q_dim, device="cuda", dtype=torch.float32)
        kv.encode_prefill_rows(_stream(), buf.data_ptr() + pad * 4, kd.data_ptr(), vd.data_ptr(), chunk,
                               out.data_ptr())
        got = out.cpu().numpy()
        want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
        assert np.abs(got - want).max() <= 1e-4
        results.append(got)
    assert np.array_equal(results[0], results[1]) and np.array_equal(results[0], results[2])


def test_attention_launches_replay_correctly_from_a_hip_graph(state):
    """The *_device entry points only queue kernels (no allocation, no synchronisation, no
    memset), so a caller may capture them in a HIP graph; what is captured is the work at the
    lengths of capture time. Several layers' attention captured once, replayed three times
    with eager work and synchronisations in between, each replay against the eager result
    (short context: single split; long context: split + merge)."""
    q_heads, kv_heads, head_dim = 16, 2, 256
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(21)
    layers = []
    for n in (100, 5000, 900):
        kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
        kv.seed(rng.standard_normal((n, kv_dim), dtype=np.float32),
                rng.standard_normal((n, kv_dim), dtype=np.float32), n)
        layers.append(kv)
    q = _dev(rng.standard_normal(q_dim, dtype=np.float32))
    outs = [torch.zeros(q_dim, device="cuda") for _ in layers]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):      # warm up outside the capture (lazy kernel attributes)
        for kv, o in zip(layers, outs):
            kv.encode_attention_decode(side.cuda_stream, q.data_ptr(), o.data_ptr())
    torch.cuda.synchronize()
    eager = [o.clone() for o in outs]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for kv, o in zip(layers, outs):
            kv.encode_attention_decode(side.cuda_stream, q.data_ptr(), o.data_ptr())
    for replay in range(3):
        for o in outs:
            o.fill_(float(replay))                                      # eager work between replays
        layers[0].encode_attention_decode(_stream(), q.data_ptr(), outs[0].data_ptr())
        torch.cuda.synchronize()
        outs[0].zero_()
        graph.replay()
        torch.cuda.synchronize()
        for o, e in zip(outs, eager):
            assert torch.equal(o, e), f"replay {replay}"


def test_measurement_probes_leave_the_cache_untouched(state):
    # the read-only, merge-only and empty launches that the benchmark times beside the attention
    # launch: they run on full and ring layers at ragged lengths and change nothing
    rng = np.random.default_rng(31)
    for (q_heads, kv_heads, head_dim), window, n in (((16, 2, 256), None, 1000), ((8, 2, 128), 64, 333),
                                                     ((8, 8, 64), None, 1), ((4, 1, 512), None, 47)):
        kv_dim = kv_heads * head_dim
        kv = state.full_attention_bf16(n + 4, q_heads, kv_heads, head_dim, window=window or 0)
        with pytest.raises(skv.DimensionError):
            kv.encode_probe_read_pages(_stream())
        kv.seed(rng.standard_normal((n, kv_dim), dtype=np.float32),
                rng.standard_normal((n, kv_dim), dtype=np.float32), n)
        first = max(0, n - window) if window else 0
        before = kv.read_rows(first)
        q = rng.standard_normal(q_heads * head_dim, dtype=np.float32)
        attend = (lambda: kv.attention_decode_windowed(q, first)) if window else (lambda: kv.attention_decode(q))
        want = attend()
        scratch_out = torch.empty(q_heads * head_dim, device="cuda")
        for _ in range(3):
            kv.encode_probe_read_pages(_stream())
            kv.encode_probe_merge(_stream(), scratch_out.data_ptr())
            state.encode_probe_empty_launch(_stream())
        torch.cuda.synchronize()
        after = kv.read_rows(first)
        assert np.array_equal(before[0], after[0]) and np.array_equal(before[1], after[1])
        assert np.array_equal(attend(), want)
        kv.close()
