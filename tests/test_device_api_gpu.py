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
    assert kv.pages() == 2 and kv.window() == window
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
        kv.attention_decode_windowed(q, n - window - 1)  # older than the ring holds
    with pytest.raises(skv.DimensionError):
        kv.read_rows(0, 4)
    gk, _ = kv.read_rows_f32(n - window, window)
    assert np.array_equal(gk, cache.keys()[n - window:])
