"""skv_decode_step_static_device: the decode step whose split-K partials live in the library's
static device array (for callers that cannot allocate) against skv_decode_step_device, which
keeps them in the layer's own buffers. Same kernels, same split policy: contexts and cache
rows must be identical, on two calls in a row, the second with a smaller input (fewer splits,
narrower heads), so that what the first call left in the shared array is seen not to matter."""
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


def _pair(state, dims, rows, window, dtype, seed):
    """Two layers with the same rows behind the same permuted block table, and the oracle's cache."""
    q_heads, kv_heads, head_dim = dims
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(seed)
    keys = rng.standard_normal((rows, kv_dim), dtype=np.float32)
    values = rng.standard_normal((rows, kv_dim), dtype=np.float32)
    layers = []
    table = None
    for _ in range(2):
        kv = state.full_attention_with_element(rows + 64, q_heads, kv_heads, head_dim, dtype, window)
        if table is None:
            table = rng.permutation(kv.pages()).astype(np.int32)
        kv.set_block_table(table)
        kv.seed(keys, values, rows)
        layers.append(kv)
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r" if dtype == skv.DTYPE_BF16 else "f32")
    cache.append_batch(keys, values, lay)
    return layers, cache, lay, rng


def _steps(layers, cache, lay, rng, dims, n_steps):
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    static, plain = layers
    out_s = torch.empty(q_dim, device="cuda", dtype=torch.float32)
    out_p = torch.empty(q_dim, device="cuda", dtype=torch.float32)
    for _ in range(n_steps):
        k = rng.standard_normal(kv_dim, dtype=np.float32)
        v = rng.standard_normal(kv_dim, dtype=np.float32)
        q = rng.standard_normal(q_dim, dtype=np.float32)
        kd, vd, qd = _dev(k), _dev(v), _dev(q)
        static.encode_decode_step_static(_stream(), kd.data_ptr(), 0, vd.data_ptr(), 0, qd.data_ptr(),
                                         out_s.data_ptr())
        plain.encode_decode_step(_stream(), kd.data_ptr(), 0, vd.data_ptr(), 0, qd.data_ptr(),
                                 out_p.data_ptr())
        torch.cuda.synchronize()
        got_s, got_p = out_s.cpu().numpy(), out_p.cpu().numpy()
        assert np.array_equal(got_s, got_p)
        cache.append(k, v, lay)
        want = oracle.cached_attention_one(q, cache, lay)
        assert np.abs(got_s - want).max() <= 1e-4
    assert static.len() == plain.len() == len(cache)
    first = max(0, static.len() - 40)
    sk, sv = static.read_rows_f32(first, static.len() - first)
    pk, pv = plain.read_rows_f32(first, plain.len() - first)
    assert np.array_equal(sk, pk) and np.array_equal(sv, pv)
    assert np.array_equal(sk, cache.keys()[first:]) and np.array_equal(sv, cache.values()[first:])


@pytest.mark.parametrize("dtype", [skv.DTYPE_BF16, skv.DTYPE_F32])
def test_static_scratch_step_equals_the_allocating_one_twice_in_a_row(state, dtype):
    big = (16, 2, 256)      # 6000 rows: many splits, partials fill a good part of the array
    layers, cache, lay, rng = _pair(state, big, 6000, 0, dtype, 21)
    _steps(layers, cache, lay, rng, big, 3)
    small = (8, 4, 64)      # 300 rows right after: few splits, narrow heads, stale bytes all around
    layers2, cache2, lay2, rng2 = _pair(state, small, 300, 0, dtype, 22)
    _steps(layers2, cache2, lay2, rng2, small, 3)
    # and the first pair again: the array now holds the small call's partials
    _steps(layers, cache, lay, rng, big, 2)


def test_static_scratch_step_on_a_ring_layer_and_a_single_split(state):
    dims = (8, 2, 64)
    layers, cache, lay, rng = _pair(state, dims, 90, 48, skv.DTYPE_BF16, 23)   # ring, wraps
    _steps(layers, cache, lay, rng, dims, 30)
    layers, cache, lay, rng = _pair(state, dims, 20, 0, skv.DTYPE_BF16, 24)    # one split: no partials at all
    _steps(layers, cache, lay, rng, dims, 3)


def test_static_scratch_step_rejects_what_does_not_fit(state):
    # q_heads * splits * (head_dim + 2) * 4 bytes of partials: 128 heads of 512 dims with 64
    # splits are 16.8 MB, beyond the 8 MiB array; the layer is left as it was
    q_heads, kv_heads, head_dim, rows = 128, 4, 512, 64 * 64
    kv_dim = kv_heads * head_dim
    kv = state.full_attention_bf16(rows + 4, q_heads, kv_heads, head_dim)
    z = torch.zeros(rows, kv_dim, device="cuda", dtype=torch.float32)
    kv.encode_append_batch(_stream(), z.data_ptr(), z.data_ptr(), rows)
    q = torch.zeros(q_heads * head_dim, device="cuda", dtype=torch.float32)
    out = torch.empty_like(q)
    with pytest.raises(skv.DimensionError, match="tampon statique"):
        kv.encode_decode_step_static(_stream(), z.data_ptr(), 0, z.data_ptr(), 0, q.data_ptr(), out.data_ptr())
    assert kv.len() == rows
    torch.cuda.synchronize()


def test_static_scratch_step_on_wide_f32_heads_takes_the_separate_launches(state):
    """f32 rows of head_dim 512 have no fused append: the entry point appends, then attends with
    the partials in the static array (its other branch)."""
    dims = (16, 8, 512)
    layers, cache, lay, rng = _pair(state, dims, 2000, 0, skv.DTYPE_F32, 25)
    _steps(layers, cache, lay, rng, dims, 3)


@pytest.mark.parametrize("dtype", [skv.DTYPE_BF16, skv.DTYPE_F32])
def test_static_scratch_step_is_captured_into_a_graph_and_replayed(state, dtype):
    """What the entry point exists for: a caller under HIP graph capture, where an allocation, a
    free or a synchronisation fails the capture. One call is captured (after an eager call, so
    that per-kernel set-up is done), the graph replayed three times with a new query each time
    and eager work in between; every replay's context equals the plain attention call of a twin
    layer over the same rows. (A replay re-runs the captured launch: the same row is written
    to the same slot again and the same length is attended.)"""
    dims = (16, 2, 256)
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    layers, cache, lay, rng = _pair(state, dims, 5000, 0, dtype, 26)
    _steps(layers, cache, lay, rng, dims, 1)                 # eager first: kernels loaded, attributes set
    static, plain = layers
    kd = _dev(rng.standard_normal(kv_dim, dtype=np.float32))
    vd = _dev(rng.standard_normal(kv_dim, dtype=np.float32))
    qd = _dev(rng.standard_normal(q_dim, dtype=np.float32))
    out_s = torch.zeros(q_dim, device="cuda", dtype=torch.float32)
    out_p = torch.zeros(q_dim, device="cuda", dtype=torch.float32)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static.encode_decode_step_static(torch.cuda.current_stream().cuda_stream, kd.data_ptr(), 0, vd.data_ptr(), 0,
                                         qd.data_ptr(), out_s.data_ptr())
    assert static.len() == plain.len() + 1                  # the bookkeeping advanced at capture time
    plain.encode_append_kv(_stream(), kd.data_ptr(), vd.data_ptr())
    for r in range(3):
        qd.copy_(_dev(rng.standard_normal(q_dim, dtype=np.float32)))
        out_s.zero_()
        torch.cuda.synchronize()
        graph.replay()
        plain.encode_attention_decode_windowed(_stream(), qd.data_ptr(), out_p.data_ptr(), 0)
        torch.cuda.synchronize()
        assert np.array_equal(out_s.cpu().numpy(), out_p.cpu().numpy()), r
        # the program's own eager work between the replays
        scratch = torch.randn(1 << 20, device="cuda")
        assert float(scratch.abs().sum()) > 0
    sk, sv = static.read_rows_f32(static.len() - 8, 8)
    pk, pv = plain.read_rows_f32(plain.len() - 8, 8)
    assert np.array_equal(sk, pk) and np.array_equal(sv, pv)
