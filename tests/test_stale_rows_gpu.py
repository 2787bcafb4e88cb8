"""Rows the cache does not count (at or past `len` after a rollback, ring rows no longer in
any window, rows before a layer's window) may hold any bits, NaN and Inf included: the
reference rounds f32 to bf16 without a NaN special case (src/decode_resident/utils.rs:55-60)
and never reads past `len` (src/decode_resident/kernels.rs:11-88). A context computed after
such rows were rolled back must equal, bit for bit, the context of a cache that never held
them."""
import numpy as np
import pytest

import oracle
import saragossa_amd as skv

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _poison(rng, n, kv_dim):
    """Rows of NaN, +Inf, -Inf and values that round to Inf in bf16."""
    rows = rng.standard_normal((n, kv_dim), dtype=np.float32)
    rows[0::4] = np.nan
    rows[1::4] = np.inf
    rows[2::4] = -np.inf
    rows[3::4] = np.float32(3.4e38)   # finite in f32, Inf once rounded to bf16
    return rows


def _stream():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("dtype", [skv.DTYPE_BF16, skv.DTYPE_F32])
@pytest.mark.parametrize("dims,base,window", [
    ((16, 2, 256), 700, 0),     # split-K, the poisoned rows share a page with live rows
    ((32, 8, 128), 37, 0),      # one split, page boundary inside the poisoned range
    ((8, 2, 64), 100, 48),      # ring layer
    ((16, 8, 512), 300, 0),     # wide heads (four-wavefront kernel)
])
def test_rolled_back_nan_and_inf_rows_leave_no_trace(state, dtype, dims, base, window):
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(base + head_dim)
    keys = rng.standard_normal((base, kv_dim), dtype=np.float32)
    values = rng.standard_normal((base, kv_dim), dtype=np.float32)
    table = None
    pair = []
    for _ in range(2):
        kv = state.full_attention_with_element(base + 64, q_heads, kv_heads, head_dim, dtype, window)
        if table is None:
            table = rng.permutation(kv.pages()).astype(np.int32)
        kv.set_block_table(table)
        kv.seed(keys, values, base)
        pair.append(kv)
    dirty, clean = pair
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r" if dtype == skv.DTYPE_BF16 else "f32")
    cache.append_batch(keys, values, lay)
    # a speculative verify of 7 poisoned rows (one multi-query launch), all rejected
    bad = _poison(rng, 7, kv_dim)
    q7 = rng.standard_normal((7, q_dim), dtype=np.float32)
    dirty.prefill_rows(q7, bad, bad)
    dirty.truncate(base)
    # decode steps and a chunk afterwards: the poisoned rows are overwritten one at a time, the
    # rest of them stay in the pages next to live rows
    for step in range(3):
        k = rng.standard_normal(kv_dim, dtype=np.float32)
        v = rng.standard_normal(kv_dim, dtype=np.float32)
        q = rng.standard_normal(q_dim, dtype=np.float32)
        for kv in pair:
            kv.append_row(k, v)
        cache.append(k, v, lay)
        ws = skv.flags.window_start(clean.len() - 1, window)
        got_d = dirty.attention_decode_windowed(q, ws)
        got_c = clean.attention_decode_windowed(q, ws)
        assert np.isfinite(got_d).all()
        assert np.array_equal(got_d, got_c)
        assert np.abs(got_d - oracle.cached_attention_one(q, cache, lay)).max() <= 1e-4
    # the fused decode step (append inside the attention launch) over the same pages
    k = torch.randn(kv_dim, device="cuda")
    v = torch.randn(kv_dim, device="cuda")
    q = torch.randn(q_dim, device="cuda")
    outs = []
    for kv in pair:
        out = torch.empty(q_dim, device="cuda", dtype=torch.float32)
        kv.encode_decode_step(_stream(), k.data_ptr(), 0, v.data_ptr(), 0, q.data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    assert np.isfinite(outs[0]).all() and np.array_equal(outs[0], outs[1])
    # a chunk of 2 rows (multi-query mode) and one of 70 (tile kernel where it applies)
    for n in (2, 70 if window == 0 else 20):
        if clean.len() + n > clean.capacity():
            break
        qn = rng.standard_normal((n, q_dim), dtype=np.float32)
        kn = rng.standard_normal((n, kv_dim), dtype=np.float32)
        vn = rng.standard_normal((n, kv_dim), dtype=np.float32)
        got_d = dirty.prefill_rows(qn, kn, vn)
        got_c = clean.prefill_rows(qn, kn, vn)
        assert np.isfinite(got_d).all()
        assert np.array_equal(got_d, got_c)


def test_rows_before_the_window_may_hold_anything(state):
    """attention_decode_windowed never reads rows before window_start
    (src/decode_resident/attention.rs:738-756): poison there changes nothing."""
    q_heads, kv_heads, head_dim, n = 16, 2, 256, 500
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(77)
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    bad_k, bad_v = keys.copy(), values.copy()
    bad_k[:203] = _poison(rng, 203, kv_dim)
    bad_v[:203] = _poison(rng, 203, kv_dim)
    q = rng.standard_normal(q_dim, dtype=np.float32)
    outs = []
    for k, v in ((bad_k, bad_v), (keys, values)):
        kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
        kv.seed(k, v, n)
        outs.append(kv.attention_decode_windowed(q, 203))   # 203: inside a page
    assert np.isfinite(outs[0]).all() and np.array_equal(outs[0], outs[1])
