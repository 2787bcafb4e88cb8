"""Speculative decoding at the KV boundary: k draft rows are verified in one multi-query
launch over the cache (the per-row loop of the resident verify, src/decoder/resident/
verify.rs:157-203, as one call), then the cache is rolled back to the accepted length with
truncate (restore_mtp_resident_progress, src/decoder/generation.rs:1026-1064). After the
rollback the layer must behave as if the rejected rows had never been appended."""
import numpy as np
import pytest

import oracle
import saragossa_amd as skv

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.mark.parametrize("dims,window,base,rounds", [
    ((16, 2, 256), 0, 700, 6),      # full layer, split-K
    ((32, 8, 128), 0, 40, 8),       # short cache
    ((8, 2, 64), 20, 100, 10),      # ring layer, window not a multiple of the page
    ((8, 2, 64), 64, 200, 10),      # ring layer, window a multiple of 16: the ring's own slack rows
    ((16, 8, 256), 1024, 1500, 4),  # the local layers of a sliding-window model (window 1024)
])
def test_verify_rows_then_rollback_equals_never_appended(state, dims, window, base, rounds):
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(base + rounds)
    k_draft = 5
    cap = base + rounds * k_draft + 8
    kv = state.full_attention_bf16(cap, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    k0 = rng.standard_normal((base, kv_dim), dtype=np.float32)
    v0 = rng.standard_normal((base, kv_dim), dtype=np.float32)
    kv.seed(k0, v0, base)
    cache.append_batch(k0, v0, lay)
    for r in range(rounds):
        q = rng.standard_normal((k_draft, q_dim), dtype=np.float32)
        k = rng.standard_normal((k_draft, kv_dim), dtype=np.float32)
        v = rng.standard_normal((k_draft, kv_dim), dtype=np.float32)
        start = kv.len()
        got = kv.prefill_rows(q, k, v)                       # verify the k draft rows at once
        accepted = int(rng.integers(1, k_draft + 1))         # at least the first row is kept
        # the oracle only ever sees the accepted rows, one by one
        want = oracle.cached_attention_prefill_rows(q[:accepted], k[:accepted], v[:accepted], cache, lay)
        assert np.abs(got[:accepted] - want).max() <= 1e-4
        kv.truncate(start + accepted)                        # rollback
        assert kv.len() == len(cache) == start + accepted
    # after all the rollbacks: contents and a decode step agree with the oracle
    first = 0 if window == 0 else max(0, kv.len() - window)
    gk, gv = kv.read_rows_f32(first, kv.len() - first)
    assert np.array_equal(gk, cache.keys()[first:]) and np.array_equal(gv, cache.values()[first:])
    q = rng.standard_normal(q_dim, dtype=np.float32)
    ws = skv.flags.window_start(kv.len() - 1, window)
    assert np.abs(kv.attention_decode_windowed(q, ws) - oracle.cached_attention_one(q, cache, lay)).max() <= 1e-4


def test_rollback_deeper_than_the_rings_slack_is_an_error_not_stale_data(state):
    """A ring keeps its window plus 32 rows: a rollback of more rows than that needs rows the
    ring has overwritten, and the next attention reports it instead of reading them."""
    q_heads, kv_heads, head_dim, window = 8, 2, 64, 32
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(4)
    kv = state.full_attention_bf16(200, q_heads, kv_heads, head_dim, window=window)
    k = rng.standard_normal((100, kv_dim), dtype=np.float32)
    kv.seed(k, k, 100)
    q = rng.standard_normal((40, q_heads * head_dim), dtype=np.float32)
    kv.prefill_rows(q, k[:40], k[:40])
    kv.truncate(101)
    with pytest.raises(skv.DimensionError):
        kv.attention_decode_windowed(q[0], skv.flags.window_start(100, window))


@pytest.mark.parametrize("element", ["bf16", "f32"])
@pytest.mark.parametrize("slack", [0, 16, 64])
def test_ring_rollback_depth_is_a_create_argument(state, element, slack):
    """skv_layer_create_ring: a ring layer of window 1024 created with a rollback depth of 0, 16
    or 64 rows. A verify of up to that many rows can be rolled back completely (the reference
    truncates freely, src/decoder/attention_cache.rs:72-100; src/decoder/generation.rs:924-1026)
    and the layer then behaves as if the rows had never been appended; one row more than the
    depth is reported by the next attention call, never served stale."""
    q_heads, kv_heads, head_dim, window = 16, 8, 64, 1024
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(1000 + slack)
    dtype = skv.DTYPE_BF16 if element == "bf16" else skv.DTYPE_F32
    base = 2 * window + 37                              # the ring has wrapped
    kv = state.full_attention_with_element(base + 400, q_heads, kv_heads, head_dim, dtype, window, rollback_rows=slack)
    assert kv.pages() == (window + slack + 15) // 16
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    assert skv.flags.layer_bytes(base + 400, q_heads, kv_heads, head_dim, dtype, window, rollback_rows=slack) \
        < skv.flags.layer_bytes(base + 400, q_heads, kv_heads, head_dim, dtype, window, rollback_rows=slack + 4096)
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r" if element == "bf16" else "f32")
    k0 = rng.standard_normal((base, kv_dim), dtype=np.float32)
    v0 = rng.standard_normal((base, kv_dim), dtype=np.float32)
    kv.seed(k0, v0, base)
    cache.append_batch(k0, v0, lay)
    tol = 1e-4 if element == "bf16" else 2e-5
    for depth in sorted({1, max(slack, 1)} if slack else {1}):
        if depth > slack:
            break
        q = rng.standard_normal((depth, q_dim), dtype=np.float32)
        k = rng.standard_normal((depth, kv_dim), dtype=np.float32)
        v = rng.standard_normal((depth, kv_dim), dtype=np.float32)
        start = kv.len()
        kv.prefill_rows(q, k, v)                        # the draft rows
        kv.truncate(start)                              # all of them rejected
        qd = rng.standard_normal(q_dim, dtype=np.float32)
        kd = rng.standard_normal(kv_dim, dtype=np.float32)
        vd = rng.standard_normal(kv_dim, dtype=np.float32)
        kv.append_row(kd, vd)
        got = kv.attention_decode_windowed(qd, skv.flags.window_start(kv.len() - 1, window))
        want = oracle.decode_step(cache, kd, vd, qd, lay)
        assert np.abs(got - want).max() <= tol
    first = kv.len() - window
    gk, gv = kv.read_rows_f32(first, window)
    assert np.array_equal(gk, cache.keys()[first:]) and np.array_equal(gv, cache.values()[first:])
    # one row deeper than the ring kept (the ring holds whole pages, so "kept" is its row count)
    kept = kv.pages() * 16 - window
    n_over = kept + 1
    q = rng.standard_normal((n_over, q_dim), dtype=np.float32)
    k = rng.standard_normal((n_over, kv_dim), dtype=np.float32)
    start = kv.len()
    kv.prefill_rows(q, k, k)
    kv.truncate(start)
    with pytest.raises(skv.DimensionError):
        kv.attention_decode_windowed(q[0], skv.flags.window_start(start - 1, window))
    kv.close()
