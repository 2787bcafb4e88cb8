"""Chunked prefill at seeded random shapes: a cache of random geometry, element and window
behind a permuted block table is filled in chunks of random length, every chunk attended as
one call (cached_attention_prefill_rows, src/decoder/attention_ops.rs:976-1017: append, then
cached_attention_one, row by row). Every chunk's context agrees with the oracle within 1e-4
(bound to hold: 1e-2) and the rows held at the end are the oracle's bit for bit."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

GEOMETRIES = [(16, 2, 256), (32, 8, 128), (8, 2, 64), (6, 1, 40), (4, 2, 16), (8, 1, 32), (4, 1, 320),
              (12, 4, 96), (40, 1, 64), (8, 2, 512), (16, 8, 256)]


@pytest.mark.parametrize("case", range(24))
def test_random_chunks_match_the_oracle(state, case):
    rng = np.random.default_rng(7700 + case)
    q_heads, kv_heads, head_dim = GEOMETRIES[int(rng.integers(len(GEOMETRIES)))]
    element = "f32" if case % 2 else "bf16"
    start, chunk = int(rng.integers(0, 2500)), int(rng.integers(1, 300))
    window = 0 if rng.random() < 0.6 else int(rng.integers(17, 400))
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    make = state.full_attention_f32 if element == "f32" else state.full_attention_bf16
    kv = make(start + chunk + 3, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("f32" if element == "f32" else "bf16r")
    done = 0
    while done < start + chunk:
        c = min(int(rng.integers(1, 700)), start - done) if done < start else chunk
        q = rng.standard_normal((c, q_dim), dtype=np.float32)
        k = rng.standard_normal((c, kv_dim), dtype=np.float32)
        v = rng.standard_normal((c, kv_dim), dtype=np.float32)
        got = kv.prefill_rows(q, k, v)
        want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
        assert np.abs(got - want).max() <= 1e-4, (element, (q_heads, kv_heads, head_dim), window, done, c)
        done += c
    assert kv.len() == len(cache) == start + chunk
    first = 0 if window == 0 else max(0, kv.len() - window)
    gk, gv = kv.read_rows_f32(first, kv.len() - first)
    assert np.array_equal(gk, cache.keys()[first:]) and np.array_equal(gv, cache.values()[first:])
    kv.close()
