"""Random batches through skv_decode_step_batch_device: 2 to 6 independent sequences of random
lengths (empty ones included) on a random geometry, element and window, a random number of steps;
every context against the oracle's decode_step, the rows left behind bit for bit. Covers the
shapes that take one launch pair and those that fall back to a launch pair per sequence (more
than 16 heads per group, wide f32 heads)."""
import numpy as np
import pytest
import torch

import oracle
import saragossa_amd as skv

pytestmark = pytest.mark.gpu

GEOMETRIES = [(16, 2, 256), (32, 8, 128), (8, 2, 64), (6, 1, 40), (4, 2, 16), (8, 1, 32), (4, 1, 320), (12, 4, 96),
              (16, 1, 64), (8, 2, 512), (16, 8, 256), (20, 1, 128)]


@pytest.mark.parametrize("case", range(24))
def test_random_batch_matches_the_oracle(state, case):
    rng = np.random.default_rng(1000 + case)
    q_heads, kv_heads, head_dim = GEOMETRIES[int(rng.integers(len(GEOMETRIES)))]
    element = "f32" if case % 2 else "bf16"
    window = 0 if rng.random() < 0.6 else int(rng.integers(17, 300))
    n_seq = int(rng.integers(2, 7))
    steps = int(rng.integers(1, 25))
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    make = state.full_attention_f32 if element == "f32" else state.full_attention_bf16
    seqs = []
    for _ in range(n_seq):
        n = int(rng.integers(0, 5000)) if rng.random() < 0.8 else int(rng.integers(0, 40))
        kv = make(n + steps + 4, q_heads, kv_heads, head_dim, window=window)
        kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
        lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
        cache = oracle.LayerKvCache("f32" if element == "f32" else "bf16r")
        if n:
            k0 = rng.standard_normal((n, kv_dim), dtype=np.float32)
            v0 = rng.standard_normal((n, kv_dim), dtype=np.float32)
            kv.seed(k0, v0, n)
            cache.append_batch(k0, v0, lay)
        seqs.append((kv, cache, lay))
    stream = torch.cuda.current_stream().cuda_stream
    tol = 2e-5 if element == "f32" else 1e-4
    for _ in range(steps):
        rows = [(rng.standard_normal(kv_dim, dtype=np.float32), rng.standard_normal(kv_dim, dtype=np.float32),
                 rng.standard_normal(q_dim, dtype=np.float32)) for _ in seqs]
        dev = [[torch.from_numpy(a).cuda() for a in r] for r in rows]
        outs = [torch.empty(q_dim, device="cuda") for _ in seqs]
        skv.encode_decode_step_batch([s[0] for s in seqs], stream, [d[0].data_ptr() for d in dev],
                                     [d[1].data_ptr() for d in dev], [d[2].data_ptr() for d in dev],
                                     [o.data_ptr() for o in outs])
        for (kv, cache, lay), (k, v, q), o in zip(seqs, rows, outs):
            want = oracle.decode_step(cache, k, v, q, lay)
            assert np.abs(o.cpu().numpy() - want).max() <= tol
    for kv, cache, lay in seqs:
        m = kv.len()
        keep = min(m, window) if window else m
        gk, gv = kv.read_rows_f32(m - keep, keep)
        assert np.array_equal(gk, cache.keys()[m - keep:]) and np.array_equal(gv, cache.values()[m - keep:])
        kv.close()


def test_full_batch_of_sixteen_heads_per_group_at_head_dim_256(state):
    """16 sequences (the most one launch takes) of q32/kv2/hd256 at about 600 rows: 320
    four-wavefront workgroups, each with the largest exchange area the kernel has (16 query
    heads x 256 columns per wavefront), more workgroups than the device holds at once."""
    rng = np.random.default_rng(77)
    q_heads, kv_heads, head_dim = 32, 2, 256
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    seqs = []
    for i in range(16):
        n = 590 + i
        kv = state.full_attention_bf16(n + 8, q_heads, kv_heads, head_dim)
        kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
        lay = oracle.layout(q_heads, kv_heads, head_dim)
        cache = oracle.LayerKvCache("bf16r")
        k0 = rng.standard_normal((n, kv_dim), dtype=np.float32)
        v0 = rng.standard_normal((n, kv_dim), dtype=np.float32)
        kv.seed(k0, v0, n)
        cache.append_batch(k0, v0, lay)
        seqs.append((kv, cache, lay))
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        rows = [(rng.standard_normal(kv_dim, dtype=np.float32), rng.standard_normal(kv_dim, dtype=np.float32),
                 rng.standard_normal(q_dim, dtype=np.float32)) for _ in seqs]
        dev = [[torch.from_numpy(a).cuda() for a in r] for r in rows]
        outs = [torch.empty(q_dim, device="cuda") for _ in seqs]
        skv.encode_decode_step_batch([s[0] for s in seqs], stream, [d[0].data_ptr() for d in dev],
                                     [d[1].data_ptr() for d in dev], [d[2].data_ptr() for d in dev],
                                     [o.data_ptr() for o in outs])
        for (kv, cache, lay), (k, v, q), o in zip(seqs, rows, outs):
            want = oracle.decode_step(cache, k, v, q, lay)
            assert np.abs(o.cpu().numpy() - want).max() <= 1e-4
    for kv, _, _ in seqs:
        kv.close()
