"""Seeded random lifetimes of one cache, in both element types (bf16 against the oracle's
rounding cache, f32 against its plain one): seed, single appends, chunks, decode steps, verify
chunks with rollback and block snapshots in random order, on full and ring layers of random
geometry behind a permuted block table. After every operation the device cache and the CPU
oracle (LayerKvCache + cached_attention_one, src/decoder/attention_cache.rs:7-100,
src/decoder/attention_ops.rs:976-1046) hold the same rows bit for bit and give the same
attention within 1e-3 (bound to hold: 1e-2). Rows are drawn at up to three standard deviations'
scale, so scores reach several tens, where the device's two-term bf16 products differ from the
CPU's f32 ones by a few 1e-4; at unit scale the difference stays under 1e-4
(tests/test_attention_gpu.py)."""
import numpy as np
import pytest

import oracle
import saragossa_amd as skv

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

TOL = 1e-3

GEOMETRIES = [(16, 2, 256), (32, 8, 128), (8, 2, 64), (6, 1, 40), (4, 2, 16), (8, 1, 32), (4, 1, 320),
              (12, 4, 96)]


def _held_first(n, window):
    return 0 if window == 0 else max(0, n - window)


def _check_contents(kv, cache, window):
    first = _held_first(kv.len(), window)
    if kv.len() == first:
        return
    gk, gv = kv.read_rows_f32(first, kv.len() - first)
    assert np.array_equal(gk, cache.keys()[first:]) and np.array_equal(gv, cache.values()[first:])


@pytest.mark.parametrize("element", ["bf16", "f32"])
@pytest.mark.parametrize("seed", range(32))
def test_random_lifetime_matches_the_oracle(state, seed, element):
    rng = np.random.default_rng(1000 + seed)
    q_heads, kv_heads, head_dim = GEOMETRIES[seed % len(GEOMETRIES)]
    make = state.full_attention_f32 if element == "f32" else state.full_attention_bf16
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    window = 0 if seed % 3 else int(rng.integers(17, 90))
    cap = int(rng.integers(700, 1500))
    kv = make(cap, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("f32" if element == "f32" else "bf16r")
    # rows a ring keeps beyond its window: a rollback may not reach below them
    ring_rows = 0 if window == 0 else (window + 15) // 16 * 16
    log = []

    def rows(n, dim):
        return rng.standard_normal((n, dim), dtype=np.float32) * float(rng.choice([0.3, 1.0, 3.0]))

    for step in range(60):
        n = kv.len()
        room = cap - n
        op = rng.choice(["append", "chunk", "decode", "verify", "attend", "snapshot"])
        log.append((step, str(op), n))
        if op == "append" and room >= 1:
            k, v = rows(1, kv_dim), rows(1, kv_dim)
            kv.append_row(k[0], v[0])
            cache.append(k, v, lay)
        elif op == "chunk" and room >= 2:
            m = int(min(room - 1, rng.choice([2, 7, 16, 33, 70, 150])))
            if m < 1:
                continue
            q, k, v = rows(m, q_dim), rows(m, kv_dim), rows(m, kv_dim)
            want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
            got = kv.prefill_rows(q, k, v)
            assert np.abs(got - want).max() <= TOL, (seed, log[-3:])
        elif op == "decode" and room >= 1:
            k, v, q = rows(1, kv_dim)[0], rows(1, kv_dim)[0], rows(1, q_dim)[0]
            dk, dv, dq = (torch.from_numpy(a).cuda() for a in (k, v, q))
            out = torch.empty(q_dim, dtype=torch.float32, device="cuda")
            kv.encode_decode_step(torch.cuda.current_stream().cuda_stream, dk.data_ptr(), 0,
                                  dv.data_ptr(), 0, dq.data_ptr(), out.data_ptr())
            want = oracle.decode_step(cache, k, v, q, lay)
            assert np.abs(out.cpu().numpy() - want).max() <= TOL, (seed, log[-3:])
        elif op == "verify" and room >= 6 and n >= 1:
            m = 5
            q, k, v = rows(m, q_dim), rows(m, kv_dim), rows(m, kv_dim)
            got = kv.prefill_rows(q, k, v)
            # a ring has overwritten rows (n + m - ring_rows) and older: keep at least those
            least = 1 if window == 0 else max(1, m - (ring_rows - window))
            accepted = int(rng.integers(least, m + 1))
            want = oracle.cached_attention_prefill_rows(q[:accepted], k[:accepted], v[:accepted], cache, lay)
            assert np.abs(got[:accepted] - want).max() <= TOL, (seed, log[-3:])
            kv.truncate(n + accepted)
        elif op == "attend" and n >= 1:
            q = rows(1, q_dim)[0]
            ws = skv.flags.window_start(n - 1, window)
            got = kv.attention_decode_windowed(q, ws)
            assert np.abs(got - oracle.cached_attention_one(q, cache, lay)).max() <= TOL, (seed, log[-3:])
        elif op == "snapshot" and window == 0 and n >= 32:
            # two full pages copied out and into the same logical pages of a second layer
            # that holds other rows: there they read as the oracle's rows
            pages = sorted(int(p) for p in rng.choice(n // 16, size=2, replace=False))
            snap = skv.snapshot_blocks(state, [kv], pages)
            other = make(cap, q_heads, kv_heads, head_dim)
            other.seed(rows(n, kv_dim), rows(n, kv_dim), n)
            skv.restore_blocks(state, snap, [other], pages)
            gk, gv = other.read_rows_f32()
            for p in pages:
                assert np.array_equal(gk[p * 16:(p + 1) * 16], cache.keys()[p * 16:(p + 1) * 16])
                assert np.array_equal(gv[p * 16:(p + 1) * 16], cache.values()[p * 16:(p + 1) * 16])
            snap.close()
            other.close()
        else:
            continue
        assert kv.len() == len(cache), (seed, log[-3:])
        _check_contents(kv, cache, window)
    kv.close()
