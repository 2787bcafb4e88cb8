"""Cache-content parity on the GPU, restating the reference's KV tests
(src/decode_resident/tests.rs:380-538, 1930-2018) against the paged bf16 cache.
Contents are compared bit for bit with the oracle's bf16 rounding."""
import numpy as np
import pytest

import oracle
import saragossa_amd as skv
from conftest import bf16_bits_to_f32

pytestmark = pytest.mark.gpu


def test_kv_bf16_seed_then_append_rounds_to_bf16(state):
    # src/decode_resident/tests.rs:435-478
    q_heads, kv_heads, head_dim = 16, 2, 256
    kv_dim = kv_heads * head_dim
    capacity = 4
    kv = state.full_attention_bf16(capacity, q_heads, kv_heads, head_dim)
    assert kv.kv_dim() == kv_dim
    assert kv.byte_len() == capacity * kv_dim * 2
    seed_rows = 2
    i = np.arange(seed_rows * kv_dim, dtype=np.float32)
    seed_k = ((i - np.float32(333.0)) * np.float32(0.0017)).astype(np.float32)
    seed_v = ((i + np.float32(17.0)) * np.float32(-0.0023)).astype(np.float32)
    kv.seed(seed_k, seed_v, seed_rows)
    c = np.arange(kv_dim, dtype=np.float32)
    row_k = (np.float32(1.0) + c * np.float32(0.0009)).astype(np.float32)
    row_v = (np.float32(-1.0) + c * np.float32(0.0011)).astype(np.float32)
    kv.append_row(row_k, row_v)
    assert kv.len() == seed_rows + 1
    cpu_k = np.concatenate([seed_k, row_k])
    cpu_v = np.concatenate([seed_v, row_v])
    gk, gv = kv.read_rows()
    assert np.array_equal(gk.reshape(-1), oracle.f32_to_bf16_bits(cpu_k))
    assert np.array_equal(gv.reshape(-1), oracle.f32_to_bf16_bits(cpu_v))
    assert np.array_equal(bf16_bits_to_f32(gk).reshape(-1), oracle.bf16_round(cpu_k))


def test_kv_seed_then_append_matches_cpu(state):
    # src/decode_resident/tests.rs:380-430, against the oracle cache in bf16-rounded mode
    q_heads, kv_heads, head_dim = 16, 2, 256
    kv_dim = kv_heads * head_dim
    lay = oracle.layout(q_heads, kv_heads, head_dim)
    kv = state.full_attention_bf16(6, q_heads, kv_heads, head_dim)
    cpu = oracle.LayerKvCache("bf16r")
    seed_rows = 3
    idx = np.arange(seed_rows * kv_dim, dtype=np.float32)
    seed_k = (idx * np.float32(0.001)).astype(np.float32)
    seed_v = (idx * np.float32(-0.002) + np.float32(1.0)).astype(np.float32)
    kv.seed(seed_k, seed_v, seed_rows)
    cpu.append_batch(seed_k.reshape(seed_rows, kv_dim), seed_v.reshape(seed_rows, kv_dim), lay)
    assert kv.len() == seed_rows
    for r in range(seed_rows, seed_rows + 2):
        c = (r * kv_dim + np.arange(kv_dim)).astype(np.float32)
        k = (c * np.float32(0.003)).astype(np.float32)
        v = (c * np.float32(0.004) - np.float32(0.5)).astype(np.float32)
        kv.append_row(k, v)
        cpu.append(k.reshape(1, -1), v.reshape(1, -1), lay)
    assert kv.len() == seed_rows + 2 == len(cpu)
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk, cpu.keys())
    assert np.array_equal(gv, cpu.values())


def test_kv_append_writes_at_nonzero_offset(state):
    # src/decode_resident/tests.rs:482-503 (toy dims, kv_dim = 4)
    kv = state.full_attention_bf16(4, 4, 2, 2)
    kv.append_row([1.0, 2.0, 3.0, 4.0], [5.0, 6.0, 7.0, 8.0])
    kv.append_row([10.0, 20.0, 30.0, 40.0], [50.0, 60.0, 70.0, 80.0])
    gk, gv = kv.read_rows_f32()
    assert gk.tolist() == [[1.0, 2.0, 3.0, 4.0], [10.0, 20.0, 30.0, 40.0]]
    assert gv.tolist() == [[5.0, 6.0, 7.0, 8.0], [50.0, 60.0, 70.0, 80.0]]


def test_kv_overflow_at_capacity_errors(state):
    # src/decode_resident/tests.rs:507-525
    q_heads, kv_heads, head_dim = 4, 2, 2
    kv_dim = kv_heads * head_dim
    prefill_len = 3
    kv = state.full_attention_bf16(prefill_len, q_heads, kv_heads, head_dim)
    seed = np.arange(prefill_len * kv_dim, dtype=np.float32)
    kv.seed(seed, seed, prefill_len)
    assert kv.len() == kv.capacity()
    row = np.zeros(kv_dim, dtype=np.float32)
    with pytest.raises(skv.DimensionError):
        kv.append_row(row, row)
    assert kv.len() == prefill_len


def test_full_attention_state_rejects_non_multiple_gqa(state):
    # src/decode_resident/tests.rs:528-538
    with pytest.raises(skv.ConfigError):
        state.full_attention_bf16(4, 3, 2, 8)


def test_full_attention_state_rejects_zero_dims(state):
    # src/decode_resident/attention.rs:64-68
    for dims in [(0, 4, 2, 8), (4, 0, 2, 8), (4, 4, 0, 8), (4, 4, 2, 0)]:
        with pytest.raises(skv.ConfigError):
            state.full_attention_bf16(*dims)


def test_seed_and_append_shape_errors(state):
    # src/decode_resident/attention.rs:556-573, 613-619
    kv = state.full_attention_bf16(4, 4, 2, 8)
    kv_dim = 16
    with pytest.raises(skv.DimensionError):
        kv.seed(np.zeros(5 * kv_dim), np.zeros(5 * kv_dim), 5)  # n_rows > capacity
    with pytest.raises(skv.DimensionError):
        kv.seed(np.zeros(2 * kv_dim), np.zeros(2 * kv_dim - 1), 2)
    with pytest.raises(skv.DimensionError):
        kv.append_row(np.zeros(kv_dim - 1), np.zeros(kv_dim))
    with pytest.raises(skv.DimensionError):
        kv.truncate(5)
    kv.truncate(0)


@pytest.mark.parametrize("dims", [(32, 8, 128), (16, 2, 256), (4, 2, 16), (8, 8, 64), (6, 2, 96),
                                  (2, 1, 40)])
def test_paged_contents_with_permuted_block_table(state, dims):
    """Logical row r lives at (block_table[r/16], r%16): seeding through a random permutation
    and appending must read back bit-exact, and rows must land in the permuted pages."""
    q_heads, kv_heads, head_dim = dims
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(7)
    capacity = 16 * 9 + 5
    kv = state.full_attention_bf16(capacity, q_heads, kv_heads, head_dim)
    table = rng.permutation(kv.pages()).astype(np.int32)
    kv.set_block_table(table)
    n = 16 * 7 + 3
    k = rng.standard_normal((n, kv_dim), dtype=np.float32)
    v = rng.standard_normal((n, kv_dim), dtype=np.float32)
    kv.seed(k, v, n)
    for _ in range(20):
        kr = rng.standard_normal(kv_dim, dtype=np.float32)
        vr = rng.standard_normal(kv_dim, dtype=np.float32)
        kv.append_row(kr, vr)
        k = np.vstack([k, kr[None]])
        v = np.vstack([v, vr[None]])
    gk, gv = kv.read_rows()
    assert np.array_equal(gk, oracle.f32_to_bf16_bits(k))
    assert np.array_equal(gv, oracle.f32_to_bf16_bits(v))
    # partial reads through the table
    gk2, gv2 = kv.read_rows(17, 40)
    assert np.array_equal(gk2, gk[17:57]) and np.array_equal(gv2, gv[17:57])
    # truncate drops rows without touching the kept ones
    kv.truncate(33)
    gk3, _ = kv.read_rows()
    assert np.array_equal(gk3, gk[:33])
    with pytest.raises(skv.DimensionError):
        kv.read_rows(0, 34)


def test_bf16_rounding_special_values(state):
    """The device conversion is the reference's integer formula, including ties to even,
    the carry into the exponent, infinities and the NaN non-special-case."""
    vals = np.array([1.00390625, -0.33325195, 42.125, 0.0, -0.0, 1.0, 3.3895314e38, np.inf,
                     -np.inf, 1.0039062, 1.0117188, 1e-40, -1e-45, 65504.0, 1.9960938,
                     1.9980469, 0.1, -0.1], dtype=np.float32)
    bits = np.array([0x7FC00000, 0x7F800001, 0xFFFFFFFF, 0x7FFF7FFF, 0x00008000, 0x00018000,
                     0x00017FFF], dtype=np.uint32).view(np.float32)
    vals = np.concatenate([vals, bits])
    kv_dim = 32
    pad = np.zeros(kv_dim - vals.size % kv_dim if vals.size % kv_dim else 0, dtype=np.float32)
    data = np.concatenate([vals, pad]).reshape(-1, kv_dim)
    kv = state.full_attention_bf16(data.shape[0], 1, 1, kv_dim)
    kv.seed(data, data, data.shape[0])
    gk, gv = kv.read_rows()
    want = oracle.f32_to_bf16_bits(data)
    assert np.array_equal(gk, want)
    assert np.array_equal(gv, want)


def test_buffers_of_a_destroyed_layer_are_reused_clean(state):
    """The context keeps the device buffers of destroyed layers for the next layer of about
    the same size (the arena of DecodeResidentState, src/decode_resident/arena.rs:116-211). A
    layer that inherits them must not see what the previous owner left: its padded dims and
    unwritten rows are zero again (head_dim 96 is padded to 128, so stale values there would
    enter every score)."""
    import oracle
    rng = np.random.default_rng(123)
    first = state.full_attention_bf16(512, 8, 2, 128)
    first.seed(rng.standard_normal((512, 256), dtype=np.float32) * 50,
               rng.standard_normal((512, 256), dtype=np.float32) * 50, 512)
    first.close()
    # same pool bytes (512 rows x 2 heads x 128 padded dims), other logical shape
    kv = state.full_attention_bf16(512, 6, 2, 96)
    n, kv_dim = 300, 2 * 96
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    kv.seed(keys, values, n)
    q = rng.standard_normal(6 * 96, dtype=np.float32)
    lay = oracle.layout(6, 2, 96)
    cache = oracle.LayerKvCache("bf16r")
    cache.append_batch(keys, values, lay)
    want = oracle.cached_attention_one(q, cache, lay)
    assert np.abs(kv.attention_decode(q) - want).max() <= 1e-4
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk, cache.keys()) and np.array_equal(gv, cache.values())
    kv.close()


def test_a_context_gives_all_device_memory_back():
    """Handles own their device memory exactly once (src/decoder.rs:434-446): after a context
    of its own has created and dropped layers, snapshots, a rotation table and a hot cache,
    and has itself been destroyed (which empties its arena), the device has as much free
    memory as before. (A first context goes through the same motions beforehand, so that what
    the runtime keeps for itself after first use is not counted.)"""
    torch = pytest.importorskip("torch")

    def lifetime(rounds):
        st = skv.DecodeResidentState(0)
        rng = np.random.default_rng(9)
        for _ in range(rounds):
            layers = [st.full_attention_bf16(4096, 32, 8, 128, window=(1024 if i == 1 else 0)) for i in range(4)]
            for kv in layers:
                kv.seed(rng.standard_normal((600, 1024), dtype=np.float32),
                        rng.standard_normal((600, 1024), dtype=np.float32), 600)
            q = rng.standard_normal(32 * 128, dtype=np.float32)
            layers[0].attention_decode(q)
            layers[0].prefill_rows(rng.standard_normal((40, 4096), dtype=np.float32),
                                   rng.standard_normal((40, 1024), dtype=np.float32),
                                   rng.standard_normal((40, 1024), dtype=np.float32))
            snap = skv.snapshot_blocks(st, [layers[0], layers[2]], [0, 5, 7])
            copy = snap.clone()
            rope = st.rope_table(4096, 128, 1.0e6)
            hot = skv.HotCache(st, 16, 64, 32, layers)
            root = skv.BlockHash.root()
            h = skv.BlockHash.chain(root, list(range(16)))
            assert hot.remember_prefix_block(root, h, 16, layers)
            hot.close()
            rope.close()
            copy.close()
            snap.close()
            for kv in layers:
                kv.close()
        st.close()
        torch.cuda.synchronize()

    lifetime(1)
    torch.cuda.empty_cache()
    free0, _ = torch.cuda.mem_get_info()
    lifetime(3)
    free1, _ = torch.cuda.mem_get_info()
    assert free0 - free1 <= 16 << 20, (free0, free1)


def test_objects_may_outlive_their_context():
    """Finalisers of a garbage-collected binding run in any order: a layer, a rope table, a
    snapshot and a hot cache stay usable after skv_ctx_destroy and are destroyed afterwards,
    and all device memory still comes back."""
    torch = pytest.importorskip("torch")

    def lifetime():
        st = skv.DecodeResidentState(0)
        rng = np.random.default_rng(10)
        layers = [st.full_attention_bf16(2048, 32, 8, 128) for _ in range(3)]
        keys = rng.standard_normal((300, 1024), dtype=np.float32)
        values = rng.standard_normal((300, 1024), dtype=np.float32)
        for kv in layers:
            kv.seed(keys, values, 300)
        snap = skv.snapshot_blocks(st, layers[:2], [0, 3])
        rope = st.rope_table(1024, 128, 1.0e6)
        hot = skv.HotCache(st, 16, 32, 32, layers)
        q = rng.standard_normal(32 * 128, dtype=np.float32)
        want = layers[0].attention_decode(q)
        copy = snap.clone()
        layers[2].close()  # into the arena, which the next line empties
        st.close()
        assert np.array_equal(layers[0].attention_decode(q), want)
        layers[1].append_row(keys[0], values[0])
        assert layers[1].len() == 301
        for obj in (layers[0], hot, copy, rope, snap, layers[1]):
            obj.close()
        torch.cuda.synchronize()

    lifetime()
    torch.cuda.empty_cache()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        lifetime()
    free1, _ = torch.cuda.mem_get_info()
    assert free0 - free1 <= 16 << 20, (free0, free1)


@pytest.mark.parametrize("dtype,window", [(skv.DTYPE_BF16, 0), (skv.DTYPE_F32, 0), (skv.DTYPE_BF16, 1024)])
def test_layer_bytes_is_what_a_created_layer_takes(dtype, window):
    """skv_layer_bytes (the figure a host budgets with, as setup.rs:897-962 budgets the resident
    KV) against the device memory a freshly created layer really takes: a context of its own,
    so nothing comes out of an arena, and hipMemGetInfo before and after."""
    torch = pytest.importorskip("torch")
    from saragossa_amd import flags
    st = skv.DecodeResidentState(0)
    try:
        shape = (65536, 16, 8, 256)
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        kv = st.full_attention_with_element(*shape, dtype, window)
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        want = flags.layer_bytes(*shape, dtype, window)
        took = free0 - free1
        # the allocator rounds large buffers up to its granule (2 MiB) and carves small ones out of
        # chunks it already holds, so each of the layer's nine buffers may be off by one granule
        assert abs(took - want) <= 9 * (2 << 20), (want, took)
        if want >= 256 << 20:   # where the granules are small against the layer
            assert 0.98 * took <= want <= 1.02 * took, (want, took)
        kv.close()
    finally:
        st.close()
