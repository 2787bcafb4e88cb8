"""Decode attention on the GPU against the CPU oracle, restating the reference's
differential tests (src/decode_resident/tests.rs:1228-1621). The oracle reads K/V
rounded to bf16, the reference's own convention for a bf16 device cache
(tests.rs:1443-1492); its bounds there are max-abs 2e-3 / mean-abs 2e-4. The bound
asserted here is tighter (1e-4 / 1e-5, the reference's f32 bound), far inside the
1e-2 this build is held to."""
import os

import numpy as np
import pytest

import oracle
import saragossa_amd as skv
from conftest import pseudo

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 1.0e-4, 1.0e-5


def cpu_attention(q, keys, values, q_heads, kv_heads, head_dim, window=0):
    """cached_attention_one over bf16-rounded K/V (oracle mode BF16R)."""
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    cache.append_batch(keys, values, lay)
    return oracle.cached_attention_one(q, cache, lay)


def run_attention_case(state, n, q_heads=16, kv_heads=2, head_dim=256, permute=True):
    kv_dim = kv_heads * head_dim
    kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
    if permute:
        kv.set_block_table(np.random.default_rng(n).permutation(kv.pages()).astype(np.int32))
    keys = pseudo(np.arange(n * kv_dim)).reshape(n, kv_dim)
    values = pseudo(np.arange(n * kv_dim) + 7).reshape(n, kv_dim)
    kv.seed(keys, values, n)
    q = pseudo(np.arange(q_heads * head_dim) + 99)
    gpu = kv.attention_decode(q)
    cpu = cpu_attention(q, keys, values, q_heads, kv_heads, head_dim)
    delta = np.abs(gpu - cpu)
    assert delta.max() <= MAX_ABS, f"len={n}: max_abs={delta.max():e}"
    assert delta.mean() <= MEAN_ABS, f"len={n}: mean_abs={delta.mean():e}"
    return gpu


@pytest.mark.parametrize("n", [1, 64, 257])
def test_attention_decode_matches_cpu_short(state, n):
    # src/decode_resident/tests.rs:1599-1621
    run_attention_case(state, n)


@pytest.mark.parametrize("n", [4096, 8193, 33000])
def test_attention_decode_2pass_matches_cpu(state, n):
    # src/decode_resident/tests.rs:1544-1565 (q16/kv2/hd256)
    run_attention_case(state, n)


@pytest.mark.parametrize("n", [4096, 8193, 33000])
def test_attention_decode_2pass_d128_matches_cpu(state, n):
    # src/decode_resident/tests.rs:1567-1596 (q32/kv4/hd128)
    run_attention_case(state, n, 32, 4, 128)


@pytest.mark.parametrize("dims", [(4, 2, 16), (4, 4, 64), (8, 1, 32), (6, 2, 96), (2, 1, 40),
                                  (32, 8, 128), (16, 8, 256), (32, 2, 128),
                                  (40, 1, 64), (48, 2, 32),    # these two: more than 16 heads per group
                                  (8, 2, 512), (6, 1, 320), (34, 2, 512)])  # head_dim above 256: four-wavefront workgroups
@pytest.mark.parametrize("n", [3, 100, 1500])
def test_attention_decode_other_shapes(state, dims, n):
    run_attention_case(state, n, *dims)


@pytest.mark.parametrize("dims", [
    (4, 2, 18), (6, 1, 30),   # head_dim not a multiple of four: the merge that reduces through LDS
    (6, 2, 72),               # five column groups: the last merge workgroup has an idle wavefront
    (3, 1, 8), (2, 2, 4),     # fewer columns than a column group
    (16, 16, 64),             # one head per group
])
@pytest.mark.parametrize("n", [40, 700, 5000])
def test_attention_decode_merge_paths(state, dims, n):
    """Split counts from two to the device's fill (n = 40: two or three pages) over the head
    widths that take the merge kernel's less common paths."""
    run_attention_case(state, n, *dims)


def test_qwen_uniform_attention_decode_is_byte_exact_single_key(state):
    # src/decode_resident/tests.rs:1356-1385: one key -> softmax is exactly 1, context == V row
    q_heads, kv_heads, head_dim = 4, 2, 16
    kv_dim = kv_heads * head_dim
    ones = np.ones(head_dim, dtype=np.float32)
    q_raw = pseudo(50_000 + np.arange(q_heads * head_dim))
    k_raw = pseudo(60_000 + np.arange(kv_dim))
    value = pseudo(70_000 + np.arange(kv_dim))
    q = oracle.rms_norm_rope_heads_at(q_raw, q_heads, head_dim, head_dim, ones, 1e-6, 10000.0, 7)
    k = oracle.rms_norm_rope_heads_at(k_raw, kv_heads, head_dim, head_dim, ones, 1e-6, 10000.0, 7)
    kv = state.full_attention_bf16(1, q_heads, kv_heads, head_dim)
    kv.append_row(k, value)
    gpu = kv.attention_decode(q)
    cpu = cpu_attention(q, k, value.reshape(1, -1), q_heads, kv_heads, head_dim)
    assert np.array_equal(gpu, cpu)
    want = np.repeat(oracle.bf16_round(value).reshape(kv_heads, head_dim), q_heads // kv_heads, 0)
    assert np.array_equal(gpu, want.reshape(-1))


@pytest.mark.parametrize("position,seed", [(1, 5), (4, 23), (8, 47)])
def test_gemma_sliding_attention_decode_matches_windowed_oracle(state, position, seed):
    # src/decode_resident/tests.rs:1228-1325: excluded rows carry +2.0 so that including one
    # moves the answer by more than 1e-2
    q_heads, kv_heads, head_dim, window = 4, 2, 256, 4
    n = position + 1
    window_start = max(n - window, 0)
    kv_dim = kv_heads * head_dim
    eps, theta = 1e-6, 10000.0
    d = np.arange(head_dim)
    q_norm = (np.float32(0.75) + np.abs(pseudo(seed + 7 * d))).astype(np.float32)
    k_norm = (np.float32(0.8) + np.abs(pseudo(seed + 11 * d))).astype(np.float32)
    q_raw = pseudo(seed + 20_000 + np.arange(q_heads * head_dim))
    q = oracle.rms_norm_rope_heads_at(q_raw, q_heads, head_dim, head_dim, q_norm, eps, theta,
                                      position).reshape(-1)
    keys = np.empty((n, kv_dim), dtype=np.float32)
    values = np.empty((n, kv_dim), dtype=np.float32)
    for row in range(n):
        k_raw = pseudo(seed + row * 521 + np.arange(kv_dim))
        keys[row] = oracle.rms_norm_rope_heads_at(k_raw, kv_heads, head_dim, head_dim, k_norm,
                                                  eps, theta, row).reshape(-1)
        base = pseudo(seed + 50_000 + row * 523 + np.arange(kv_dim))
        values[row] = base + np.float32(2.0) if row < window_start else base
    kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
    kv.seed(keys, values, n)
    gpu = kv.attention_decode_windowed(q, window_start)
    want = cpu_attention(q, keys, values, q_heads, kv_heads, head_dim, window=window)
    unwindowed = cpu_attention(q, keys, values, q_heads, kv_heads, head_dim)
    delta = np.abs(gpu - want)
    assert delta.max() <= 2.0e-4 and delta.mean() <= 2.0e-5
    if window_start > 0:
        assert np.abs(want - unwindowed).max() > 1.0e-2, "fixture does not discriminate"


@pytest.mark.parametrize("seed", [13, 37, 71])
def test_attention_decode_window_start_zero_is_byte_exact(state, seed):
    # src/decode_resident/tests.rs:1328-1351
    q_heads, kv_heads, head_dim, n = 4, 2, 256, 7
    kv_dim = kv_heads * head_dim
    keys = pseudo(seed + np.arange(n * kv_dim))
    values = pseudo(seed + 10_000 + np.arange(n * kv_dim))
    q = pseudo(seed + 20_000 + np.arange(q_heads * head_dim))
    kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
    kv.seed(keys, values, n)
    assert np.array_equal(kv.attention_decode(q), kv.attention_decode_windowed(q, 0))


def test_attention_errors(state):
    # src/decode_resident/attention.rs:676-690, 745-756
    kv = state.full_attention_bf16(8, 4, 2, 16)
    q = np.zeros(64, dtype=np.float32)
    with pytest.raises(skv.DimensionError):
        kv.attention_decode(q)  # empty KV
    kv.append_row(np.ones(32), np.ones(32))
    with pytest.raises(skv.DimensionError):
        kv.attention_decode(np.zeros(63, dtype=np.float32))
    with pytest.raises(skv.DimensionError):
        kv.attention_decode_windowed(q, 1)  # window_start >= len
    assert kv.attention_decode(q).shape == (64,)


@pytest.mark.parametrize("n,window_start", [(300, 17), (300, 160), (5000, 3977), (5000, 4999)])
def test_windowed_attention_long(state, n, window_start):
    """A window over a long cache equals attention over the truncated cache
    (src/decoder/tests.rs:911-964), on the split-K path too."""
    q_heads, kv_heads, head_dim = 16, 8, 128
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(n + window_start)
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    q = rng.standard_normal(q_heads * head_dim, dtype=np.float32)
    kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    kv.seed(keys, values, n)
    gpu = kv.attention_decode_windowed(q, window_start)
    want = cpu_attention(q, keys[window_start:], values[window_start:], q_heads, kv_heads, head_dim)
    assert np.abs(gpu - want).max() <= 2e-4


def test_normal_inputs_config0(state):
    """BASELINE config 0: 32/8/128, 1024 cached rows N(0,1) in 16-token pages behind a random
    permuted block table; append one row, then decode attention with scale 1/sqrt(128)."""
    q_heads, kv_heads, head_dim, n = 32, 8, 128, 1024
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(0)
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    kv = state.full_attention_bf16(n + 1, q_heads, kv_heads, head_dim)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    kv.seed(keys, values, n)
    k_new = rng.standard_normal(kv_dim, dtype=np.float32)
    v_new = rng.standard_normal(kv_dim, dtype=np.float32)
    q = rng.standard_normal(q_heads * head_dim, dtype=np.float32)
    kv.append_row(k_new, v_new)
    gpu = kv.attention_decode(q)
    lay = oracle.layout(q_heads, kv_heads, head_dim)
    cache = oracle.LayerKvCache("bf16r")
    cache.append_batch(keys, values, lay)
    want = oracle.decode_step(cache, k_new, v_new, q, lay)
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk, cache.keys()) and np.array_equal(gv, cache.values())
    delta = np.abs(gpu - want)
    assert delta.max() <= 1e-4, delta.max()


@pytest.mark.parametrize("q_scale,k_scale,v_scale,tol", [
    # Scores in the hundreds and thousands: softmax is nearly one-hot and near-tied keys
    # trade weight on the last bits of their scores. Against an fp64 evaluation of the same
    # rows the CPU path and the device are equally far off at |score| ~ 100 (2e-4 each); at
    # |score| ~ 1000 the device's two-term bf16 query split (2^-17 relative) shows: 1e-3
    # against the CPU path's 1e-4. The bounds follow that and stay under the contract's 1e-2.
    (30.0, 30.0, 1.0, 8e-3),
    (10.0, 10.0, 1.0, 2e-3),
    (1e-3, 1e-3, 1e4, 8e-4),     # scores ~ 0: uniform weights over large values
    (8.0, 8.0, 1e-6, 8e-4),      # peaked weights over tiny values (no flush to zero in the product)
])
def test_attention_extreme_magnitudes(state, q_scale, k_scale, v_scale, tol):
    """The online softmax (running maximum, base-2 exponent) and the hi/lo operand split must
    neither overflow nor lose the answer when scores are huge, vanish, or values are tiny:
    decode (split context) and a prefill chunk against the CPU path, error relative to the
    scale of the values."""
    q_heads, kv_heads, head_dim, n, chunk = 16, 2, 256, 3000, 80
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(5)
    keys = (rng.standard_normal((n, kv_dim)) * k_scale).astype(np.float32)
    values = (rng.standard_normal((n, kv_dim)) * v_scale).astype(np.float32)
    lay = oracle.layout(q_heads, kv_heads, head_dim)
    cache = oracle.LayerKvCache("bf16r")
    cache.append_batch(keys, values, lay)
    kv = state.full_attention_bf16(n + chunk, q_heads, kv_heads, head_dim)
    kv.seed(keys, values, n)
    q = (rng.standard_normal(q_dim) * q_scale).astype(np.float32)
    got = kv.attention_decode(q)
    want = oracle.cached_attention_one(q, cache, lay)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= tol * v_scale, np.abs(got - want).max()
    qs = (rng.standard_normal((chunk, q_dim)) * q_scale).astype(np.float32)
    ks = (rng.standard_normal((chunk, kv_dim)) * k_scale).astype(np.float32)
    vs = (rng.standard_normal((chunk, kv_dim)) * v_scale).astype(np.float32)
    got = kv.prefill_rows(qs, ks, vs)
    want = oracle.cached_attention_prefill_rows(qs, ks, vs, cache, lay)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= tol * v_scale, np.abs(got - want).max()


# ---- chunked prefill over the cache (multi-query, matrix cores) ----------------------------
@pytest.fixture(params=["by-shape", "one-tile", "two-tiles"])
def tiles_per_wavefront(request):
    """The LDS-shared prefill kernel holds one or two 16-slot query tiles per wavefront; the
    library picks by head_dim and context length (two only for long contexts), the knob forces
    either so that contexts a test can afford reach both instantiations."""
    if request.param == "by-shape":
        yield request.param
        return
    os.environ["SKV_PREFILL_TILES2_MIN_PAGES"] = "0" if request.param == "two-tiles" else "1000000000"
    skv.flags.reload()
    try:
        yield request.param
    finally:
        os.environ.pop("SKV_PREFILL_TILES2_MIN_PAGES", None)
        skv.flags.reload()


@pytest.mark.parametrize("dims,start,chunk,window", [
    ((32, 8, 128), 0, 64, 0),        # first chunk from an empty cache
    ((32, 8, 128), 300, 200, 0),     # later chunk, crosses page boundaries
    ((16, 2, 256), 1000, 37, 0),     # head_dim 256, ragged chunk
    ((16, 2, 256), 5, 3, 0),         # speculative-verify sized chunk (split over the context)
    ((4, 2, 16), 0, 50, 0),
    ((6, 1, 40), 17, 33, 0),         # head_dim padded to 64, GQA 6
    # chunks of 64 query slots and more take the kernel that shares K/V pages through LDS
    ((16, 2, 256), 5000, 600, 0),    # several workgroups per kv head, split context, ragged tail
    ((32, 8, 128), 0, 1000, 0),      # from an empty cache: early tiles see few pages (empty splits)
    ((6, 1, 40), 100, 100, 0),       # rows too short for 16-byte query loads, padded head_dim
    ((8, 1, 32), 33, 77, 0),         # head_dim 32, odd page count
    ((40, 1, 64), 10, 9, 0),         # GQA 40: 360 slots from 9 rows
    ((8, 2, 512), 100, 70, 0),       # head_dim 512: four wavefronts, 64 slots per workgroup
    ((4, 1, 512), 700, 300, 0),      # head_dim 512, several workgroups and splits
    ((4, 1, 320), 0, 33, 0),         # padded to 512
])
def test_prefill_rows_match_per_row_oracle(state, tiles_per_wavefront, dims, start, chunk, window):
    """One launch == the reference's per-row loop (append, then cached_attention_one)."""
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(start * 7 + chunk)
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    kv = state.full_attention_bf16(start + chunk, q_heads, kv_heads, head_dim)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    if start:
        k0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        v0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        kv.seed(k0, v0, start)
        cache.append_batch(k0, v0, lay)
    q = rng.standard_normal((chunk, q_dim), dtype=np.float32)
    k = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    v = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    got = kv.prefill_rows(q, k, v)
    want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
    assert kv.len() == len(cache) == start + chunk
    assert np.abs(got - want).max() <= 1e-4, np.abs(got - want).max()
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk, cache.keys()) and np.array_equal(gv, cache.values())


@pytest.mark.parametrize("window,chunks,heads", [
    (32, [40, 7, 64], (8, 2)), (20, [5, 30, 3], (8, 2)),
    (250, [7, 300, 20], (32, 2)),   # 7-row steps of 16 heads per group: the LDS-shared kernel on a ring
    (100, [130, 50], (64, 4)),
])
def test_prefill_rows_on_ring_layer(state, tiles_per_wavefront, window, chunks, heads):
    """A ring that holds exactly its window advances row by row; results equal the oracle's
    sliding-window attention."""
    (q_heads, kv_heads), head_dim = heads, 64
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(window)
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    kv = state.full_attention_bf16(sum(chunks), q_heads, kv_heads, head_dim, window=window)
    for c in chunks:
        q = rng.standard_normal((c, q_dim), dtype=np.float32)
        k = rng.standard_normal((c, kv_dim), dtype=np.float32)
        v = rng.standard_normal((c, kv_dim), dtype=np.float32)
        got = kv.prefill_rows(q, k, v)
        want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
        assert np.abs(got - want).max() <= 1e-4


def test_prefill_rows_on_ring_layer_head_dim_512(state):
    """head_dim 512 on a ring layer: whole chunks in two phases around the append, on the
    four-wavefront shape of the prefill kernel."""
    q_heads, kv_heads, head_dim, window = 4, 2, 512, 40
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(77)
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    kv = state.full_attention_bf16(120, q_heads, kv_heads, head_dim, window=window)
    for c in (30, 50, 9):
        q = rng.standard_normal((c, q_dim), dtype=np.float32)
        k = rng.standard_normal((c, kv_dim), dtype=np.float32)
        v = rng.standard_normal((c, kv_dim), dtype=np.float32)
        got = kv.prefill_rows(q, k, v)
        want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
        assert np.abs(got - want).max() <= 1e-4


def test_prefill_rows_errors(state):
    kv = state.full_attention_bf16(8, 4, 2, 16)
    with pytest.raises(skv.DimensionError):
        kv.prefill_rows(np.zeros((0, 64)), np.zeros((0, 32)), np.zeros((0, 32)))
    with pytest.raises(skv.DimensionError):
        kv.prefill_rows(np.zeros((2, 64)), np.zeros((3, 32)), np.zeros((2, 32)))
    with pytest.raises(skv.DimensionError):
        kv.prefill_rows(np.zeros((9, 64)), np.zeros((9, 32)), np.zeros((9, 32)))   # over capacity
    assert kv.len() == 0


# ---- kill-switches -----------------------------------------------------------------------
@pytest.fixture
def env_flags():
    saved = {}

    def set_env(**kv):
        for k, v in kv.items():
            saved.setdefault(k, os.environ.get(k))
            os.environ[k] = v
        skv.flags.reload()

    yield set_env
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v
    skv.flags.reload()


@pytest.mark.parametrize("n,dims", [(1, (16, 2, 256)), (257, (16, 2, 256)), (4096, (16, 2, 256)),
                                    (700, (4, 2, 16)), (300, (2, 1, 40))])
def test_flash_sdpa_off_uses_plain_kernel(state, env_flags, n, dims):
    """RETI_RUST_FLASH_SDPA=0 (src/decode_resident/utils.rs:182-185) selects the plain
    three-phase kernel; its sequential sums track the CPU path more closely still."""
    env_flags(RETI_RUST_FLASH_SDPA="0")
    assert not skv.flags.flash_sdpa_enabled()
    gpu = run_attention_case(state, n, *dims)
    env_flags(RETI_RUST_FLASH_SDPA="1")
    again = run_attention_case(state, n, *dims)
    assert np.abs(gpu - again).max() <= 2e-5      # the two device kernels agree with each other


@pytest.mark.parametrize("n", [9000, 40000])
def test_attention_decode_head_dim_512_long_context(state, n):
    """Global layers of Gemma-4-style models (global_head_dim 512, src/config/accessors.rs:118-123)
    at lengths where the context is split."""
    run_attention_case(state, n, 8, 2, 512)


@pytest.mark.parametrize("flash", ["0", "1"])
def test_head_dim_512_with_windows_on_both_kernels(state, env_flags, flash):
    """head_dim 512 on the plain kernel (RETI_RUST_FLASH_SDPA=0) and on the matrix-core kernel;
    the windowed entry masks the rows before window_start on both (the reference's naive kernel
    is its windowed path, src/decode_resident/attention.rs:780-786)."""
    env_flags(RETI_RUST_FLASH_SDPA=flash)
    q_heads, kv_heads, head_dim, n = 4, 2, 512, 90
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(512)
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    q = rng.standard_normal(q_heads * head_dim, dtype=np.float32)
    kv = state.full_attention_bf16(n, q_heads, kv_heads, head_dim)
    kv.seed(keys, values, n)
    for ws in (0, 33):
        got = kv.attention_decode_windowed(q, ws)
        want = cpu_attention(q, keys[ws:], values[ws:], q_heads, kv_heads, head_dim)
        assert np.abs(got - want).max() <= 1e-5
    gk, _ = kv.read_rows_f32()
    assert np.array_equal(gk, oracle.bf16_round(keys))


def test_sdpa_2pass_off_and_min_len(state, env_flags):
    """RETI_RUST_SDPA_2PASS=0 keeps one split; RETI_RUST_SDPA_2PASS_MIN_LEN moves the
    switch-over (src/decode_resident/utils.rs:260-278). Results are split-independent to
    fp32 rounding (the invariant that pins the merge)."""
    base = run_attention_case(state, 3000, 32, 8, 128)
    env_flags(RETI_RUST_SDPA_2PASS="0")
    single = run_attention_case(state, 3000, 32, 8, 128)
    env_flags(RETI_RUST_SDPA_2PASS="1", RETI_RUST_SDPA_2PASS_MIN_LEN="100000")
    assert skv.flags.sdpa_2pass_min_len() == 100000
    below = run_attention_case(state, 3000, 32, 8, 128)
    assert np.abs(base - single).max() <= 2e-6 and np.array_equal(single, below)
    for splits_env in ("64", "1024"):
        os.environ["SKV_DECODE_WGS"] = splits_env
        env_flags(RETI_RUST_SDPA_2PASS_MIN_LEN="128")
        try:
            other = run_attention_case(state, 3000, 32, 8, 128)
        finally:
            os.environ.pop("SKV_DECODE_WGS", None)
        assert np.abs(base - other).max() <= 2e-6


@pytest.mark.parametrize("dims,chunk", [((32, 8, 128), 64), ((32, 8, 128), 1000), ((16, 2, 256), 300), ((6, 1, 40), 50),
                                         ((4, 2, 16), 7)])
@pytest.mark.parametrize("element", ["bf16", "f32"])
def test_first_chunk_matches_causal_attention_divide_form(state, dims, chunk, element):
    """A first chunk from an empty cache is the reference's `causal_attention`
    (src/decoder/attention_ops.rs:1052-1116): scores are dot / sqrt(attn_scalar), a division,
    where the cached path multiplies by the reciprocal. The device takes one form for both; it
    must stay within the bound of either."""
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(chunk * 13 + head_dim)
    lay = oracle.layout(q_heads, kv_heads, head_dim)
    q = rng.standard_normal((chunk, q_dim), dtype=np.float32)
    k = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    v = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    make = state.full_attention_bf16 if element == "bf16" else state.full_attention_f32
    kv = make(chunk, q_heads, kv_heads, head_dim)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    got = kv.prefill_rows(q, k, v)
    # the rows the cache holds (rounded once at the append on a bf16 layer), from the oracle's cache
    rows = oracle.LayerKvCache("bf16r" if element == "bf16" else "f32")
    rows.append_batch(k, v, lay)
    want = oracle.causal_attention(q, rows.keys(), rows.values(), lay)
    assert np.abs(got - want).max() <= (1e-4 if element == "bf16" else 2e-5), np.abs(got - want).max()
    kv.close()


def test_non_finite_row_in_a_chunk_stays_inside_its_launch_tile(state):
    """bf16 rounding of a finite f32 at or above 3.39e38 is an infinity (the reference's rounding
    has no special case, src/decode_resident/utils.rs:55-60), so a live row of a chunk can hold
    one. The reference's causal loop never reads a later row; a multi-query launch shares each
    V page among the query slots of a workgroup and masks by the workgroup's range, so there
    0 x Inf can reach the contexts of earlier query rows of the SAME workgroup tile (at most
    256 query slots). What is asserted: rows that attend the infinite row are non-finite in
    both; every row of an earlier workgroup tile equals the oracle's finite context; the
    infinity is stored as the reference stores it."""
    q_heads, kv_heads, head_dim = 16, 2, 64
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    start, chunk, bad = 100, 200, 150          # the infinite V row is row `bad` of the chunk
    rng = np.random.default_rng(77)
    lay = oracle.layout(q_heads, kv_heads, head_dim)
    cache = oracle.LayerKvCache("bf16r")
    kv = state.full_attention_bf16(start + chunk + 4, q_heads, kv_heads, head_dim)
    k0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
    v0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
    kv.seed(k0, v0, start)
    cache.append_batch(k0, v0, lay)
    q = rng.standard_normal((chunk, q_dim), dtype=np.float32)
    k = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    v = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    v[bad, 5] = np.float32(3.4e38)             # finite in f32, +Inf once rounded to bf16
    got = kv.prefill_rows(q, k, v)
    with np.errstate(invalid="ignore", over="ignore"):
        want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk, cache.keys()) and np.array_equal(gv, cache.values())
    assert np.isinf(gv[start + bad, 5])
    # rows that attend the infinite row: non-finite in that column of the kv head's query heads, in both
    gqa = q_heads // kv_heads
    cols = [h * head_dim + 5 for h in range(gqa)]           # kv head 0 serves query heads 0..gqa-1
    assert not np.isfinite(want[bad:][:, cols]).any() and not np.isfinite(got[bad:][:, cols]).any()
    # a workgroup tile holds at most 256 query slots = 256 / gqa rows: rows before that are untouched
    safe = bad - 256 // gqa
    assert np.isfinite(got[:safe]).all()
    assert np.abs(got[:safe] - want[:safe]).max() <= 1e-4
    kv.close()
