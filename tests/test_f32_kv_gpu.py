"""The f32 element of the cache (KvElement::F32, src/decode_resident/attention.rs:26-108):
what full_attention chooses for greedy decoding unless RETI_RUST_KV_BF16 says otherwise
(src/decode_resident/utils.rs:202-229). Rows are kept verbatim, so contents are compared bit
for bit with the oracle's f32 cache, and attention with cached_attention_one on it (the
reference's own bound for its f32 GPU path is 1e-4, tests.rs:1443-1492; the bound to hold here
is 1e-2)."""
import os

import numpy as np
import pytest

import oracle
import saragossa_amd as skv
from test_prekv_gpu import run_gated, run_prekv

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

TOL = 2e-5


@pytest.fixture
def env_flags():
    saved = {k: os.environ.get(k) for k in ("RETI_RUST_KV_BF16",)}
    yield os.environ
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v
    skv.flags.reload()


def _filled(state, dims, n, seed, window=0, cap=None):
    q_heads, kv_heads, head_dim = dims
    kv_dim = kv_heads * head_dim
    rng = np.random.default_rng(seed)
    kv = state.full_attention_f32(cap or n + 8, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("f32")
    keys = rng.standard_normal((n, kv_dim), dtype=np.float32)
    values = rng.standard_normal((n, kv_dim), dtype=np.float32)
    if n:
        kv.seed(keys, values, n)
        cache.append_batch(keys, values, lay)
    return kv, cache, lay, rng


def test_policy_chooses_the_element(state, env_flags):
    # kv_bf16_for: the override wins, else bf16 when sampling and f32 for greedy decoding
    env_flags.pop("RETI_RUST_KV_BF16", None)
    skv.flags.reload()
    greedy = state.full_attention(64, 8, 2, 64, sampled=False)
    sampled = state.full_attention(64, 8, 2, 64, sampled=True)
    assert greedy.byte_len() == 64 * 2 * 64 * 4 and sampled.byte_len() == 64 * 2 * 64 * 2
    env_flags["RETI_RUST_KV_BF16"] = "1"
    skv.flags.reload()
    assert state.full_attention(64, 8, 2, 64, sampled=False).byte_len() == 64 * 2 * 64 * 2
    env_flags["RETI_RUST_KV_BF16"] = "off"
    skv.flags.reload()
    assert state.full_attention(64, 8, 2, 64, sampled=True).byte_len() == 64 * 2 * 64 * 4


@pytest.mark.parametrize("dims", [(16, 2, 256), (32, 8, 128), (8, 8, 64), (6, 2, 96), (6, 1, 40), (4, 2, 16),
                                  (4, 1, 320), (8, 2, 512)])
def test_rows_are_kept_verbatim(state, dims):
    kv, cache, lay, rng = _filled(state, dims, 333, seed=dims[2])
    kv_dim = dims[1] * dims[2]
    special = np.array([0.0, -0.0, 1e-45, -1e-38, 3.4e38, np.inf, -np.inf, 1.0 + 2.0 ** -23], np.float32)
    k1 = np.resize(special, kv_dim).astype(np.float32)
    v1 = np.resize(special[::-1], kv_dim).astype(np.float32)
    kv.append_row(k1, v1)
    cache.append(k1[None], v1[None], lay)
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk.view(np.uint32), cache.keys().view(np.uint32))
    assert np.array_equal(gv.view(np.uint32), cache.values().view(np.uint32))
    gk2, _ = kv.read_rows_f32(17, 40)
    assert np.array_equal(gk2, cache.keys()[17:57])
    with pytest.raises(skv.ConfigError):
        kv.read_rows()  # bf16 bit patterns of an f32 layer
    kv.truncate(100)
    assert kv.len() == 100
    with pytest.raises(skv.DimensionError):
        kv.read_rows_f32(90, 20)


@pytest.mark.parametrize("dims,n", [((16, 2, 256), 1), ((16, 2, 256), 257), ((16, 2, 256), 33000),
                                    ((32, 8, 128), 4096), ((6, 1, 40), 1500), ((40, 1, 64), 700),
                                    ((4, 4, 16), 100), ((8, 2, 512), 9000), ((4, 1, 320), 300)])
def test_attention_decode_matches_cpu(state, dims, n):
    kv, cache, lay, rng = _filled(state, dims, n, seed=n)
    q = rng.standard_normal(dims[0] * dims[2], dtype=np.float32)
    got = kv.attention_decode(q)
    want = oracle.cached_attention_one(q, cache, lay)
    assert np.abs(got - want).max() <= TOL, np.abs(got - want).max()
    # a window start inside the cache
    if n > 20:
        ws = n // 3
        got = kv.attention_decode_windowed(q, ws)
        sub = oracle.LayerKvCache("f32")
        sub.append_batch(cache.keys()[ws:], cache.values()[ws:], lay)
        assert np.abs(got - oracle.cached_attention_one(q, sub, lay)).max() <= TOL


@pytest.mark.parametrize("dims,start,chunk", [((16, 2, 256), 5000, 300), ((32, 8, 128), 0, 700),
                                               ((16, 2, 256), 5, 3), ((6, 1, 40), 100, 100),
                                               ((4, 1, 512), 700, 150)])
def test_prefill_rows_match_per_row_oracle(state, dims, start, chunk):
    q_heads, kv_heads, head_dim = dims
    kv, cache, lay, rng = _filled(state, dims, start, seed=start + chunk, cap=start + chunk)
    q = rng.standard_normal((chunk, q_heads * head_dim), dtype=np.float32)
    k = rng.standard_normal((chunk, kv_heads * head_dim), dtype=np.float32)
    v = rng.standard_normal((chunk, kv_heads * head_dim), dtype=np.float32)
    got = kv.prefill_rows(q, k, v)
    want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
    assert np.abs(got - want).max() <= TOL, np.abs(got - want).max()
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk, cache.keys()) and np.array_equal(gv, cache.values())


def test_ring_layer_chunks_and_steps(state):
    dims, window = (8, 2, 64), 100
    kv, cache, lay, rng = _filled(state, dims, 0, seed=5, window=window, cap=2000)
    q_dim, kv_dim = dims[0] * dims[2], dims[1] * dims[2]
    for chunk in (70, 1, 250, 33, 1, 1, 112):
        q = rng.standard_normal((chunk, q_dim), dtype=np.float32)
        k = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
        v = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
        got = kv.prefill_rows(q, k, v)
        want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
        assert np.abs(got - want).max() <= TOL
    n = kv.len()
    gk, gv = kv.read_rows_f32(n - window, window)
    assert np.array_equal(gk, cache.keys()[n - window:]) and np.array_equal(gv, cache.values()[n - window:])


def test_snapshot_restore_and_hot_cache_on_f32_layers(state):
    dims = (8, 2, 128)
    layers, caches = [], []
    for li in range(3):
        kv, cache, lay, rng = _filled(state, dims, 160, seed=40 + li, cap=400)
        layers.append(kv)
        caches.append(cache)
    snap = skv.snapshot_blocks(state, layers, [1, 4, 9])
    assert snap.estimated_bytes() == 3 * 3 * 2 * 16 * dims[1] * dims[2] * 4
    others = [_filled(state, dims, 160, seed=90 + li, cap=400)[0] for li in range(3)]
    skv.restore_blocks(state, snap, others, [1, 4, 9])
    for kv, cache in zip(others, caches):
        gk, gv = kv.read_rows_f32()
        for p in (1, 4, 9):
            assert np.array_equal(gk[p * 16:(p + 1) * 16], cache.keys()[p * 16:(p + 1) * 16])
            assert np.array_equal(gv[p * 16:(p + 1) * 16], cache.values()[p * 16:(p + 1) * 16])
    # the hot cache: remember two blocks of 32 tokens, restore them into fresh layers
    hot = skv.HotCache(state, 32, 8, 8, layers)
    root = skv.BlockHash.root()
    tokens = list(range(64))
    h1 = skv.BlockHash.chain(root, tokens[:32])
    h2 = skv.BlockHash.chain(h1, tokens[32:])
    assert hot.remember_prefix_block(root, h1, 32, layers)
    assert hot.remember_prefix_block(root, h2, 64, layers)
    fresh = [state.full_attention_f32(400, *dims) for _ in range(3)]
    assert hot.match_restore(root, tokens + [7, 8, 9], fresh)[0] == 64
    for kv, cache in zip(fresh, caches):
        assert kv.len() == 64
        gk, gv = kv.read_rows_f32()
        assert np.array_equal(gk, cache.keys()[:64]) and np.array_equal(gv, cache.values()[:64])
    # layers of the other element do not fit the pool, not even when their pages have the
    # same size (bf16 at twice the head_dim)
    with pytest.raises(skv.KvError):
        hot.remember_prefix_block(root, h1, 32, [state.full_attention_bf16(400, *dims) for _ in range(3)])
    with pytest.raises(skv.KvError):
        hot.remember_prefix_block(root, h1, 32, [state.full_attention_bf16(400, 8, 2, 256) for _ in range(3)])
    with pytest.raises(skv.KvError):
        skv.restore_blocks(state, snap, [state.full_attention_bf16(400, 8, 2, 256) for _ in range(3)], [1, 4, 9])


def test_device_steps_on_f32_layers(state):
    # wide f32 heads: norm and rotation, append and attention as launches of their own
    run_prekv(state, (8, 2, 512), 0, 300, 20, 128, 1.0e6, None, (True, True), element="f32")
    run_prekv(state, (4, 2, 384), 40, 10, 60, 96, 1.0e6, 300.0, (True, False), element="f32")
    run_gated(state, (4, 2, 512), 0, 100, 20, 128, 1.0e6, element="f32")
    # the pre-KV and gated entry points are one launch pair on an f32 layer too (head_dim <= 256)
    run_prekv(state, (16, 2, 256), 0, 300, 6, 64, 1.0e7, None, (True, True), element="f32")
    run_prekv(state, (8, 2, 64), 40, 100, 30, 64, 1.0e6, None, (True, False), element="f32")
    run_gated(state, (16, 2, 256), 0, 200, 5, 64, 1.0e7, element="f32")


@pytest.mark.parametrize("dims,start,window", [((16, 2, 256), 0, 0), ((16, 2, 256), 4090, 0), ((32, 8, 128), 1000, 0),
                                               ((8, 2, 64), 15, 0), ((4, 1, 80), 31, 0), ((16, 8, 256), 100, 64),
                                               ((16, 2, 256), 20000, 0),
                                               # shapes whose step is an append launch, then the kernel that also
                                               # serves chunks: wide heads, padded wide heads, more than 16 heads per
                                               # group, from empty, on a ring, split-K
                                               ((16, 8, 512), 0, 0), ((4, 1, 320), 2040, 0), ((8, 2, 512), 9000, 0),
                                               ((8, 2, 512), 40, 48), ((40, 2, 64), 500, 0), ((20, 1, 128), 3, 32)])
def test_fused_decode_steps_on_f32_layers(state, dims, start, window):
    """skv_decode_step_device on an f32 layer is one launch pair: the attention kernel stores the
    new row itself and patches it into the registers of the wavefront that walks its page
    (encode_append_kv + attention_decode, src/decode_resident/attention.rs:941-1038). Steps
    across page boundaries, from an empty cache, on a ring, with four and with eight
    wavefronts: rows bit for bit, contexts within the f32 bound."""
    q_dim, kv_dim = dims[0] * dims[2], dims[1] * dims[2]
    kv, cache, lay, rng = _filled(state, dims, start, seed=start + dims[2], window=window, cap=start + 64)
    stream = torch.cuda.current_stream().cuda_stream
    for step in range(35):
        k = rng.standard_normal(kv_dim, dtype=np.float32)
        v = rng.standard_normal(kv_dim, dtype=np.float32)
        q = rng.standard_normal(q_dim, dtype=np.float32)
        kd, vd, qd = (torch.from_numpy(a).cuda() for a in (k, v, q))
        out = torch.empty(q_dim, device="cuda")
        if step % 5 == 4:   # the variant that allocates nothing shares the kernels
            kv.encode_decode_step_static(stream, kd.data_ptr(), 0, vd.data_ptr(), 0, qd.data_ptr(), out.data_ptr())
        else:
            kv.encode_decode_step(stream, kd.data_ptr(), 0, vd.data_ptr(), 0, qd.data_ptr(), out.data_ptr())
        want = oracle.decode_step(cache, k, v, q, lay)
        assert np.abs(out.cpu().numpy() - want).max() <= TOL, step
    n = kv.len()
    assert n == start + 35
    keep = min(n, window) if window else n
    gk, gv = kv.read_rows_f32(n - keep, keep)
    assert np.array_equal(gk, cache.keys()[n - keep:]) and np.array_equal(gv, cache.values()[n - keep:])


@pytest.mark.parametrize("dims,lens,window,steps", [
    ((16, 2, 256), (50, 700, 3000), 0, 3),          # configs[2]'s heads, lengths far apart
    ((16, 2, 256), (15, 16, 31, 1), 0, 20),         # page boundaries crossed inside the run
    ((32, 8, 128), (2047, 5, 333, 900, 64), 0, 4),  # configs[1]'s heads
    ((8, 8, 64), (200, 40), 0, 5),                  # one head per group
    ((10, 2, 80), (90, 300, 17), 0, 6),             # padded head_dim, five heads per group
    ((16, 4, 128), (100, 30, 70), 48, 40),          # rings: the window slides and wraps
    ((4, 1, 320), (40, 200), 0, 3),                 # head_dim above 256: one launch pair per sequence
])
def test_decode_step_batch_on_f32_layers(state, dims, lens, window, steps):
    """skv_decode_step_batch_device on f32 layers: up to head_dim 256 and 16 heads per group one
    launch pair appends and attends every sequence (f32_decode_batch_kernel); contexts and the
    rows the launch stored are checked against the oracle's decode_step per sequence."""
    q_dim, kv_dim = dims[0] * dims[2], dims[1] * dims[2]
    seqs = [_filled(state, dims, n, seed=n, window=window, cap=n + steps + 8) for n in lens]
    rng = np.random.default_rng(3)
    for _ in range(steps):
        rows = [(rng.standard_normal(kv_dim, dtype=np.float32), rng.standard_normal(kv_dim, dtype=np.float32),
                 rng.standard_normal(q_dim, dtype=np.float32)) for _ in seqs]
        dev = [[torch.from_numpy(a).cuda() for a in r] for r in rows]
        outs = [torch.empty(q_dim, device="cuda") for _ in seqs]
        skv.encode_decode_step_batch([s[0] for s in seqs], torch.cuda.current_stream().cuda_stream,
                                     [d[0].data_ptr() for d in dev], [d[1].data_ptr() for d in dev],
                                     [d[2].data_ptr() for d in dev], [o.data_ptr() for o in outs])
        for (kv, cache, lay, _), (k, v, q), o in zip(seqs, rows, outs):
            want = oracle.decode_step(cache, k, v, q, lay)
            assert np.abs(o.cpu().numpy() - want).max() <= TOL
    for (kv, cache, lay, _), n0 in zip(seqs, lens):
        n = kv.len()
        assert n == n0 + steps
        keep = min(n, window) if window else n
        gk, gv = kv.read_rows_f32(n - keep, keep)
        assert np.array_equal(gk, cache.keys()[n - keep:]) and np.array_equal(gv, cache.values()[n - keep:])


def test_head_dim_above_512_is_rejected_loudly(state):
    with pytest.raises(skv.ConfigError):
        state.full_attention_f32(64, 4, 1, 520)


@pytest.mark.parametrize("dims,n", [((16, 2, 256), 700), ((6, 1, 40), 300), ((4, 1, 320), 90)])
def test_flash_sdpa_off_uses_the_plain_kernel_on_f32_rows(state, dims, n):
    """RETI_RUST_FLASH_SDPA=0 (src/decode_resident/utils.rs:182-185): the plain three-phase
    kernel reads the f32 tiles too; its sequential sums are an independent check of the matrix
    kernel."""
    kv, cache, lay, rng = _filled(state, dims, n, seed=n)
    q = rng.standard_normal(dims[0] * dims[2], dtype=np.float32)
    want = oracle.cached_attention_one(q, cache, lay)
    saved = os.environ.get("RETI_RUST_FLASH_SDPA")
    try:
        os.environ["RETI_RUST_FLASH_SDPA"] = "0"
        skv.flags.reload()
        assert not skv.flags.flash_sdpa_enabled()
        plain = kv.attention_decode(q)
    finally:
        if saved is None:
            os.environ.pop("RETI_RUST_FLASH_SDPA", None)
        else:
            os.environ["RETI_RUST_FLASH_SDPA"] = saved
        skv.flags.reload()
    matrix = kv.attention_decode(q)
    assert np.abs(plain - want).max() <= 2e-6
    assert np.abs(plain - matrix).max() <= TOL
