"""Prefix hot cache on the GPU: block snapshot / restore / gather through the hash index
with LRU eviction, bit-exact against re-derived contents and, for the control flow,
against the restatement of the reference's serve algorithm (src/serve/state.rs:560-639)."""
import os

import numpy as np
import pytest

import oracle
import saragossa_amd as skv
from oracle import prefix_cache as pc
from saragossa_amd import BlockHash

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def _stream():
    return torch.cuda.current_stream().cuda_stream


ELEMENT = "bf16"  # what make_layers builds and check_contents expects; see the `element` fixture


@pytest.fixture(params=["bf16", "f32"])
def element(request):
    """Runs a test once per element of the cache (the hot cache copies pages of either)."""
    global ELEMENT
    ELEMENT = request.param
    yield request.param
    ELEMENT = "bf16"


def make_layers(state, n_layers, capacity, dims=(32, 8, 128), seed=0, window=0):
    rng = np.random.default_rng(seed)
    layers = []
    for _ in range(n_layers):
        make = state.full_attention_f32 if ELEMENT == "f32" else state.full_attention_bf16
        kv = make(capacity, *dims, window=window)
        kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
        layers.append(kv)
    return layers


def rows_for(layer, positions, tokens, kv_dim, seed=3):
    """K/V rows as a deterministic function of (layer, position, the token prefix), so that any
    restored row can be re-derived and a wrong block is detected."""
    tokens = np.asarray(tokens, dtype=np.uint64)
    prefix = np.cumsum(tokens * np.uint64(2654435761) + np.uint64(97), dtype=np.uint64)
    out_k = np.empty((len(positions), kv_dim), dtype=np.float32)
    out_v = np.empty_like(out_k)
    cols = np.arange(kv_dim, dtype=np.uint64)
    for i, p in enumerate(positions):
        base = (prefix[p] ^ np.uint64(layer * 7919 + seed * 104729 + p * 31)) & np.uint64(0xFFFFFFFF)
        x = (base * np.uint64(1103515245) + cols * np.uint64(12345)) & np.uint64(0xFFFFFF)
        out_k[i] = (x.astype(np.float32) / np.float32(2 ** 23) - np.float32(1.0))
        out_v[i] = -out_k[i] * np.float32(0.75) + np.float32(0.125)
    return out_k, out_v


def fill(layers, first, last, tokens, kv_dim):
    for li, kv in enumerate(layers):
        k, v = rows_for(li, range(first, last), tokens, kv_dim)
        kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
        kv.encode_append_batch(_stream(), kd.data_ptr(), vd.data_ptr(), last - first)
        torch.cuda.synchronize()


def check_contents(layers, n, tokens, kv_dim):
    for li, kv in enumerate(layers):
        assert kv.len() == n
        k, v = rows_for(li, range(n), tokens, kv_dim)
        if ELEMENT == "f32":
            gk, gv = kv.read_rows_f32()
            assert np.array_equal(gk, k) and np.array_equal(gv, v), f"layer {li}"
            continue
        gk, gv = kv.read_rows()
        assert np.array_equal(gk, oracle.f32_to_bf16_bits(k)), f"layer {li} K"
        assert np.array_equal(gv, oracle.f32_to_bf16_bits(v)), f"layer {li} V"


@pytest.fixture(params=["slot-order", "layer-order"])
def restore_order(request):
    """Both workgroup orders of the restore copy; launches of 64 pages and more take the
    layer order by default, the knob forces it on the small launches of these tests."""
    if request.param == "slot-order":
        yield request.param
        return
    os.environ["SKV_COPY_LAYER_MAJOR_MIN_PAGES"] = "1"
    skv.flags.reload()
    try:
        yield request.param
    finally:
        os.environ.pop("SKV_COPY_LAYER_MAJOR_MIN_PAGES", None)
        skv.flags.reload()


def test_snapshot_restore_roundtrip_and_clone_independence(state, restore_order):
    # the decoder/tests.rs:297-346 pattern: restoring from a copy leaves the entry pristine
    dims, kv_dim, n = (16, 2, 256), 512, 16 * 6
    tokens = list(range(n))
    a = make_layers(state, 3, n, dims, seed=1)
    fill(a, 0, n, tokens, kv_dim)
    snap = skv.snapshot_blocks(state, a, [1, 2, 4], stream=_stream())
    assert snap.estimated_bytes() == 3 * 3 * 2 * 16 * kv_dim * 2
    copy = snap.clone(stream=_stream())
    torch.cuda.synchronize()
    # overwrite the source blocks, then restore into another set of layers at other block ids
    b = make_layers(state, 3, n, dims, seed=2)
    fill(b, 0, n, [t + 1000 for t in tokens], kv_dim)
    skv.restore_blocks(state, copy, b, [0, 5, 3], stream=_stream())
    torch.cuda.synchronize()
    for li in range(3):
        ak, av = a[li].read_rows()
        bk, bv = b[li].read_rows()
        for src, dst in [(1, 0), (2, 5), (4, 3)]:
            assert np.array_equal(bk[dst * 16:dst * 16 + 16], ak[src * 16:src * 16 + 16])
            assert np.array_equal(bv[dst * 16:dst * 16 + 16], av[src * 16:src * 16 + 16])
        k_other, _ = rows_for(li, range(16, 32), [t + 1000 for t in tokens], kv_dim)
        assert np.array_equal(bk[16:32], oracle.f32_to_bf16_bits(k_other))   # untouched block
    # the original snapshot still restores the original bytes after the copy was used
    a[0].truncate(0)
    fill([a[0]], 0, n, [7] * n, kv_dim)
    for kv in a[1:]:
        kv.truncate(0)
        kv.truncate(n)
    a[0].truncate(n)
    skv.restore_blocks(state, snap, a, [1, 2, 4], stream=_stream())
    k0, _ = rows_for(0, range(16, 48), tokens, kv_dim)
    gk, _ = a[0].read_rows(16, 32)
    assert np.array_equal(gk, oracle.f32_to_bf16_bits(k0))
    # shape / count mismatches are Dimension errors (src/decoder/generation.rs:3086-3092)
    with pytest.raises(skv.DimensionError):
        skv.restore_blocks(state, snap, a[:2], [1, 2, 4])
    with pytest.raises(skv.DimensionError):
        skv.restore_blocks(state, snap, a, [1, 2])
    with pytest.raises(skv.DimensionError):
        skv.snapshot_blocks(state, a, [6])       # beyond len
    other = make_layers(state, 3, n, (8, 2, 64))
    with pytest.raises(skv.DimensionError):
        skv.restore_blocks(state, snap, other, [1, 2, 4])


def test_linear_attn_state_snapshot_restore_roundtrip(state):
    # src/metal_backend/tests/linear_attention.rs:12-...: conv (96 KiB) + ssm (2 MiB) per layer
    gen = torch.Generator(device="cuda").manual_seed(5)
    sizes = [3 * 8192 * 4, 32 * 128 * 128 * 4] * 4 + [100]        # an odd-sized buffer too
    bufs = [torch.randint(0, 255, (s,), dtype=torch.uint8, device="cuda", generator=gen)
            for s in sizes]
    want = [b.clone() for b in bufs]
    snap = skv.state_snapshot(state, [b.data_ptr() for b in bufs], sizes, stream=_stream())
    assert snap.estimated_bytes() >= sum(sizes)
    for b in bufs:
        b.zero_()
    skv.state_restore(state, snap, [b.data_ptr() for b in bufs], sizes, stream=_stream())
    torch.cuda.synchronize()
    for b, w in zip(bufs, want):
        assert torch.equal(b, w)
    with pytest.raises(skv.DimensionError):
        skv.state_restore(state, snap, [b.data_ptr() for b in bufs[:-1]], sizes[:-1])


class SimDecoder(pc.PromptDecoder):
    """The oracle side of the multi-turn run: state = number of tokens consumed."""

    class S:
        def __init__(self, n): self.n = n
        def clone(self): return SimDecoder.S(self.n)

    def prefill_uncached(self, tokens): return SimDecoder.S(len(tokens))
    def extend(self, state, tokens): state.n += len(tokens)


@pytest.mark.parametrize("dims,n_layers,bt,prefix,pool_frac,chunk_blocks", [
    ((32, 8, 128), 4, 16, 256, 0.6, 1),  # BASELINE config 3 shapes, scaled down
    ((16, 2, 256), 2, 32, 128, 0.5, 1),  # two pages per hash block
    ((32, 8, 128), 3, 16, 256, 0.6, 8),  # several blocks prefilled and remembered per call
    ((32, 8, 128), 2, 16, 128, 0.15, 5), # a pool so small that blocks of one call evict each other
    ((4, 1, 32), 52, 16, 128, 0.6, 4),   # more layers than one copy launch takes (48): two launches per batch
])
def test_multi_turn_hot_cache_is_bit_exact_and_follows_reference_lru(state, dims, n_layers, bt,
                                                                     prefix, pool_frac,
                                                                     chunk_blocks, restore_order, element):
    kv_dim = dims[1] * dims[2]
    rng = np.random.default_rng(33)
    n_sessions, vocab = 6, 151936
    shared = [int(t) for t in rng.integers(0, vocab, size=prefix)]
    hist = [[int(t) for t in rng.integers(0, vocab, size=rng.integers(bt, 4 * bt))]
            for _ in range(n_sessions)]
    turns = [[int(t) for t in rng.integers(0, vocab, size=2 * bt + 5)] for _ in range(n_sessions)]
    # distinct blocks the traffic produces: the shared prefix once, then each session's own
    demand = len(shared) // bt + sum((len(shared) + len(h) + len(t)) // bt - len(shared) // bt
                                     for h, t in zip(hist, turns))
    pool_blocks = int(demand * pool_frac)
    cap = max(len(shared + h + t) for h, t in zip(hist, turns)) + 16
    proto = make_layers(state, n_layers, 16, dims)
    hot = skv.HotCache(state, bt, 10 ** 6, pool_blocks, proto)
    assert hot.pool_blocks() == pool_blocks and hot.block_bytes() == n_layers * 2 * bt * kv_dim * (4 if element == "f32" else 2)
    # oracle run of the same traffic: byte budget = pool size
    ocache = pc.BlockAwarePrefixCache(bt, 10 ** 6, state_bytes=lambda s, m: 1)
    over = lambda extra: len(ocache.entries) + extra > pool_blocks
    odec = SimDecoder()

    model = skv.LoadedModelKv(hot, enabled=True)

    def run_turn(session_key, tokens):
        layers = make_layers(state, n_layers, cap, dims, seed=len(tokens))
        reused = model.prefill_prompt_state(
            tokens, session_key, layers,
            lambda first, last: fill(layers, first, last, tokens, kv_dim), stream=_stream(),
            blocks_per_chunk=chunk_blocks)
        _, want_reused = pc.prefill_prompt_state(ocache, odec, tokens, session_key, over)
        assert reused == want_reused
        torch.cuda.synchronize()
        check_contents(layers, len(tokens), tokens, kv_dim)
        assert [(e["hash"], e["tokens"]) for e in hot.entries] == \
               [(e.hash, e.tokens) for e in ocache.entries]
        for kv in layers:
            kv.close()
        return reused

    total_reused = 0
    for s in range(n_sessions):                 # first contact: shared prefix + history
        total_reused += run_turn(None, shared + hist[s])
    for s in range(n_sessions):                 # second turn: everything so far + the new turn
        total_reused += run_turn(None, shared + hist[s] + turns[s])
    assert hot.evictions() > 0 and (total_reused > 0 or pool_frac < 0.3)
    assert len(hot) <= pool_blocks and hot.free_blocks() == pool_blocks - len(hot)
    # sessions are isolated by their root
    assert run_turn("agent-a", shared + hist[0]) == 0
    # the kill-switch path prefills everything and touches no cache state
    before = [(e["hash"], e["tokens"]) for e in hot.entries]
    off_layers = make_layers(state, n_layers, cap, dims, seed=5)
    off_tokens = shared + hist[1]
    assert skv.LoadedModelKv(hot, enabled=False).prefill_prompt_state(
        off_tokens, None, off_layers,
        lambda first, last: fill(off_layers, first, last, off_tokens, kv_dim)) == 0
    check_contents(off_layers, len(off_tokens), off_tokens, kv_dim)
    assert [(e["hash"], e["tokens"]) for e in hot.entries] == before
    # drain: evict_lru_block returns the bytes of each victim, then None
    n = len(hot)
    got = [hot.evict_lru_block() for _ in range(n)]
    assert got == [hot.block_bytes()] * n and hot.evict_lru_block() is None
    assert hot.free_blocks() == pool_blocks
    hot.close()


def test_hot_cache_with_recurrent_state_and_skip_when_nothing_to_evict(state):
    dims, kv_dim, bt = (16, 2, 256), 512, 16
    layers = make_layers(state, 2, 64, dims)
    tokens = list(range(100, 148))
    fill(layers, 0, 48, tokens, kv_dim)
    ssm = torch.arange(4096, dtype=torch.float32, device="cuda")
    hot = skv.HotCache(state, bt, 8, 2, layers)
    root = BlockHash.root()
    h1 = BlockHash.chain(root, tokens[:16])
    h2 = BlockHash.chain(h1, tokens[16:32])
    assert hot.remember_prefix_block(root, h1, 16, layers, [ssm.data_ptr()], [ssm.numel() * 4])
    ssm += 1.0
    assert hot.remember_prefix_block(root, h2, 32, layers, [ssm.data_ptr()], [ssm.numel() * 4])
    assert hot.estimated_bytes() == 2 * (hot.block_bytes() + ssm.numel() * 4)
    fresh = make_layers(state, 2, 64, dims, seed=9)
    out = torch.zeros_like(ssm)
    reused, h = hot.match_restore(root, tokens, fresh, [out.data_ptr()], [out.numel() * 4])
    torch.cuda.synchronize()
    assert reused == 32 and h == h2
    assert torch.equal(out, torch.arange(4096, dtype=torch.float32, device="cuda") + 1.0)
    check_contents(fresh, 32, tokens, kv_dim)
    # a pool of one block: remembering another session's block evicts the first and takes over
    # its state buffer; what is restored afterwards is the newcomer's state, byte for byte
    solo = skv.HotCache(state, bt, 8, 1, layers)
    assert solo.remember_prefix_block(root, h1, 16, layers, [ssm.data_ptr()], [ssm.numel() * 4])
    other_root = BlockHash.for_session("another session")
    g1 = BlockHash.chain(other_root, tokens[:16])
    ssm += 5.0
    assert solo.remember_prefix_block(other_root, g1, 16, layers, [ssm.data_ptr()], [ssm.numel() * 4])
    assert solo.evictions() == 1 and len(solo) == 1
    again = make_layers(state, 2, 64, dims, seed=11)
    out.zero_()
    reused, _ = solo.match_restore(other_root, tokens, again, [out.data_ptr()], [out.numel() * 4])
    torch.cuda.synchronize()
    assert reused == 16 and torch.equal(out, ssm)
    check_contents(again, 16, tokens, kv_dim)
    reused, _ = solo.match_restore(root, tokens, again, [out.data_ptr()], [out.numel() * 4])
    assert reused == 0                                        # the evicted block is gone
    # a disabled cache (capacity 0) and a pool with no room and nothing to evict both skip silently
    off = skv.HotCache(state, bt, 0, 2, layers)
    assert not off.remember_prefix_block(root, h1, 16, layers)
    tiny = skv.HotCache(state, bt, 8, 0, layers)
    assert not tiny.remember_prefix_block(root, h1, 16, layers) and tiny.skipped() == 1
    with pytest.raises(skv.DimensionError):
        hot.remember_prefix_block(root, h1, 24, layers)        # not a block boundary
    with pytest.raises(skv.DimensionError):
        hot.remember_prefix_block(root, h1, 64, layers)        # beyond len
    with pytest.raises(skv.ConfigError):
        skv.HotCache(state, 24, 8, 2, layers)                  # not a multiple of the page size


def test_config3_full_size_multi_turn_bit_exact_and_reference_lru(state):
    """BASELINE configs[3] at its full size: 8 sessions share a 4096-token prefix, each adds a
    256..1024-token history and then a 512-token turn; 16-token hash blocks over the 36 layers
    of Qwen3-4B KV (8 kv heads, head_dim 128, bf16); the page pool holds 60 % of the distinct
    blocks, so the LRU evicts. After every turn every row of every layer equals its re-derived
    value bit for bit, the reused-token count equals the oracle's, and the cache's entries are
    the oracle's entries in the oracle's recency order (src/serve/state.rs:560-639,
    src/serve/cache.rs:121-198). Rows are generated and compared on the device."""
    qh, kvh, hd, nl, bt, n_sessions, vocab = 32, 8, 128, 36, 16, 8, 151936
    kv_dim = kvh * hd
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(3)
    shared = rng.integers(0, vocab, size=4096)
    hist = [rng.integers(0, vocab, size=int(rng.integers(256, 1025))) for _ in range(n_sessions)]
    turn = [rng.integers(0, vocab, size=512) for _ in range(n_sessions)]
    base = len(shared) // bt
    demand = base + sum((len(shared) + len(h) + len(t)) // bt - base for h, t in zip(hist, turn))
    pool_blocks = int(demand * 0.6)

    def rows_of(layer, tokens, which):
        t = torch.from_numpy(np.asarray(tokens, dtype=np.int64)).to(dev)
        c = torch.cumsum(t * 2654435761 % 1000003, 0)
        pos = torch.arange(t.numel(), device=dev, dtype=torch.int64)
        d = torch.arange(kv_dim, device=dev, dtype=torch.int64)
        x = (pos[:, None] * 7919 + c[:, None] * 104729 + d[None, :] * 31 + layer * 1299709 + which * 15485863)
        x = (x * 6364136223846793005 + 1442695040888963407) >> 40
        return ((x & 0xffff).to(torch.float32) / 65536.0 - 0.5) * 4.0

    def layers_of(cap, seed):
        out = []
        for i in range(nl):
            kv = state.full_attention_bf16(cap, qh, kvh, hd)
            kv.set_block_table(np.random.default_rng(seed * 100 + i).permutation(kv.pages()).astype(np.int32))
            out.append(kv)
        return out

    proto = layers_of(16, 0)
    hot = skv.HotCache(state, bt, 10 ** 6, pool_blocks, proto)
    model = skv.LoadedModelKv(hot, enabled=True)
    ocache = pc.BlockAwarePrefixCache(bt, 10 ** 6, state_bytes=lambda s, m: 1)
    over = lambda extra: len(ocache.entries) + extra > pool_blocks
    odec = SimDecoder()
    layers = layers_of(len(shared) + 1024 + 512 + 16, 1)
    gk = torch.empty(5700, kv_dim, device=dev, dtype=torch.int16)
    gv = torch.empty(5700, kv_dim, device=dev, dtype=torch.int16)
    totals = dict(reused=0, hits=0)

    def run_turn(tokens):
        n = len(tokens)
        for kv in layers:
            kv.truncate(0)
        ks = [rows_of(i, tokens, 0) for i in range(nl)]
        vs = [rows_of(i, tokens, 1) for i in range(nl)]

        def prefill_rows(first, last):
            for i, kv in enumerate(layers):
                kv.encode_append_batch(_stream(), ks[i][first].data_ptr(), vs[i][first].data_ptr(), last - first)

        reused = model.prefill_prompt_state([int(t) for t in tokens], None, layers, prefill_rows,
                                            stream=_stream(), blocks_per_chunk=32)
        _, want_reused = pc.prefill_prompt_state(ocache, odec, [int(t) for t in tokens], None, over)
        assert reused == want_reused
        for i, kv in enumerate(layers):
            assert kv.len() == n
            kv.encode_gather(_stream(), 0, n, gk.data_ptr(), gv.data_ptr())
            assert torch.equal(gk[:n], ks[i].to(torch.bfloat16).view(torch.int16)), f"K of layer {i}"
            assert torch.equal(gv[:n], vs[i].to(torch.bfloat16).view(torch.int16)), f"V of layer {i}"
        assert [(e["hash"], e["tokens"]) for e in hot.entries] == [(e.hash, e.tokens) for e in ocache.entries]
        totals["reused"] += reused
        totals["hits"] += 1 if reused else 0

    for s in range(n_sessions):
        run_turn(np.concatenate([shared, hist[s]]))
    for s in range(n_sessions):
        run_turn(np.concatenate([shared, hist[s], turn[s]]))
    assert hot.evictions() > 0 and totals["hits"] >= n_sessions and totals["reused"] > 0
    assert len(hot) <= pool_blocks
    hot.close()
    for kv in proto + layers:
        kv.close()


def test_whole_prompt_cache_follows_the_reference(state, element):
    """prefix_cache_get / prefix_cache_put (src/decoder/generation.rs:2998-3025, 3105-3139) on
    the GPU against the oracle's WholePromptCache over the same traffic: same hits, same cached
    lengths, same entries in the same recency order after every request; after a hit the
    layers hold the whole prompt's rows bit for bit and the state buffer holds the state that
    was put with the matched entry."""
    dims, n_layers = (8, 2, 64), 3
    kv_dim = dims[1] * dims[2]
    rng = np.random.default_rng(91)
    tok = lambda n: [int(t) for t in rng.integers(0, 151936, size=n)]
    a, b, c, d, e, f = tok(40), tok(30), tok(33), tok(17), tok(50), tok(21)
    traffic = [a, a + b, c, a[:20], a + b + d, a, e, f, c, a + b + d + tok(3), a + b, []]
    cache = skv.WholePromptCache(state, capacity=3)
    ocache = pc.WholePromptCache(capacity=3)
    assert cache.capacity() == 3 and len(cache) == 0
    state_of = lambda toks: float(len(toks) * 1000 + sum(toks) % 997)
    ssm = torch.zeros(300, device="cuda", dtype=torch.float32)
    ptrs, sizes = [ssm.data_ptr()], [ssm.numel() * 4]

    class S:
        def __init__(self, n): self.n = n
        def clone(self): return S(self.n)

    def o_extend(st, toks): st.n += len(toks)

    for step, prompt in enumerate(traffic):
        layers = make_layers(state, n_layers, 200, dims, seed=step)
        ssm.fill_(-1.0)

        def extend(first, last):
            # what the lookup restored is the matched entry's state
            assert float(ssm[0]) == state_of(prompt[:first]) and float(ssm[-1]) == state_of(prompt[:first])
            fill(layers, first, last, prompt, kv_dim)
            ssm.fill_(state_of(prompt))

        got = cache.get(prompt, layers, extend, ptrs, sizes, stream=_stream())
        want = ocache.get(prompt, o_extend)
        assert (got is None) == (want is None), step
        if got is None:
            if prompt:   # an empty prompt is never cached by the caller (nothing to prefill)
                fill(layers, 0, len(prompt), prompt, kv_dim)
                ssm.fill_(state_of(prompt))
                cache.put(prompt, layers, ptrs, sizes, stream=_stream())
                ocache.put(prompt, S(len(prompt)))
        else:
            assert want.n == len(prompt)
            torch.cuda.synchronize()
            check_contents(layers, len(prompt), prompt, kv_dim)
            assert float(ssm[0]) == state_of(prompt)
        assert cache.entries == [list(t) for t, _ in ocache.entries], step
        assert len(cache) <= 3
        for kv in layers:
            kv.close()
    assert cache.estimated_bytes() > 0
    # the entry a hit restored is independent of what the caller appended afterwards
    layers = make_layers(state, n_layers, 200, dims, seed=50)
    top = cache.entries[0]
    assert cache.lookup(top + [5, 6, 7], layers, ptrs, sizes, stream=_stream()) == len(top)
    torch.cuda.synchronize()
    check_contents(layers, len(top), top, kv_dim)
    # errors precede any copy: too small a layer, a state buffer of another size
    small = make_layers(state, n_layers, 16, dims, seed=51)
    with pytest.raises(skv.DimensionError):
        cache.lookup(top, small, ptrs, sizes, stream=_stream())
    assert all(kv.len() == 0 for kv in small)
    with pytest.raises(skv.DimensionError):
        cache.lookup(top, layers, ptrs, [sizes[0] - 4], stream=_stream())
    with pytest.raises(skv.DimensionError):
        cache.put(top[:5], layers, ptrs, sizes)      # the layers hold len(top) rows, not 5
    # capacity 0: put keeps nothing (generation.rs:3110-3113)
    off = skv.WholePromptCache(state, capacity=0)
    off.put(top, layers, ptrs, sizes, stream=_stream())
    assert len(off) == 0 and off.lookup(top, layers, ptrs, sizes) == 0
    off.close()
    cache.close()


@pytest.mark.parametrize("n_prompt", [40, 96, 300, 1000])
def test_whole_prompt_cache_with_sliding_window_layers(state, element, n_prompt):
    """The whole-prompt cache over a model with sliding-window layers (ring buffers): a prompt
    shorter than the ring, one that just fills it and ones that wrapped it several times. The
    reference's put clones the whole cache whatever the window (generation.rs:3105-3139); its
    sliding layers never attend rows behind the window again, so here an entry holds a ring
    layer's live pages only. After a hit the full layer holds every row, the ring layers the
    last `window` rows, bit for bit, and decode steps on all of them equal the oracle's."""
    dims, window = (8, 2, 64), 64
    kv_dim, q_dim = dims[1] * dims[2], dims[0] * dims[2]
    rng = np.random.default_rng(n_prompt)
    prompt = [int(t) for t in rng.integers(0, 151936, size=n_prompt)]
    tail = [int(t) for t in rng.integers(0, 151936, size=23)]
    windows = [0, window, window]
    make = state.full_attention_f32 if ELEMENT == "f32" else state.full_attention_bf16

    def build():
        out = []
        for li, w in enumerate(windows):
            kv = make(n_prompt + 64, *dims, window=w)
            kv.set_block_table(np.random.default_rng(li + n_prompt).permutation(kv.pages()).astype(np.int32))
            out.append(kv)
        return out

    cache = skv.WholePromptCache(state, capacity=2)
    src = build()
    fill(src, 0, n_prompt, prompt, kv_dim)
    cache.put(prompt, src, stream=_stream())
    dst = build()
    assert cache.lookup(prompt + tail, dst, stream=_stream()) == n_prompt
    torch.cuda.synchronize()
    fill(dst, n_prompt, n_prompt + len(tail), prompt + tail, kv_dim)     # the request goes on from the hit
    n = n_prompt + len(tail)
    mode = "f32" if ELEMENT == "f32" else "bf16r"
    for li, (kv, w) in enumerate(zip(dst, windows)):
        assert kv.len() == n
        first = 0 if w == 0 else max(0, n - w)
        k, v = rows_for(li, range(n), prompt + tail, kv_dim)
        lay = oracle.layout(*dims, sliding_window=w)
        c = oracle.LayerKvCache(mode)
        c.append_batch(k, v, lay)
        gk, gv = kv.read_rows_f32(first, n - first)
        assert np.array_equal(gk, c.keys()[first:]) and np.array_equal(gv, c.values()[first:]), li
        q = rng.standard_normal(q_dim, dtype=np.float32)
        got = kv.attention_decode_windowed(q, skv.flags.window_start(n - 1, w))
        assert np.abs(got - oracle.cached_attention_one(q, c, lay)).max() <= 1e-4, li
    # the entry is untouched by what the request appended: a second hit restores the same rows
    again = build()
    assert cache.lookup(prompt, again, stream=_stream()) == n_prompt
    torch.cuda.synchronize()
    k, v = rows_for(1, range(n_prompt), prompt, kv_dim)
    first = max(0, n_prompt - window)
    c = oracle.LayerKvCache(mode)
    c.append_batch(k, v, oracle.layout(*dims, sliding_window=window))
    gk, gv = again[1].read_rows_f32(first, n_prompt - first)
    assert np.array_equal(gk, c.keys()[first:]) and np.array_equal(gv, c.values()[first:])
    # an entry that holds only a ring layer's window cannot fill a layer that keeps every row
    if n_prompt > window + 48:
        full = [make(n_prompt + 64, *dims) for _ in windows]
        with pytest.raises(skv.DimensionError):
            cache.lookup(prompt, full, stream=_stream())
        assert all(kv.len() == 0 for kv in full)
        for kv in full:
            kv.close()
    for kv in src + dst + again:
        kv.close()
