"""BASELINE.json configurations at their real shapes (layer counts reduced where a layer is
a repeat of another), against the CPU oracle: cache contents bit-exact, attention within 1e-4
(bound held to: 1e-2), plus size-independent properties at full size."""
import numpy as np
import pytest

import oracle
import saragossa_amd as skv

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _seed_device(kv, rows, kv_dim, gen):
    k = torch.randn(rows, kv_dim, device="cuda", dtype=torch.float32, generator=gen)
    v = torch.randn(rows, kv_dim, device="cuda", dtype=torch.float32, generator=gen)
    kv.encode_append_batch(_stream(), k.data_ptr(), v.data_ptr(), rows)
    torch.cuda.synchronize()
    return k.cpu().numpy(), v.cpu().numpy()


def test_config2_hybrid_32k_decode_steps(state):
    """configs[2]: full-attention layers 16/2/256 at 32768 cached rows (2 of the 10 identical
    layers), random block tables, decode steps with fresh q, k, v (20 of them: the cache grows
    past 32784 rows, so the newest rows start a page the block table has not used yet); the 30
    recurrent states (96 KiB conv + 2 MiB ssm each) are snapshotted once and restored
    byte-identically."""
    qh, kvh, hd, ctx, steps, n_layers = 16, 2, 256, 32768, 20, 2
    kv_dim, q_dim = kvh * hd, qh * hd
    gen = torch.Generator(device="cuda").manual_seed(2)
    rng = np.random.default_rng(2)
    lay = oracle.layout(qh, kvh, hd)
    layers, caches = [], []
    for _ in range(n_layers):
        kv = state.full_attention_bf16(ctx + steps, qh, kvh, hd)
        kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
        k, v = _seed_device(kv, ctx, kv_dim, gen)
        c = oracle.LayerKvCache("bf16r")
        c.append_batch(k, v, lay)
        layers.append(kv)
        caches.append(c)
    qs = torch.randn(steps, n_layers, q_dim, device="cuda", generator=gen)
    ks = torch.randn(steps, n_layers, kv_dim, device="cuda", generator=gen)
    vs = torch.randn(steps, n_layers, kv_dim, device="cuda", generator=gen)
    out = torch.empty(steps, n_layers, q_dim, device="cuda")
    for t in range(steps):
        for li, kv in enumerate(layers):
            kv.encode_decode_step(_stream(), ks[t, li].data_ptr(), 0, vs[t, li].data_ptr(), 0,
                                  qs[t, li].data_ptr(), out[t, li].data_ptr())
    got = out.cpu().numpy()
    qn, kn, vn = qs.cpu().numpy(), ks.cpu().numpy(), vs.cpu().numpy()
    worst = 0.0
    for t in range(steps):
        for li in range(n_layers):
            want = oracle.decode_step(caches[li], kn[t, li], vn[t, li], qn[t, li], lay)
            worst = max(worst, float(np.abs(got[t, li] - want).max()))
    assert worst <= 1e-4, worst
    # an implementation that shares nothing with the oracle: the last step of layer 0 again
    # as textbook softmax attention in float64 (torch, on the device) over the rows read back
    # from the cache
    gk, gv = layers[0].read_rows_f32()
    K = torch.from_numpy(gk).cuda().double().view(ctx + steps, kvh, hd)
    V = torch.from_numpy(gv).cuda().double().view(ctx + steps, kvh, hd)
    qd = qs[steps - 1, 0].double().view(kvh, qh // kvh, hd)
    p = torch.softmax(torch.einsum("kgd,nkd->kgn", qd, K) / hd ** 0.5, dim=-1)
    ref = torch.einsum("kgn,nkd->kgd", p, V).reshape(-1)
    assert float((out[steps - 1, 0].double() - ref).abs().max()) <= 1e-5
    for kv, c in zip(layers, caches):
        gk, gv = kv.read_rows_f32(ctx - 40, 40 + steps)
        assert np.array_equal(gk, c.keys()[ctx - 40:]) and np.array_equal(gv, c.values()[ctx - 40:])
    # recurrent state: snapshot once, clobber, restore
    sizes = [3 * 8192 * 4, 32 * 128 * 128 * 4] * 30
    bufs = [torch.randn(s // 4, device="cuda", generator=gen) for s in sizes]
    keep = [b.clone() for b in bufs]
    snap = skv.state_snapshot(state, [b.data_ptr() for b in bufs], sizes, stream=_stream())
    assert snap.estimated_bytes() == sum(sizes)
    for b in bufs:
        b.add_(1.0)
    skv.state_restore(state, snap, [b.data_ptr() for b in bufs], sizes, stream=_stream())
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(bufs, keep))


def test_config4_sliding_window_model_batch1_and_batch4(state):
    """configs[4]: 16/8/256, local layers keep a 1024-token ring, global layers the full paged
    cache at 65536 rows, local:global 5:1 (one group of six layers); decode steps at batch 1
    and at batch 4 with independent sequences that own their tables."""
    qh, kvh, hd, ctx, window = 16, 8, 256, 65536, 1024
    kv_dim, q_dim = kvh * hd, qh * hd
    gen = torch.Generator(device="cuda").manual_seed(4)
    rng = np.random.default_rng(4)

    def build_sequence(steps, rows=ctx):
        layers, caches, lays = [], [], []
        for li in range(6):
            is_global = (li + 1) % 6 == 0          # src/decoder.rs:890-898
            w = 0 if is_global else window
            kv = state.full_attention_bf16(rows + steps, qh, kvh, hd, window=w)
            kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
            lay = oracle.layout(qh, kvh, hd, sliding_window=w)
            c = oracle.LayerKvCache("bf16r")
            if is_global:
                k, v = _seed_device(kv, rows, kv_dim, gen)
                c.append_batch(k, v, lay)
            else:
                # a local layer only ever attends its last `window` rows, so it starts with its
                # window exactly full (position 1024) and wraps within the first decode steps
                k, v = _seed_device(kv, min(window, rows), kv_dim, gen)
                c.append_batch(k, v, lay)
            layers.append(kv)
            caches.append(c)
            lays.append(lay)
        return layers, caches, lays

    def run(seqs, steps):
        worst = 0.0
        for t in range(steps):
            for layers, caches, lays in seqs:
                for kv, c, lay in zip(layers, caches, lays):
                    q = torch.randn(q_dim, device="cuda", generator=gen)
                    k = torch.randn(kv_dim, device="cuda", generator=gen)
                    v = torch.randn(kv_dim, device="cuda", generator=gen)
                    o = torch.empty(q_dim, device="cuda")
                    kv.encode_decode_step(_stream(), k.data_ptr(), 0, v.data_ptr(), 0, q.data_ptr(),
                                          o.data_ptr())
                    want = oracle.decode_step(c, k.cpu().numpy(), v.cpu().numpy(), q.cpu().numpy(), lay)
                    worst = max(worst, float(np.abs(o.cpu().numpy() - want).max()))
        return worst

    def run_batched(seqs, steps):
        """One skv_decode_step_batch_device call per layer covers all the sequences."""
        worst = 0.0
        n = len(seqs)
        for t in range(steps):
            for li in range(6):
                q = torch.randn(n, q_dim, device="cuda", generator=gen)
                k = torch.randn(n, kv_dim, device="cuda", generator=gen)
                v = torch.randn(n, kv_dim, device="cuda", generator=gen)
                o = torch.empty(n, q_dim, device="cuda")
                skv.encode_decode_step_batch([s[0][li] for s in seqs], _stream(),
                                             [k[i].data_ptr() for i in range(n)],
                                             [v[i].data_ptr() for i in range(n)],
                                             [q[i].data_ptr() for i in range(n)],
                                             [o[i].data_ptr() for i in range(n)])
                got, qh_, kh_, vh_ = o.cpu().numpy(), q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()
                for i, (_, caches, lays) in enumerate(seqs):
                    want = oracle.decode_step(caches[li], kh_[i], vh_[i], qh_[i], lays[li])
                    worst = max(worst, float(np.abs(got[i] - want).max()))
        return worst

    slack_pages = 2   # a ring keeps 32 rows behind its window
    one = [build_sequence(4)]
    assert run(one, 4) <= 1e-4
    # ring layers hold their window (plus the slack) after wrapping; global layer keeps everything
    layers, caches, _ = one[0]
    assert layers[0].pages() == window // 16 + slack_pages and layers[5].pages() == (ctx + 4 + 15) // 16
    gk, _ = layers[0].read_rows_f32(layers[0].len() - window, window)
    assert np.array_equal(gk, caches[0].keys()[-window:])
    # independent of the oracle: one more attention over the global layer (all 65540 rows) and
    # over a ring layer (its last 1024 rows) against float64 softmax attention in torch
    for li in (5, 0):
        kv = layers[li]
        n = kv.len()
        first = 0 if li == 5 else n - window
        gk, gv = kv.read_rows_f32(first, n - first)
        K = torch.from_numpy(gk).cuda().double().view(n - first, kvh, hd)
        V = torch.from_numpy(gv).cuda().double().view(n - first, kvh, hd)
        q = torch.randn(q_dim, device="cuda", generator=gen)
        o = torch.empty(q_dim, device="cuda")
        kv.encode_attention_decode_windowed(_stream(), q.data_ptr(), o.data_ptr(), first)
        p = torch.softmax(torch.einsum("kgd,nkd->kgn", q.double().view(kvh, qh // kvh, hd), K) / hd ** 0.5, dim=-1)
        ref = torch.einsum("kgn,nkd->kgd", p, V).reshape(-1)
        assert float((o.double() - ref).abs().max()) <= 1e-5, li
    for kv in layers:
        kv.close()
    del one, layers, caches
    # batch 4 at full size: four independent sequences at 65536 rows, every layer's step for
    # the four of them in one launch pair (skv_decode_step_batch_device)
    four = [build_sequence(3) for _ in range(4)]
    assert run_batched(four, 3) <= 1e-4
    # sequences are independent: same layer index, different contents
    a, _ = four[0][0][5].read_rows(ctx, 3)
    b, _ = four[1][0][5].read_rows(ctx, 3)
    assert not np.array_equal(a, b)
    for layers, _, _ in four:
        for kv in layers:
            kv.close()
    del four
    # sequences of unequal length in one batch: the workgroup budget is shared in proportion,
    # the short ones take fewer splits (down to one) and their rings are at different fills
    mixed = [build_sequence(5, rows=r) for r in (65536, 9000, 700, 40)]
    assert run_batched(mixed, 5) <= 1e-4
    for (layers, caches, _), r in zip(mixed, (65536, 9000, 700, 40)):
        gk, gv = layers[5].read_rows_f32(r - 10, 15)
        assert np.array_equal(gk, caches[5].keys()[r - 10:]) and np.array_equal(gv, caches[5].values()[r - 10:])
        n = layers[0].len()
        first = max(0, n - window)
        gk, _ = layers[0].read_rows_f32(first, n - first)
        assert np.array_equal(gk, caches[0].keys()[first:])


def test_config4_batch_of_unequal_sequences_on_f32_layers(state):
    """configs[4]'s group of six layers with the f32 element (what greedy decoding keeps), four
    sequences of very different lengths per call: every layer's step for the four of them is one
    launch pair of the f32 batch kernel (global layer at 65536 rows, rings at different fills)."""
    qh, kvh, hd, window = 16, 8, 256, 1024
    kv_dim, q_dim = kvh * hd, qh * hd
    gen = torch.Generator(device="cuda").manual_seed(44)
    rng = np.random.default_rng(44)
    lengths, steps = (65536, 9000, 700, 40), 3
    seqs = []
    for rows in lengths:
        layers, caches, lays = [], [], []
        for li in range(6):
            w = 0 if (li + 1) % 6 == 0 else window
            kv = state.full_attention_f32(rows + steps, qh, kvh, hd, window=w)
            kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
            lay = oracle.layout(qh, kvh, hd, sliding_window=w)
            c = oracle.LayerKvCache("f32")
            k, v = _seed_device(kv, rows if w == 0 else min(window, rows), kv_dim, gen)
            c.append_batch(k, v, lay)
            layers.append(kv)
            caches.append(c)
            lays.append(lay)
        seqs.append((layers, caches, lays))
    n = len(seqs)
    worst = 0.0
    for _ in range(steps):
        for li in range(6):
            q = torch.randn(n, q_dim, device="cuda", generator=gen)
            k = torch.randn(n, kv_dim, device="cuda", generator=gen)
            v = torch.randn(n, kv_dim, device="cuda", generator=gen)
            o = torch.empty(n, q_dim, device="cuda")
            skv.encode_decode_step_batch([s[0][li] for s in seqs], _stream(),
                                         [k[i].data_ptr() for i in range(n)], [v[i].data_ptr() for i in range(n)],
                                         [q[i].data_ptr() for i in range(n)], [o[i].data_ptr() for i in range(n)])
            got, qh_, kh_, vh_ = o.cpu().numpy(), q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()
            for i, (_, caches, lays) in enumerate(seqs):
                want = oracle.decode_step(caches[li], kh_[i], vh_[i], qh_[i], lays[li])
                worst = max(worst, float(np.abs(got[i] - want).max()))
    assert worst <= 2e-5
    for (layers, caches, _), r in zip(seqs, lengths):
        gk, gv = layers[5].read_rows_f32(r - 10, 10 + steps)
        assert np.array_equal(gk, caches[5].keys()[r - 10:]) and np.array_equal(gv, caches[5].values()[r - 10:])
        m = layers[0].len()
        first = max(0, m - window)
        gk, _ = layers[0].read_rows_f32(first, m - first)
        assert np.array_equal(gk, caches[0].keys()[first:])
        for kv in layers:
            kv.close()


def test_config4_local_layer_chunked_prefill_on_the_ring(state):
    """BASELINE configs[4] local layer (q16/kv8/hd256, window 1024 = the ring's rows exactly):
    a prompt prefilled in 512-row chunks equals the oracle's per-row sliding-window attention,
    and decode continues from the ring it leaves."""
    q_heads, kv_heads, head_dim, window = 16, 8, 256, 1024
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    rng = np.random.default_rng(44)
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("bf16r")
    n_prompt, chunk = 1536 + 100, 512
    kv = state.full_attention_bf16(n_prompt + 8, q_heads, kv_heads, head_dim, window=window)
    assert kv.pages() == window // 16 + 2   # the window plus 32 rows of slack
    worst = 0.0
    for first in range(0, n_prompt, chunk):
        c = min(chunk, n_prompt - first)
        q = rng.standard_normal((c, q_dim), dtype=np.float32)
        k = rng.standard_normal((c, kv_dim), dtype=np.float32)
        v = rng.standard_normal((c, kv_dim), dtype=np.float32)
        got = kv.prefill_rows(q, k, v)
        want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
        worst = max(worst, float(np.abs(got - want).max()))
    assert worst <= 1e-4, worst
    assert kv.len() == len(cache) == n_prompt
    gk, gv = kv.read_rows_f32(n_prompt - window, window)
    assert np.array_equal(gk, cache.keys()[-window:]) and np.array_equal(gv, cache.values()[-window:])
    for _ in range(4):
        q = rng.standard_normal(q_dim, dtype=np.float32)
        k = rng.standard_normal(kv_dim, dtype=np.float32)
        v = rng.standard_normal(kv_dim, dtype=np.float32)
        kv.append_row(k, v)
        want = oracle.decode_step(cache, k, v, q, lay)
        got = kv.attention_decode_windowed(q, skv.flags.window_start(kv.len() - 1, window))
        assert np.abs(got - want).max() <= 1e-4
