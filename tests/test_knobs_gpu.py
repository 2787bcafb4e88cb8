"""The launch-shaping environment knobs choose among kernel instantiations and grids, never among
results: under each setting a decode run (fused append, ring included), a batch step and a
prefill chunk on both elements must match the oracle exactly as they do by default."""
import os

import numpy as np
import pytest
import torch

import oracle
import saragossa_amd as skv

pytestmark = pytest.mark.gpu

KNOBS = [
    {"SKV_DECODE_WAVES": "4"},
    {"SKV_DECODE_WAVES": "8", "SKV_DECODE_WGS": "1024"},
    {"SKV_DECODE_WGS": "16"},
    {"SKV_DECODE_MIN_PAGES": "4"},
    {"SKV_FUSED_APPEND": "0"},
    {"SKV_Q_VEC": "0"},
    {"SKV_PREFILL_TILES": "0"},
    {"SKV_PREFILL_TILES2_MIN_PAGES": "0", "SKV_PREFILL_WGS": "64"},
    {"SKV_PREFILL_MAX_SPLITS": "1"},
]


@pytest.fixture(params=KNOBS, ids=lambda k: ",".join("%s=%s" % kv for kv in k.items()))
def knobs(request):
    saved = {k: os.environ.get(k) for k in request.param}
    os.environ.update(request.param)
    skv.flags.reload()
    yield request.param
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v
    skv.flags.reload()


def _layer(state, element, dims, n, window, cap, rng):
    q_heads, kv_heads, head_dim = dims
    kv_dim = kv_heads * head_dim
    make = state.full_attention_f32 if element == "f32" else state.full_attention_bf16
    kv = make(cap, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("f32" if element == "f32" else "bf16r")
    if n:
        k0 = rng.standard_normal((n, kv_dim), dtype=np.float32)
        v0 = rng.standard_normal((n, kv_dim), dtype=np.float32)
        kv.seed(k0, v0, n)
        cache.append_batch(k0, v0, lay)
    return kv, cache, lay


@pytest.mark.parametrize("element,tol", [("bf16", 1e-4), ("f32", 2e-5)])
@pytest.mark.parametrize("dims,n,window", [((16, 2, 256), 1500, 0), ((32, 8, 128), 60, 0), ((8, 2, 64), 70, 48)])
def test_decode_steps_under_knobs(state, knobs, element, tol, dims, n, window):
    rng = np.random.default_rng(n)
    steps = 20
    kv, cache, lay = _layer(state, element, dims, n, window, n + steps + 8, rng)
    q_dim, kv_dim = dims[0] * dims[2], dims[1] * dims[2]
    stream = torch.cuda.current_stream().cuda_stream
    out = torch.empty(q_dim, device="cuda")
    for step in range(steps):
        k = rng.standard_normal(kv_dim, dtype=np.float32)
        v = rng.standard_normal(kv_dim, dtype=np.float32)
        q = rng.standard_normal(q_dim, dtype=np.float32)
        kd, vd, qd = (torch.from_numpy(a).cuda() for a in (k, v, q))
        kv.encode_decode_step(stream, kd.data_ptr(), 0, vd.data_ptr(), 0, qd.data_ptr(), out.data_ptr())
        want = oracle.decode_step(cache, k, v, q, lay)
        assert np.abs(out.cpu().numpy() - want).max() <= tol, step
    m = kv.len()
    keep = min(m, window) if window else m
    gk, gv = kv.read_rows_f32(m - keep, keep)
    assert np.array_equal(gk, cache.keys()[m - keep:]) and np.array_equal(gv, cache.values()[m - keep:])


@pytest.mark.parametrize("element,tol", [("bf16", 1e-4), ("f32", 2e-5)])
def test_batch_step_under_knobs(state, knobs, element, tol):
    dims = (16, 2, 256)
    q_dim, kv_dim = dims[0] * dims[2], dims[1] * dims[2]
    rng = np.random.default_rng(11)
    seqs = [_layer(state, element, dims, n, 0, n + 16, rng) for n in (31, 900, 16)]
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
            assert np.abs(o.cpu().numpy() - want).max() <= tol
    for kv, cache, lay in seqs:
        gk, gv = kv.read_rows_f32()
        assert np.array_equal(gk, cache.keys()) and np.array_equal(gv, cache.values())


@pytest.mark.parametrize("element,tol", [("bf16", 1e-4), ("f32", 2e-5)])
@pytest.mark.parametrize("dims,start,chunk", [((16, 2, 256), 700, 90), ((32, 8, 128), 0, 130), ((6, 1, 40), 50, 5)])
def test_prefill_chunk_under_knobs(state, knobs, element, tol, dims, start, chunk):
    rng = np.random.default_rng(start + chunk)
    kv, cache, lay = _layer(state, element, dims, start, 0, start + chunk, rng)
    q_dim, kv_dim = dims[0] * dims[2], dims[1] * dims[2]
    q = rng.standard_normal((chunk, q_dim), dtype=np.float32)
    k = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    v = rng.standard_normal((chunk, kv_dim), dtype=np.float32)
    got = kv.prefill_rows(q, k, v)
    want = oracle.cached_attention_prefill_rows(q, k, v, cache, lay)
    assert np.abs(got - want).max() <= tol
    gk, gv = kv.read_rows_f32()
    assert np.array_equal(gk, cache.keys()) and np.array_equal(gv, cache.values())
