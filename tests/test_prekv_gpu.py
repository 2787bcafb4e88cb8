"""The step before the cache on the device: per-head RMSNorm + rotation at the token's
position (rms_norm_rope_decode, src/decode_resident/tests.rs:1867-1930) and the fused
norm + rotation + query scale + append + attention step (encode_resident_full_layer,
src/decode_resident/layers.rs:214-288), against the oracle's rms_norm_rope_heads_at +
LayerKvCache::append + cached_attention_one."""
import os

import numpy as np
import pytest

import oracle
import saragossa_amd as skv
from conftest import pseudo

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def test_rms_norm_rope_decode_matches_cpu(state):
    # src/decode_resident/tests.rs:1871-1930 (bound there: 1e-5; here the rows are identical)
    heads, head_dim, position, eps, theta = 2, 8, 5, 1.0e-6, 10000.0
    x = (np.arange(heads * head_dim, dtype=np.float32) % 11.0 - 5.0) * np.float32(0.1)
    w = np.float32(0.5) + np.arange(head_dim, dtype=np.float32) * np.float32(0.1)
    for rope_dims in (8, 4):
        got = state.rms_norm_rope_decode(x, w, heads, head_dim, rope_dims, position, eps, theta)
        want = oracle.rms_norm_rope_heads_at(x, heads, head_dim, rope_dims, w, eps, theta, position)[0]
        assert np.abs(got - want).max() <= 1e-5
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("heads,head_dim,rope_dims,theta,position,style,scale,freq", [
    (16, 256, 64, 1.0e7, 32768, 0, 1.0, 0),      # partial rotary, config 2's shape
    (32, 128, 128, 1.0e6, 2303, 0, 1.0, 0),      # Qwen3-4B
    (8, 256, 256, 1.0e6, 65535, 0, 0.125, 0),    # scaled positions
    (4, 16, 4, 1.0e6, 9, 0, 1.0, 16),            # frequency_dim != rope_dims
    (3, 40, 20, 10000.0, 77, 1, 1.0, 0),         # interleaved pairs, head_dim not a power of two
    (2, 512, 512, 10000.0, 1000, 0, 1.0, 0),
])
def test_rms_norm_rope_decode_is_bit_exact_on_random_rows(state, heads, head_dim, rope_dims, theta,
                                                          position, style, scale, freq):
    rng = np.random.default_rng(heads * head_dim + position)
    x = rng.standard_normal(heads * head_dim, dtype=np.float32) * 2
    w = (0.5 + rng.random(head_dim, dtype=np.float32)).astype(np.float32)
    got = state.rms_norm_rope_decode(x, w, heads, head_dim, rope_dims, position, 1e-6, theta,
                                     position_scale=scale, frequency_dim=freq, style=style)
    want = oracle.rms_norm_rope_heads_at(x, heads, head_dim, rope_dims, w, 1e-6, theta, position,
                                         style=style, position_scale=scale,
                                         frequency_dim=freq or None)[0]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # rotation only (apply_rope_heads_at, src/decoder/attention_ops.rs:779-834)
    got = state.rms_norm_rope_decode(x, None, heads, head_dim, rope_dims, position, 1e-6, theta,
                                     position_scale=scale, frequency_dim=freq, style=style)
    want = oracle.apply_rope_heads_at(x, heads, head_dim, rope_dims, theta, position, style=style,
                                      position_scale=scale, frequency_dim=freq or None)[0]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("heads,head_dim,rope_dims,theta,offset,rows,style", [
    (32, 128, 128, 1.0e6, 1536, 512, 0),   # a prefill chunk of config 1's q rows
    (2, 256, 64, 1.0e7, 32760, 20, 0),     # partial rotary across a page boundary
    (3, 40, 20, 10000.0, 0, 7, 0),
    (16, 256, 256, 1.0e6, 0, 130, 0),      # config 2's q rows: eight (row, head) pairs per workgroup
    (1, 512, 512, 10000.0, 5, 9, 0),       # one head: every pair of a workgroup is another row
    (5, 64, 32, 10000.0, 100, 33, 1),      # interleaved pairs, four pairs per pass of the workgroup
    (8, 128, 128, 1.0e6, 11, 3, 0),        # under four rows: one workgroup per (row, head)
])
def test_rms_norm_rope_rows_is_bit_exact(state, heads, head_dim, rope_dims, theta, offset, rows, style):
    """A chunk of rows at consecutive positions == rms_norm_rope_heads_at on a [seq, dim] tensor
    with position_offset (src/decoder/attention_ops.rs:682-777)."""
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, heads * head_dim), dtype=np.float32) * 2
    w = (0.5 + rng.random(head_dim, dtype=np.float32)).astype(np.float32)
    rope = state.rope_table(offset + rows, rope_dims, theta, style=style)
    xd, wd = _dev(x), _dev(w)
    out = torch.empty_like(xd)
    state.encode_rms_norm_rope_rows(_stream(), rope, offset, xd.data_ptr(), wd.data_ptr(), rows, heads,
                                    head_dim, 1e-6, out.data_ptr())
    want = oracle.rms_norm_rope_heads_at(x, heads, head_dim, rope_dims, w, 1e-6, theta, offset,
                                         style=oracle.ROPE_INTERLEAVED if style else oracle.ROPE_HALVES)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
    with pytest.raises(skv.DimensionError):   # the last row's position is outside the table
        state.encode_rms_norm_rope_rows(_stream(), rope, offset + 1, xd.data_ptr(), wd.data_ptr(), rows,
                                        heads, head_dim, 1e-6, out.data_ptr())
    rope.close()


def test_rms_norm_rope_decode_errors(state):
    x, w = np.zeros(16, np.float32), np.ones(8, np.float32)
    with pytest.raises(skv.DimensionError):
        state.rms_norm_rope_decode(x, w, 2, 8, 6 + 1, 0, 1e-6, 1e4)    # odd rope_dims
    with pytest.raises(skv.DimensionError):
        state.rms_norm_rope_decode(x, w, 2, 8, 10, 0, 1e-6, 1e4)       # rope_dims > head_dim
    with pytest.raises(skv.DimensionError):
        state.rms_norm_rope_decode(x, w, 3, 8, 8, 0, 1e-6, 1e4)        # wrong row length
    with pytest.raises(skv.DimensionError):
        state.rms_norm_rope_decode(x, np.ones(4, np.float32), 2, 8, 8, 0, 1e-6, 1e4)
    with pytest.raises(skv.ConfigError):
        state.rope_table(1 << 29, 128, 1e4)      # a table no host vector should be asked for


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


CASES = [
    # dims, window, start, steps, rope_dims, theta, attn_scalar (None = head_dim), norms (q, k)
    ((16, 2, 256), 0, 700, 40, 64, 1.0e7, None, (True, True)),    # config 2: partial rotary, split-K
    ((32, 8, 128), 0, 5, 40, 128, 1.0e6, None, (True, True)),     # Qwen3-4B, short cache
    ((16, 8, 256), 64, 10, 150, 256, 1.0e6, 200.0, (True, True)), # ring layer, attn_scalar != head_dim
    ((4, 2, 16), 0, 3, 30, 4, 1.0e6, None, (True, True)),         # the reference's Gemma case: rope_dims = head_dim / 4
    ((8, 2, 64), 0, 0, 50, 64, 10000.0, 1.0, (False, False)),     # rotation only, from an empty cache
    ((6, 2, 96), 0, 20, 20, 32, 10000.0, None, (True, False)),    # q norm only, padded head_dim
    ((8, 2, 512), 0, 300, 12, 128, 1.0e6, None, (True, True)),    # head_dim 512: two row elements per thread
    ((16, 8, 512), 48, 10, 100, 512, 1.0e6, 300.0, (True, True)), # head_dim 512 on a ring layer, full rotation
    ((8, 2, 384), 0, 4100, 8, 96, 1.0e6, None, (True, False)),    # head_dim 384 padded to 512, split-K
]


def run_prekv(state, dims, window, start, steps, rope_dims, theta, attn_scalar, norms, element="bf16"):
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    eps = 1.0e-6
    rng = np.random.default_rng(start * 7 + steps)
    cap = start + steps
    make = state.full_attention_f32 if element == "f32" else state.full_attention_bf16
    kv = make(cap, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, attn_scalar=attn_scalar, sliding_window=window)
    cache = oracle.LayerKvCache("f32" if element == "f32" else "bf16r")
    q_norm = (0.7 + np.abs(pseudo(np.arange(head_dim) * 11))).astype(np.float32)
    k_norm = (0.8 + np.abs(pseudo(np.arange(head_dim) * 17))).astype(np.float32)

    def cpu_pre(x, heads, w, position):
        if w is None:
            return oracle.apply_rope_heads_at(x, heads, head_dim, rope_dims, theta, position)[0]
        return oracle.rms_norm_rope_heads_at(x, heads, head_dim, rope_dims, w, eps, theta, position)[0]

    qw, kw = (q_norm if norms[0] else None), (k_norm if norms[1] else None)
    if start:
        k0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        v0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        k0 = np.stack([cpu_pre(k0[r], kv_heads, kw, r) for r in range(start)])
        kv.seed(k0, v0, start)
        cache.append_batch(k0, v0, lay)
    rope = state.rope_table(cap, rope_dims, theta)
    # raw q | k | v of a token sit in one buffer, like the fused QKV projection's output
    # Without norms and with attn_scalar 1 the scores are raw dot products: keep them at a
    # magnitude a model produces (the device splits q into two bf16 terms, 2^-17 relative, so
    # scores of +-70 would cap the agreement near 2e-4, still far inside the 1e-2 bar).
    raw = rng.standard_normal((steps, q_dim + 2 * kv_dim), dtype=np.float32) * (1.5 if norms[0] else 0.4)
    rd = _dev(raw)
    qwd = _dev(q_norm) if norms[0] else None
    kwd = _dev(k_norm) if norms[1] else None
    out = torch.empty(steps, q_dim, device="cuda", dtype=torch.float32)
    for t in range(steps):
        kv.encode_decode_step_prekv(
            _stream(), rope, start + t, rd[t].data_ptr(), 0, rd[t].data_ptr(), q_dim * 4,
            rd[t].data_ptr(), (q_dim + kv_dim) * 4, qwd.data_ptr() if norms[0] else None,
            kwd.data_ptr() if norms[1] else None, eps, float(attn_scalar or head_dim),
            out[t].data_ptr())
    got = out.cpu().numpy()
    worst = 0.0
    for t in range(steps):
        pos = start + t
        q_cpu = cpu_pre(raw[t, :q_dim], q_heads, qw, pos)
        k_cpu = cpu_pre(raw[t, q_dim:q_dim + kv_dim], kv_heads, kw, pos)
        want = oracle.decode_step(cache, k_cpu, raw[t, q_dim + kv_dim:], q_cpu, lay)
        worst = max(worst, float(np.abs(got[t] - want).max()))
    assert worst <= 1e-4, worst
    assert kv.len() == len(cache) == cap
    # the appended k rows are the CPU path's rows bit for bit (and so are the v rows)
    first = 0 if window == 0 else max(0, cap - (window + 15) // 16 * 16)
    gk, gv = kv.read_rows_f32(first, cap - first)
    assert np.array_equal(gk, cache.keys()[first:]) and np.array_equal(gv, cache.values()[first:])
    with pytest.raises(skv.DimensionError):   # full
        kv.encode_decode_step_prekv(_stream(), rope, 0, rd.data_ptr(), 0, rd.data_ptr(), 0,
                                    rd.data_ptr(), 0, None, None, eps, float(head_dim),
                                    out.data_ptr())
    rope.close()
    return kv


@pytest.mark.parametrize("dims,window,start,steps,rope_dims,theta,attn_scalar,norms", CASES)
def test_fused_prekv_steps_match_oracle(state, dims, window, start, steps, rope_dims, theta,
                                        attn_scalar, norms):
    run_prekv(state, dims, window, start, steps, rope_dims, theta, attn_scalar, norms)


@pytest.mark.parametrize("dims,window,start,steps,rope_dims,theta,attn_scalar,norms",
                         [CASES[0], CASES[2], CASES[5]])
def test_prekv_steps_as_separate_launches(state, env_flags, dims, window, start, steps, rope_dims,
                                          theta, attn_scalar, norms):
    """RETI_RUST_FLASH_SDPA=0: the same entry point runs norm + rotation, append and the plain
    attention kernel as separate launches, with the same results."""
    env_flags(RETI_RUST_FLASH_SDPA="0")
    run_prekv(state, dims, window, start, steps, rope_dims, theta, attn_scalar, norms)


def test_prekv_errors(state):
    kv = state.full_attention_bf16(8, 4, 2, 16)
    rope = state.rope_table(4, 8, 10000.0)
    wide = state.rope_table(4, 32, 10000.0)
    buf = torch.zeros(4 * 16 * 3, device="cuda", dtype=torch.float32)
    p = buf.data_ptr()

    def step(r, position, attn_scalar=16.0, off=0):
        kv.encode_decode_step_prekv(_stream(), r, position, p, off, p, 0, p, 0, None, None, 1e-6,
                                    attn_scalar, p)

    with pytest.raises(skv.DimensionError):
        step(rope, 4)                 # position outside the table
    with pytest.raises(skv.DimensionError):
        step(wide, 0)                 # rope_dims > head_dim
    with pytest.raises(skv.ConfigError):
        step(rope, 0, attn_scalar=0.0)   # src/decode_resident/layers.rs:16-20
    with pytest.raises(skv.ConfigError):
        step(rope, 0, attn_scalar=float("nan"))
    with pytest.raises(skv.DimensionError):
        step(rope, 0, off=2)          # byte offset not a multiple of 4
    assert kv.len() == 0
    step(rope, 0)
    step(None, 1)                     # no rotation at all
    assert kv.len() == 2


# ---- output gate -------------------------------------------------------------------------

def test_attn_gate_matches_cpu(state):
    """encode_attn_gate (attn_gate_f32) against context * sigmoid_scalar(gate); the gate may sit
    interleaved with q in the gated projection."""
    heads, hd = 16, 256
    rng = np.random.default_rng(3)
    ctx = rng.standard_normal(heads * hd, dtype=np.float32)
    qg = rng.standard_normal(heads * 2 * hd, dtype=np.float32) * 4
    _, gate = oracle.split_attention_gate(qg, heads, hd)
    want = oracle.attention_gate(ctx, gate[0])
    cd, gd = _dev(ctx), _dev(qg)
    out = torch.empty(heads * hd, device="cuda", dtype=torch.float32)
    state.encode_attn_gate(_stream(), cd.data_ptr(), gd.data_ptr() + hd * 4, 2 * hd, heads, hd,
                           out.data_ptr())
    assert np.abs(out.cpu().numpy() - want).max() <= 1e-6
    # contiguous gate, in place
    g2 = _dev(gate[0])
    state.encode_attn_gate(_stream(), cd.data_ptr(), g2.data_ptr(), 0, heads, hd, cd.data_ptr())
    assert np.abs(cd.cpu().numpy() - want).max() <= 1e-6


GATED = [
    ((16, 2, 256), 0, 700, 30, 64, 1.0e7),    # config 2's full-attention layers (gated, partial rotary), split-K
    ((16, 2, 256), 0, 3, 30, 64, 1.0e7),      # short cache: the split kernel applies the gate itself
    ((8, 4, 64), 32, 5, 80, 64, 10000.0),     # ring layer
    ((6, 2, 96), 0, 40, 10, 48, 10000.0),     # padded head_dim
    ((4, 2, 512), 0, 100, 8, 128, 1.0e6),     # head_dim 512
    ((16, 8, 512), 0, 2100, 6, 128, 1.0e6),   # head_dim 512, split-K with the gate in the merge
]


def run_gated(state, dims, window, start, steps, rope_dims, theta, element="bf16"):
    q_heads, kv_heads, head_dim = dims
    kv_dim, q_dim = kv_heads * head_dim, q_heads * head_dim
    eps = 1.0e-6
    rng = np.random.default_rng(start * 5 + steps)
    cap = start + steps
    make = state.full_attention_f32 if element == "f32" else state.full_attention_bf16
    kv = make(cap, q_heads, kv_heads, head_dim, window=window)
    kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
    lay = oracle.layout(q_heads, kv_heads, head_dim, sliding_window=window)
    cache = oracle.LayerKvCache("f32" if element == "f32" else "bf16r")
    q_norm = (0.7 + np.abs(pseudo(np.arange(head_dim) * 11))).astype(np.float32)
    k_norm = (0.8 + np.abs(pseudo(np.arange(head_dim) * 17))).astype(np.float32)
    if start:
        k0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        v0 = rng.standard_normal((start, kv_dim), dtype=np.float32)
        kv.seed(k0, v0, start)
        cache.append_batch(k0, v0, lay)
    rope = state.rope_table(cap, rope_dims, theta)
    # gated q projection | k | v, as the fused projection leaves them
    raw = rng.standard_normal((steps, 2 * q_dim + 2 * kv_dim), dtype=np.float32) * 1.5
    rd, qwd, kwd = _dev(raw), _dev(q_norm), _dev(k_norm)
    out = torch.empty(steps, q_dim, device="cuda", dtype=torch.float32)
    for t in range(steps):
        kv.encode_decode_step_gated(
            _stream(), rope, start + t, rd[t].data_ptr(), 0, rd[t].data_ptr(), 2 * q_dim * 4,
            rd[t].data_ptr(), (2 * q_dim + kv_dim) * 4, qwd.data_ptr(), kwd.data_ptr(), eps,
            float(head_dim), out[t].data_ptr())
    got = out.cpu().numpy()
    worst = 0.0
    for t in range(steps):
        pos = start + t
        q_raw, gate = oracle.split_attention_gate(raw[t, :2 * q_dim], q_heads, head_dim)
        q_cpu = oracle.rms_norm_rope_heads_at(q_raw[0], q_heads, head_dim, rope_dims, q_norm, eps, theta, pos)[0]
        k_cpu = oracle.rms_norm_rope_heads_at(raw[t, 2 * q_dim:2 * q_dim + kv_dim], kv_heads, head_dim,
                                              rope_dims, k_norm, eps, theta, pos)[0]
        ctx = oracle.decode_step(cache, k_cpu, raw[t, 2 * q_dim + kv_dim:], q_cpu, lay)
        want = oracle.attention_gate(ctx, gate[0])
        worst = max(worst, float(np.abs(got[t] - want).max()))
    assert worst <= 1e-4, worst
    first = 0 if window == 0 else max(0, cap - (window + 15) // 16 * 16)
    gk, gv = kv.read_rows_f32(first, cap - first)
    assert np.array_equal(gk, cache.keys()[first:]) and np.array_equal(gv, cache.values()[first:])
    rope.close()


@pytest.mark.parametrize("dims,window,start,steps,rope_dims,theta", GATED)
def test_gated_steps_match_oracle(state, dims, window, start, steps, rope_dims, theta):
    """The Qwen3.5/3.6 full-attention block from the gated q projection to the o projection's
    input: split, norms, rotation, append, attention, sigmoid gate."""
    run_gated(state, dims, window, start, steps, rope_dims, theta)


@pytest.mark.parametrize("dims,window,start,steps,rope_dims,theta", [GATED[0], GATED[2]])
def test_gated_steps_as_separate_launches(state, env_flags, dims, window, start, steps, rope_dims,
                                          theta):
    env_flags(RETI_RUST_FLASH_SDPA="0")
    run_gated(state, dims, window, start, steps, rope_dims, theta)
