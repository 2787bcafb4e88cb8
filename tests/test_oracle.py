"""Pins the CPU oracle (oracle/skv_oracle.c) against the reference's own known answers,
closed forms and independent implementations, so that a plausible restatement mistake
(a dropped term, a wrong index or sign, a transposed operand) fails here. No GPU."""
import math

import numpy as np
import pytest

import oracle
from conftest import pseudo


# ---- bf16 rounding ---------------------------------------------------------------------
def test_bf16_known_answers_from_reference():
    # src/decoder/tests.rs:13-25
    got = oracle.bf16_round(np.array([1.0039062, -0.33325195, 42.125], dtype=np.float32))
    assert got.tolist() == [1.0, np.float32(-0.33398438), 42.0]


def test_bf16_matches_torch_for_finite_values():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10,
                        rng.uniform(-1e-3, 1e-3, 5000).astype(np.float32),
                        np.array([0.0, -0.0, 1.0, 65504.0, 1e38, -1e38, 1e-38], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_bits(x), want)


def test_bf16_ties_to_even_carry_and_nan_non_special_case():
    def f(bits):
        return np.array([bits], dtype=np.uint32).view(np.float32)
    b = lambda bits: int(oracle.f32_to_bf16_bits(f(bits))[0])
    assert b(0x3F808000) == 0x3F80          # tie, even mantissa stays
    assert b(0x3F818000) == 0x3F82          # tie, odd mantissa rounds up
    assert b(0x3F808001) == 0x3F81          # just above the tie
    assert b(0x3FFFFFFF) == 0x4000          # carry into the exponent
    assert b(0x7F7FFFFF) == 0x7F80          # max finite rounds to +inf
    assert b(0x7F800000) == 0x7F80          # inf stays
    assert b(0x7FC00000) == 0x7FC0          # quiet NaN
    assert b(0xFFFFFFFF) == 0x0000          # the wrapping add has no NaN special case
    assert b(0x7FFFFFFF) == 0x8000
    assert b(0x80000000) == 0x8000          # -0.0


# ---- LayerKvCache ----------------------------------------------------------------------
def test_cache_append_len_truncate_and_errors():
    # src/decoder/attention_cache.rs:7-100
    lay = oracle.layout(4, 2, 2)
    c = oracle.LayerKvCache()
    assert len(c) == 0 and c.kv_dim is None
    c.truncate(0)                                   # no kv_dim yet: only 0 is allowed
    with pytest.raises(oracle.OracleError):
        c.truncate(1)
    c.append([[1, 2, 3, 4]], [[5, 6, 7, 8]], lay)
    c.append([[10, 20, 30, 40]], [[50, 60, 70, 80]], lay)
    assert len(c) == 2 and c.kv_dim == 4
    assert c.keys().tolist() == [[1, 2, 3, 4], [10, 20, 30, 40]]
    assert c.values().tolist() == [[5, 6, 7, 8], [50, 60, 70, 80]]
    with pytest.raises(oracle.OracleError):
        c.append([[1, 2, 3]], [[1, 2, 3, 4]], lay)          # wrong key dim
    with pytest.raises(oracle.OracleError):
        c.append([[1, 2, 3, 4], [1, 2, 3, 4]], [[1, 2, 3, 4], [1, 2, 3, 4]], lay)  # 2 rows
    with pytest.raises(oracle.OracleError):
        c.append(np.zeros((1, 8)), np.zeros((1, 8)), oracle.layout(4, 2, 4))    # kv_dim latched
    with pytest.raises(oracle.OracleError):
        c.append_batch(np.zeros((0, 4)), np.zeros((0, 4)), lay)                # seq == 0
    c.append_batch(np.ones((3, 4)), np.ones((3, 4)) * 2, lay)
    assert len(c) == 5
    with pytest.raises(oracle.OracleError):
        c.truncate(6)
    c.truncate(2)
    assert c.keys().tolist() == [[1, 2, 3, 4], [10, 20, 30, 40]]
    assert c.estimated_bytes() == 2 * 2 * 4 * 4


def test_cache_clone_is_deep():
    lay = oracle.layout(2, 1, 2)
    c = oracle.LayerKvCache()
    c.append([[1, 2]], [[3, 4]], lay)
    d = c.clone()
    c.append([[5, 6]], [[7, 8]], lay)
    assert len(d) == 1 and len(c) == 2 and d.keys().tolist() == [[1, 2]]


def test_cache_bf16r_mode_rounds_on_append():
    lay = oracle.layout(1, 1, 4)
    c = oracle.LayerKvCache("bf16r")
    k = np.array([[1.0039062, -0.33325195, 42.125, 0.1]], dtype=np.float32)
    c.append(k, k * 2, lay)
    assert np.array_equal(c.keys(), oracle.bf16_round(k))
    assert np.array_equal(c.values(), oracle.bf16_round(k * 2))


# ---- softmax ---------------------------------------------------------------------------
def test_softmax_closed_forms():
    assert oracle.softmax_in_place([3.5]).tolist() == [1.0]
    two = oracle.softmax_in_place([0.0, 0.0])
    assert two.tolist() == [0.5, 0.5]
    p = oracle.softmax_in_place([1.0, 0.0])
    assert abs(p[0] - 1.0 / (1.0 + math.exp(-1.0))) < 1e-7 and abs(p.sum() - 1.0) < 1e-7
    # temperature floor 1e-4 and the uniform fallback when the sum underflows cannot trigger
    # for finite inputs (the max contributes exp(0) = 1); -inf everywhere gives NaN like Rust
    assert np.allclose(oracle.softmax_in_place([1.0, 2.0], 0.0), [0.0, 1.0])
    assert np.array_equal(oracle.softmax([1.0, 2.0, 3.0]), oracle.softmax_in_place([1.0, 2.0, 3.0]))


def test_dot_product_is_sequential():
    # 1e8 + 1 - 1e8 in order gives 0 in f32; a pairwise or reversed sum would give 1
    a = np.array([1e8, 1.0, -1e8], dtype=np.float32)
    assert oracle.dot_product(a, np.ones(3, np.float32)) == 0.0
    assert oracle.dot_product(a[[0, 2, 1]], np.ones(3, np.float32)) == 1.0


# ---- cached_attention_one --------------------------------------------------------------
def _row(x):
    return np.array([x], dtype=np.float32)


def test_attention_scale_uses_query_pre_attn_scalar():
    # src/decoder/tests.rs:966-996
    lay = oracle.layout(1, 1, 2, attn_scalar=8.0)
    c = oracle.LayerKvCache()
    c.append(_row([1.0, 0.0]), _row([1.0, 0.0]), lay)
    c.append(_row([0.0, 0.0]), _row([0.0, 1.0]), lay)
    out = oracle.cached_attention_one(_row([1.0, 0.0]), c, lay)
    p0 = 1.0 / (1.0 + math.exp(-1.0 / math.sqrt(8.0)))
    assert np.allclose(out, [p0, 1.0 - p0], atol=1e-6)


def test_cached_attention_sliding_window_matches_truncated_cache():
    # src/decoder/tests.rs:911-964
    full = oracle.layout(1, 1, 2, attn_scalar=2.0)
    win = oracle.layout(1, 1, 2, attn_scalar=2.0, sliding_window=3)
    keys = [[0.5, 0.0], [1.0, 0.5], [0.25, 1.0], [0.0, 0.75], [0.75, 0.25]]
    values = [[1.0, 2.0], [3.0, 4.0], [5.0, 6.0], [7.0, 8.0], [9.0, 10.0]]
    wc, tc = oracle.LayerKvCache(), oracle.LayerKvCache()
    for k, v in zip(keys, values):
        wc.append(_row(k), _row(v), win)
    for k, v in list(zip(keys, values))[2:]:
        tc.append(_row(k), _row(v), full)
    q = _row([1.0, 0.25])
    a = oracle.cached_attention_one(q, wc, win)
    b = oracle.cached_attention_one(q, tc, full)
    assert np.array_equal(a, b)
    assert not np.allclose(a, oracle.cached_attention_one(q, wc, full), atol=1e-3)


def test_single_key_returns_value_row_exactly():
    # src/decode_resident/tests.rs:1356-1385: softmax of one score is exactly 1
    q_heads, kv_heads, hd = 4, 2, 16
    lay = oracle.layout(q_heads, kv_heads, hd)
    c = oracle.LayerKvCache()
    k = pseudo(60_000 + np.arange(kv_heads * hd))
    v = pseudo(70_000 + np.arange(kv_heads * hd))
    c.append(k[None], v[None], lay)
    out = oracle.cached_attention_one(pseudo(50_000 + np.arange(q_heads * hd))[None], c, lay)
    want = np.repeat(v.reshape(kv_heads, hd), q_heads // kv_heads, axis=0).reshape(-1)
    assert np.array_equal(out, want)


def _attention_f64(q, k, v, q_heads, kv_heads, hd, scale, start=0):
    q = q.astype(np.float64).reshape(q_heads, hd)
    k = k.astype(np.float64)[start:].reshape(-1, kv_heads, hd)
    v = v.astype(np.float64)[start:].reshape(-1, kv_heads, hd)
    g = q_heads // kv_heads
    out = np.empty((q_heads, hd))
    for h in range(q_heads):
        s = k[:, h // g, :] @ q[h] * scale
        p = np.exp(s - s.max())
        p /= p.sum()
        out[h] = p @ v[:, h // g, :]
    return out.reshape(-1)


@pytest.mark.parametrize("dims,n,window", [((16, 2, 256), 300, 0), ((32, 8, 128), 700, 0),
                                           ((6, 3, 40), 130, 50), ((4, 4, 8), 5, 0)])
def test_attention_against_fp64_textbook_and_torch(dims, n, window):
    """GQA head mapping (h // group), scale 1/sqrt(attn_scalar), K-vs-V operand order and the
    window start are all pinned by an independent fp64 computation and by torch's SDPA."""
    q_heads, kv_heads, hd = dims
    rng = np.random.default_rng(n)
    k = rng.standard_normal((n, kv_heads * hd), dtype=np.float32)
    v = rng.standard_normal((n, kv_heads * hd), dtype=np.float32)
    q = rng.standard_normal(q_heads * hd, dtype=np.float32)
    lay = oracle.layout(q_heads, kv_heads, hd, sliding_window=window)
    c = oracle.LayerKvCache()
    c.append_batch(k, v, lay)
    got_par = oracle.cached_attention_one(q, c, lay, threads=4)
    got_ser = oracle.cached_attention_one(q, c, lay, threads=1)
    assert np.array_equal(got_par, got_ser)      # the per-head worker pool cannot change results
    start = max(n - window, 0) if window else 0
    want = _attention_f64(q, k, v, q_heads, kv_heads, hd, 1.0 / math.sqrt(hd), start)
    assert np.abs(got_par - want).max() < 2e-5
    torch = pytest.importorskip("torch")
    tq = torch.from_numpy(q).reshape(1, q_heads, 1, hd)
    tk = torch.from_numpy(k[start:]).reshape(1, -1, kv_heads, hd).transpose(1, 2)
    tv = torch.from_numpy(v[start:]).reshape(1, -1, kv_heads, hd).transpose(1, 2)
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, enable_gqa=True)
    assert np.abs(got_par - ref.reshape(-1).numpy()).max() < 2e-5


def test_attention_errors():
    lay = oracle.layout(4, 2, 4)
    c = oracle.LayerKvCache()
    with pytest.raises(oracle.OracleError):
        oracle.cached_attention_one(np.zeros(16), c, lay)        # no kv_dim / empty
    c.append(np.zeros((1, 8)), np.zeros((1, 8)), lay)
    with pytest.raises(oracle.OracleError):
        oracle.cached_attention_one(np.zeros(15), c, lay)
    with pytest.raises(oracle.OracleError):
        oracle.cached_attention_one(np.zeros((2, 16)), c, lay)   # seq != 1


# ---- prefill paths ---------------------------------------------------------------------
def test_prefill_rows_equals_append_then_attention_and_causal_attention():
    """cached_attention_prefill_rows is append + cached_attention_one per row
    (src/decoder/attention_ops.rs:1003-1014); causal_attention from position 0 agrees with it
    to rounding (it divides by sqrt where the cached path multiplies by the reciprocal)."""
    q_heads, kv_heads, hd, seq = 4, 2, 8, 9
    rng = np.random.default_rng(3)
    q = rng.standard_normal((seq, q_heads * hd), dtype=np.float32)
    k = rng.standard_normal((seq, kv_heads * hd), dtype=np.float32)
    v = rng.standard_normal((seq, kv_heads * hd), dtype=np.float32)
    for window in (0, 4):
        lay = oracle.layout(q_heads, kv_heads, hd, sliding_window=window)
        c = oracle.LayerKvCache()
        rows = oracle.cached_attention_prefill_rows(q, k, v, c, lay)
        c2 = oracle.LayerKvCache()
        for r in range(seq):
            c2.append(k[r][None], v[r][None], lay)
            assert np.array_equal(rows[r], oracle.cached_attention_one(q[r], c2, lay))
        causal = oracle.causal_attention(q, k, v, lay)
        assert np.abs(causal - rows).max() < 1e-6
        for r in range(seq):
            s = max(r + 1 - window, 0) if window else 0
            want = _attention_f64(q[r], k[:r + 1], v[:r + 1], q_heads, kv_heads, hd,
                                  1 / math.sqrt(hd), s)
            assert np.abs(causal[r] - want).max() < 1e-5
    # chunked == tokenwise for chunk sizes 1, 2, 3, 5 (src/decoder/tests.rs:376-404)
    lay = oracle.layout(q_heads, kv_heads, hd)
    whole = oracle.cached_attention_prefill_rows(q, k, v, oracle.LayerKvCache(), lay)
    for chunk in (1, 2, 3, 5):
        c = oracle.LayerKvCache()
        parts = [oracle.cached_attention_prefill_rows(q[i:i + chunk], k[i:i + chunk],
                                                      v[i:i + chunk], c, lay)
                 for i in range(0, seq, chunk)]
        assert np.array_equal(np.vstack(parts), whole)


# ---- RoPE + RMSNorm ----------------------------------------------------------------------
def _golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                           "reference_known_answers.json")) as f:
        return json.load(f)


def test_golden_known_answers_of_the_reference():
    """tests/golden/reference_known_answers.json: every known answer the reference's tests
    hold for this path, as data."""
    g = _golden()
    for case in g["bf16_round"]["cases"]:
        assert oracle.bf16_round(np.float32(case["input"]))[()] == np.float32(case["expected"])
    styles = {"halves": oracle.ROPE_HALVES, "interleaved": oracle.ROPE_INTERLEAVED}
    for case in g["apply_rope"]["cases"]:
        got = oracle.apply_rope_heads_at([case["x"]], case["heads"], case["head_dim"], case["rope_dims"],
                                         case["theta"], case["position"], styles[case["style"]],
                                         position_scale=case["position_scale"],
                                         frequency_dim=case["frequency_dim"])
        assert np.allclose(got[0], case["expected"], atol=g["apply_rope"]["tolerance"]), case
    t = g["two_key_attention"]
    lay = oracle.layout(1, 1, 2, attn_scalar=t["attn_scalar"])
    c = oracle.LayerKvCache()
    for k, v in zip(t["keys"], t["values"]):
        c.append([k], [v], lay)
    out = oracle.cached_attention_one(t["query"], c, lay)
    p0 = 1.0 / (1.0 + math.exp(-1.0 / math.sqrt(8.0)))
    assert np.abs(out - [p0, 1 - p0]).max() <= t["tolerance"]
    import hashlib
    from oracle import prefix_cache as pc
    for case in g["sha256"]["cases"]:
        assert hashlib.sha256(case["message_utf8"].encode()).hexdigest() == case["digest_hex"]
    assert pc.hash_for_session("abc").hex() == g["sha256"]["cases"][0]["digest_hex"]


def test_apply_rope_styles_match_mlx_reference():
    # src/decoder/tests.rs:998-1023: constants captured from mx.fast.rope
    x = [[1.0, 2.0, 3.0, 4.0]]
    inter = oracle.apply_rope_heads_at(x, 1, 4, 4, 10000.0, 1, oracle.ROPE_INTERLEAVED)
    assert np.allclose(inter, [[-1.14264, 1.92208, 2.95985, 4.0298]], atol=1e-4)
    halves = oracle.apply_rope_heads_at(x, 1, 4, 4, 10000.0, 1, oracle.ROPE_HALVES)
    assert np.allclose(halves, [[-1.98411, 1.9599, 2.46238, 4.0198]], atol=1e-4)


def test_apply_rope_halves_partial_rotates_inside_rope_dims():
    # src/decoder/tests.rs:1025-1045
    x = [[1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0]]
    out = oracle.apply_rope_heads_at(x, 1, 8, 4, 10000.0, 1, oracle.ROPE_HALVES, frequency_dim=4)
    assert np.allclose(out, [[-1.98411, 1.9599, 2.46238, 4.0198, 5, 6, 7, 8]], atol=1e-4)


def test_apply_rope_position_scale_matches_mlx_reference():
    # src/decoder/tests.rs:1047-1085
    x = [[1.0, 2.0, 3.0, 4.0]]
    h = oracle.apply_rope_heads_at(x, 1, 4, 4, 1e6, 5, oracle.ROPE_HALVES, position_scale=0.125)
    assert np.allclose(h, [[-0.944329, 1.9975, 3.017987, 4.001249]], atol=1e-4)
    i = oracle.apply_rope_heads_at(x, 1, 4, 4, 1e6, 5, oracle.ROPE_INTERLEAVED, position_scale=0.125)
    assert np.allclose(i, [[-0.359231, 2.207024, 2.9975, 4.001874]], atol=1e-4)
    s = oracle.apply_rope_heads_at(x, 1, 4, 4, 1e4, 3, oracle.ROPE_HALVES, position_scale=0.125)
    assert np.allclose(s, [[-0.168310, 1.984986, 3.157795, 4.007472]], atol=1e-4)


def test_fused_rms_rope_matches_two_step_and_hand_formula():
    # src/decoder/tests.rs:1087-1113, 1158-1182
    x = np.array([[0.5, -1.0, 2.0, 0.25], [-0.75, 1.5, -2.0, 0.125]], dtype=np.float32)
    w = np.array([1.5, 0.5, 1.0, 2.0], dtype=np.float32)
    for scale in (1.0, 0.125):
        for style in (oracle.ROPE_INTERLEAVED, oracle.ROPE_HALVES):
            fused = oracle.rms_norm_rope_heads_at(x, 1, 4, 4, w, 1e-6, 10000.0, 3, style,
                                                  position_scale=scale)
            normed = x / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
            two = oracle.apply_rope_heads_at(normed.astype(np.float32), 1, 4, 4, 10000.0, 3, style,
                                             position_scale=scale)
            assert np.allclose(fused, two, atol=1e-6)
    # per-head normalisation: two heads are normalised separately
    x2 = np.array([[3.0, 4.0, 0.0, 0.0, 1.0, 1.0, 1.0, 1.0]], dtype=np.float32)
    out = oracle.rms_norm_rope_heads_at(x2, 2, 4, 4, np.ones(4), 0.0, 10000.0, 0)
    assert np.allclose(out[0, :4], np.array([3, 4, 0, 0]) / math.sqrt(25 / 4), atol=1e-6)
    assert np.allclose(out[0, 4:], 1.0, atol=1e-6)
    with pytest.raises(oracle.OracleError):
        oracle.rms_norm_rope_heads_at(x2, 2, 4, 3, np.ones(4), 0.0, 10000.0, 0)   # odd rope_dims


def test_rms_norm_eps_sits_under_the_square_root():
    # inv_rms = 1 / sqrt(mean_square + eps) (src/decoder/attention_ops.rs:748). With eps = 0.5 the
    # places it could wrongly sit differ in the first digit: head (3, 4, 0, 0) has mean square
    # 6.25, so 1/sqrt(6.75) = 0.38490 against 1/(sqrt(6.25) + 0.5) = 0.33333, 1/sqrt(6.25) + 0.5
    # = 0.9 and 1/sqrt(6.25) = 0.4. Position 0: the rotation is the identity.
    x = np.array([[3.0, 4.0, 0.0, 0.0, 1.0, -1.0, 1.0, -1.0]], dtype=np.float32)
    w = np.array([1.0, 2.0, 1.0, 1.0], dtype=np.float32)
    out = oracle.rms_norm_rope_heads_at(x, 2, 4, 4, w, 0.5, 10000.0, 0)
    inv0, inv1 = 1.0 / math.sqrt(6.25 + 0.5), 1.0 / math.sqrt(1.0 + 0.5)
    assert np.allclose(out[0, :4], [3 * inv0, 4 * inv0 * 2, 0, 0], atol=1e-6)
    assert np.allclose(out[0, 4:], [inv1, -2 * inv1, inv1, -inv1], atol=1e-6)
    assert abs(out[0, 0] - 3 / (math.sqrt(6.25) + 0.5)) > 0.1   # not eps outside the root


# ---- integer policy ----------------------------------------------------------------------
def test_sdpa_2pass_blocks_and_window_start_and_capacity():
    # src/decode_resident/utils.rs:282-286: 32 blocks at 4096, 64 at 8193, 256 at 32768/33000
    assert [oracle.sdpa_2pass_blocks(n) for n in (1, 2048, 4096, 8193, 32768, 33000, 10**7)] == \
        [32, 32, 32, 64, 256, 288, 1024]
    # src/decoder/resident/types.rs:13-18
    assert oracle.window_start(0, 4) == 0 and oracle.window_start(3, 4) == 0
    assert oracle.window_start(4, 4) == 1 and oracle.window_start(100, 0) == 0
    assert oracle.resident_capacity(2048, 256, 4) == 2308
    with pytest.raises(oracle.OracleError):
        oracle.resident_capacity(2**64 - 1, 1, 0)


def test_attention_layout_rules():
    # src/decoder/attention_ops.rs:526-585
    lay = oracle.attention_layout(4096, 512, 512, 16, 2)
    assert (lay.head_dim, lay.rope_dims, lay.attn_scalar, lay.sliding_window) == (256, 256, 256.0, 0)
    lay = oracle.attention_layout(4096, 512, 512, 16, 2, head_dim=256, rope_dims=64, attn_scalar=8.0,
                                  sliding_window=1024)
    assert (lay.rope_dims, lay.attn_scalar, lay.sliding_window) == (64, 8.0, 1024)
    for bad in [dict(q_heads=3, kv_heads=2), dict(q_heads=0, kv_heads=2), dict(k_dim=500),
                dict(rope_dims=3), dict(rope_dims=512), dict(q_dim=4000)]:
        args = dict(q_dim=4096, k_dim=512, v_dim=512, q_heads=16, kv_heads=2)
        args.update(bad)
        with pytest.raises(oracle.OracleError):
            oracle.attention_layout(**args)


def test_output_gate_split_and_sigmoid():
    """split_attention_gate + sigmoid gate (src/decoder/attention_ops.rs:486-524, 217-219)."""
    heads, hd, rows = 3, 4, 2
    qp = np.arange(rows * heads * 2 * hd, dtype=np.float32).reshape(rows, -1)
    q, gate = oracle.split_attention_gate(qp, heads, hd)
    r = qp.reshape(rows, heads, 2, hd)
    assert np.array_equal(q, r[:, :, 0].reshape(rows, -1))
    assert np.array_equal(gate, r[:, :, 1].reshape(rows, -1))
    with pytest.raises(oracle.OracleError):
        oracle.split_attention_gate(qp[:, :-1], heads, hd)
    ctx = np.float32([2.0, -3.0, 0.5, 1.0, 7.0])
    g = np.float32([0.0, 0.0, 30.0, -30.0, -200.0])
    out = oracle.attention_gate(ctx, g)
    assert out[0] == 1.0 and out[1] == -1.5             # sigmoid(0) is exactly 1/2
    assert out[2] == 0.5                                # saturates to 1
    assert 0.0 < out[3] < 1e-12 and out[4] == 0.0       # exp overflows to inf: 1/inf == 0
    x = np.linspace(-20, 20, 4001).astype(np.float32)
    one = np.ones_like(x)
    s_pos, s_neg = oracle.attention_gate(one, x), oracle.attention_gate(one, -x)
    assert np.abs(s_pos + s_neg - 1.0).max() <= 2e-7
    want = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    assert np.abs(s_pos - want).max() <= 1.2e-7         # within an ulp or so of the fp64 value
