"""rope_rotations on the host side of the library (skv_rope_rotations_host) against the
oracle's restatement of src/decoder/attention_ops.rs:848-887: the same f32 operations and
the same libm, so the tables must agree bit for bit. No GPU needed."""
import numpy as np
import pytest

import oracle
import saragossa_amd as skv


def oracle_rotations(position, rope_dims, theta, scale, frequency_dim):
    """(cos, sin) per pair read off the oracle by rotating unit vectors: with x = e_pair the
    rotated head holds cos at `pair` and sin at `pair + pairs` (halves style)."""
    pairs = rope_dims // 2
    out = np.empty((pairs, 2), np.float32)
    x = np.zeros((pairs, rope_dims), np.float32)
    x[np.arange(pairs), np.arange(pairs)] = 1.0
    # one call: `pairs` heads, each a different unit vector
    y = oracle.apply_rope_heads_at(x.reshape(1, -1), pairs, rope_dims, rope_dims, theta, position,
                                   position_scale=scale, frequency_dim=frequency_dim)
    y = y.reshape(pairs, rope_dims)
    out[:, 0] = y[np.arange(pairs), np.arange(pairs)]
    out[:, 1] = y[np.arange(pairs), np.arange(pairs) + pairs]
    return out


@pytest.mark.parametrize("rope_dims,theta,scale,freq", [
    (8, 10000.0, 1.0, None), (4, 10000.0, 1.0, 8), (128, 1.0e6, 1.0, None),
    (64, 1.0e7, 1.0, 256), (256, 1.0e6, 0.125, None), (32, 500000.0, 8.0, None)])
def test_rope_rotations_match_the_oracle_bit_for_bit(rope_dims, theta, scale, freq):
    for position in [0, 1, 5, 17, 1023, 4096, 32768, 65535, 1 << 20]:
        got = skv.rope_rotations(position, rope_dims, theta, scale, freq or 0)
        want = oracle_rotations(position, rope_dims, theta, scale, freq or rope_dims)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (position, rope_dims)


def test_rope_rotations_known_values():
    # position 0: no rotation; pair 0 has frequency 1: angle == position
    r = skv.rope_rotations(0, 8, 10000.0)
    assert np.array_equal(r, np.tile(np.float32([1, 0]), (4, 1)))
    r = skv.rope_rotations(5, 8, 10000.0)
    assert abs(float(r[0, 0]) - np.cos(5.0)) <= 6e-8 and abs(float(r[0, 1]) - np.sin(5.0)) <= 6e-8
    # last pair: exponent 6/8 -> angle 5 / 10000^0.75 = 0.005
    assert abs(float(r[3, 1]) - np.sin(0.005)) <= 1e-9


def test_rope_rotations_errors():
    with pytest.raises(skv.DimensionError):
        skv.rope_rotations(1, 7, 10000.0)       # odd
    with pytest.raises(skv.DimensionError):
        skv.rope_rotations(1, 0, 10000.0)
    with pytest.raises(skv.DimensionError):
        skv.rope_rotations(1, 8, 0.0)           # apply_rope_heads_at rejects theta <= 0
