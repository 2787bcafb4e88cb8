"""CPU oracle for the KV-cache hot path (TEST INFRASTRUCTURE ONLY).

ctypes binding over ``libskv_oracle.so`` (built from ``skv_oracle.c`` by the
Makefile beside it) plus the pure-Python prefix-cache restatement in
``oracle.prefix_cache``. Only tests, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package; the product
package ``saragossa_amd`` never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libskv_oracle.so")

OK, ERR_DIMENSION, ERR_CONFIG = 0, 1, 2
ROPE_HALVES, ROPE_INTERLEAVED = 0, 1


class OracleError(Exception):
    """Mirrors InferError::{Dimension, Config} of the reference (src/error.rs:12-75)."""

    def __init__(self, code: int, what: str):
        super().__init__(f"{'Dimension' if code == ERR_DIMENSION else 'Config'}: {what}")
        self.code = code


def build() -> None:
    """Compile the oracle (always recompiles)."""
    subprocess.run(["make", "-B", "-C", _HERE], check=True, capture_output=True)


class Layout(C.Structure):
    """AttentionLayout (src/decoder/attention_ops.rs:526-585); sliding_window 0 == None."""

    _fields_ = [
        ("num_attention_heads", C.c_size_t),
        ("num_key_value_heads", C.c_size_t),
        ("head_dim", C.c_size_t),
        ("rope_dims", C.c_size_t),
        ("attn_scalar", C.c_float),
        ("sliding_window", C.c_size_t),
    ]


def layout(q_heads, kv_heads, head_dim, attn_scalar=None, sliding_window=0, rope_dims=None):
    return Layout(q_heads, kv_heads, head_dim, rope_dims or head_dim,
                  float(head_dim if attn_scalar is None else attn_scalar), sliding_window)


_lib = None
_f32p = C.POINTER(C.c_float)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        l = C.CDLL(_LIB_PATH)
        l.skvo_f32_to_bf16_bits.restype = C.c_uint16
        l.skvo_f32_to_bf16_bits.argtypes = [C.c_float]
        l.skvo_bf16_round.restype = C.c_float
        l.skvo_bf16_round.argtypes = [C.c_float]
        l.skvo_bf16_round_array.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        l.skvo_f32_to_bf16_bits_array.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        l.skvo_cache_new.restype = C.c_void_p
        l.skvo_cache_free.argtypes = [C.c_void_p]
        l.skvo_cache_clone.restype = C.c_void_p
        l.skvo_cache_clone.argtypes = [C.c_void_p]
        l.skvo_cache_set_bf16_round.argtypes = [C.c_void_p, C.c_int, C.c_int]
        for name in ("skvo_cache_append", "skvo_cache_append_batch"):
            fn = getattr(l, name)
            fn.restype = C.c_int
            fn.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t,
                           C.c_size_t, C.c_size_t, C.c_size_t]
        l.skvo_cache_len.restype = C.c_size_t
        l.skvo_cache_len.argtypes = [C.c_void_p]
        l.skvo_cache_truncate.restype = C.c_int
        l.skvo_cache_truncate.argtypes = [C.c_void_p, C.c_size_t]
        l.skvo_cache_keys.restype = _f32p
        l.skvo_cache_keys.argtypes = [C.c_void_p]
        l.skvo_cache_values.restype = _f32p
        l.skvo_cache_values.argtypes = [C.c_void_p]
        l.skvo_cache_kv_dim.restype = C.c_size_t
        l.skvo_cache_kv_dim.argtypes = [C.c_void_p]
        l.skvo_cache_has_kv_dim.restype = C.c_int
        l.skvo_cache_has_kv_dim.argtypes = [C.c_void_p]
        l.skvo_cache_estimated_bytes.restype = C.c_size_t
        l.skvo_cache_estimated_bytes.argtypes = [C.c_void_p]
        l.skvo_attention_layout.restype = C.c_int
        l.skvo_attention_layout.argtypes = [C.c_size_t] * 6 + [C.c_int, C.c_size_t, C.c_int,
                                                                C.c_float, C.c_int, C.c_size_t,
                                                                C.POINTER(Layout)]
        l.skvo_set_attention_parallel_threshold.argtypes = [C.c_size_t]
        l.skvo_attention_parallel_threshold.restype = C.c_size_t
        l.skvo_dot_product.restype = C.c_float
        l.skvo_dot_product.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        l.skvo_softmax_in_place.argtypes = [C.c_void_p, C.c_size_t, C.c_float]
        l.skvo_softmax.argtypes = [C.c_void_p, C.c_size_t, C.c_float, C.c_void_p]
        l.skvo_cached_attention_one.restype = C.c_int
        l.skvo_cached_attention_one.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p,
                                                C.POINTER(Layout), C.c_void_p, C.c_int]
        l.skvo_cached_attention_prefill_rows.restype = C.c_int
        l.skvo_cached_attention_prefill_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p,
                                                         C.c_size_t, C.c_size_t, C.c_size_t,
                                                         C.c_size_t, C.c_void_p, C.POINTER(Layout),
                                                         C.c_void_p, C.c_int]
        l.skvo_causal_attention.restype = C.c_int
        l.skvo_causal_attention.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                            C.c_size_t, C.c_size_t, C.c_size_t, C.POINTER(Layout),
                                            C.c_void_p]
        l.skvo_rms_norm_rope_heads_at.restype = C.c_int
        l.skvo_rms_norm_rope_heads_at.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t,
                                                  C.c_size_t, C.c_void_p, C.c_float, C.c_float,
                                                  C.c_float, C.c_size_t, C.c_size_t, C.c_int,
                                                  C.c_void_p]
        l.skvo_apply_rope_heads_at.restype = C.c_int
        l.skvo_apply_rope_heads_at.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t,
                                               C.c_size_t, C.c_float, C.c_float, C.c_size_t,
                                               C.c_size_t, C.c_int, C.c_void_p]
        l.skvo_sdpa_2pass_blocks.restype = C.c_size_t
        l.skvo_sdpa_2pass_blocks.argtypes = [C.c_size_t]
        l.skvo_split_attention_gate.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t,
                                                C.c_size_t, C.c_void_p, C.c_void_p]
        l.skvo_attention_gate.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        l.skvo_attention_gate.restype = None
        l.skvo_sigmoid.restype = C.c_float
        l.skvo_sigmoid.argtypes = [C.c_float]
        l.skvo_window_start.restype = C.c_size_t
        l.skvo_window_start.argtypes = [C.c_size_t, C.c_size_t]
        l.skvo_resident_capacity.restype = C.c_int
        l.skvo_resident_capacity.argtypes = [C.c_size_t, C.c_size_t, C.c_size_t,
                                             C.POINTER(C.c_size_t)]
        l.skvo_decode_step.restype = C.c_int
        l.skvo_decode_step.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.POINTER(Layout), C.c_void_p, C.c_int]
        _lib = l
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _check(rc: int, what: str) -> None:
    if rc != OK:
        raise OracleError(rc, what)


def f32_to_bf16_bits(x) -> np.ndarray:
    a = _f32(x).reshape(-1)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().skvo_f32_to_bf16_bits_array(_ptr(a), _ptr(out), a.size)
    return out.reshape(np.shape(x))


def bf16_round(x) -> np.ndarray:
    a = _f32(x)
    out = np.empty_like(a)
    lib().skvo_bf16_round_array(_ptr(a), _ptr(out), a.size)
    return out


def default_threads(q_heads: int) -> int:
    """min(q_heads, host cores): the reference goes parallel per query head only."""
    return max(1, min(q_heads, os.cpu_count() or 1))


class LayerKvCache:
    """LayerKvCache of the reference (src/decoder.rs:671-697), KV part.

    ``mode='f32'`` is the CPU path as it is; ``mode='bf16r'`` rounds every K/V
    element to bf16 when it is appended, which is the reference's own convention
    for comparing against a bf16 device cache (src/decode_resident/tests.rs:1462-1472).
    """

    def __init__(self, mode: str = "f32", _handle=None):
        self._l = lib()
        self.mode = mode
        self._h = _handle if _handle is not None else self._l.skvo_cache_new()
        if _handle is None:
            r = 1 if mode == "bf16r" else 0
            self._l.skvo_cache_set_bf16_round(self._h, r, r)

    def __del__(self):
        if getattr(self, "_h", None):
            self._l.skvo_cache_free(self._h)
            self._h = None

    def clone(self) -> "LayerKvCache":
        return LayerKvCache(self.mode, _handle=self._l.skvo_cache_clone(self._h))

    def append(self, key, value, lay: Layout) -> None:
        k, v = _f32(key), _f32(value)
        k2, v2 = np.atleast_2d(k), np.atleast_2d(v)
        _check(self._l.skvo_cache_append(self._h, _ptr(k), k2.shape[0], k2.shape[1], _ptr(v),
                                         v2.shape[0], v2.shape[1], lay.num_key_value_heads,
                                         lay.head_dim), "cache KV append")

    def append_batch(self, key, value, lay: Layout) -> None:
        k, v = _f32(key), _f32(value)
        k2, v2 = np.atleast_2d(k), np.atleast_2d(v)
        _check(self._l.skvo_cache_append_batch(self._h, _ptr(k), k2.shape[0], k2.shape[1], _ptr(v),
                                               v2.shape[0], v2.shape[1], lay.num_key_value_heads,
                                               lay.head_dim), "cache KV append_batch")

    def __len__(self) -> int:
        return self._l.skvo_cache_len(self._h)

    def truncate(self, n: int) -> None:
        _check(self._l.skvo_cache_truncate(self._h, n), f"truncate KV CPU {n}")

    @property
    def kv_dim(self):
        return self._l.skvo_cache_kv_dim(self._h) if self._l.skvo_cache_has_kv_dim(self._h) else None

    def estimated_bytes(self) -> int:
        return self._l.skvo_cache_estimated_bytes(self._h)

    def _rows(self, ptr) -> np.ndarray:
        n, d = len(self), self.kv_dim or 0
        if n == 0:
            return np.zeros((0, d), dtype=np.float32)
        return np.ctypeslib.as_array(ptr, shape=(n, d)).copy()

    def keys(self) -> np.ndarray:
        return self._rows(self._l.skvo_cache_keys(self._h))

    def values(self) -> np.ndarray:
        return self._rows(self._l.skvo_cache_values(self._h))


def cached_attention_one(q, cache: LayerKvCache, lay: Layout, threads: int | None = None):
    qa = np.atleast_2d(_f32(q))
    out = np.empty(lay.num_attention_heads * lay.head_dim, dtype=np.float32)
    t = default_threads(lay.num_attention_heads) if threads is None else threads
    _check(lib().skvo_cached_attention_one(_ptr(qa), qa.shape[0], qa.shape[1], cache._h,
                                           C.byref(lay), _ptr(out), t), "attention cache shapes")
    return out


def decode_step(cache: LayerKvCache, k_row, v_row, q, lay: Layout, threads: int | None = None):
    k, v, qa = _f32(k_row), _f32(v_row), _f32(q)
    out = np.empty(lay.num_attention_heads * lay.head_dim, dtype=np.float32)
    t = default_threads(lay.num_attention_heads) if threads is None else threads
    _check(lib().skvo_decode_step(cache._h, _ptr(k), _ptr(v), _ptr(qa), C.byref(lay), _ptr(out), t),
           "decode step")
    return out


def cached_attention_prefill_rows(q, k, v, cache: LayerKvCache, lay: Layout,
                                  threads: int | None = None):
    qa, ka, va = np.atleast_2d(_f32(q)), np.atleast_2d(_f32(k)), np.atleast_2d(_f32(v))
    if ka.shape[0] != qa.shape[0] or va.shape[0] != qa.shape[0]:
        raise OracleError(ERR_DIMENSION, "attention batch cached shapes")
    out = np.empty((qa.shape[0], lay.num_attention_heads * lay.head_dim), dtype=np.float32)
    t = default_threads(lay.num_attention_heads) if threads is None else threads
    _check(lib().skvo_cached_attention_prefill_rows(_ptr(qa), _ptr(ka), _ptr(va), qa.shape[0],
                                                    qa.shape[1], ka.shape[1], va.shape[1],
                                                    cache._h, C.byref(lay), _ptr(out), t),
           "attention batch cached shapes")
    return out


def causal_attention(q, k, v, lay: Layout):
    qa, ka, va = np.atleast_2d(_f32(q)), np.atleast_2d(_f32(k)), np.atleast_2d(_f32(v))
    if ka.shape[0] != qa.shape[0] or va.shape[0] != qa.shape[0]:
        raise OracleError(ERR_DIMENSION, "attention shapes")
    out = np.empty((qa.shape[0], lay.num_attention_heads * lay.head_dim), dtype=np.float32)
    _check(lib().skvo_causal_attention(_ptr(qa), _ptr(ka), _ptr(va), qa.shape[0], qa.shape[1],
                                       ka.shape[1], va.shape[1], C.byref(lay), _ptr(out)),
           "attention shapes")
    return out


def softmax_in_place(values, temperature: float = 1.0) -> np.ndarray:
    a = _f32(values).copy()
    lib().skvo_softmax_in_place(_ptr(a), a.size, temperature)
    return a


def softmax(values, temperature: float = 1.0) -> np.ndarray:
    a = _f32(values)
    out = np.empty_like(a)
    lib().skvo_softmax(_ptr(a), a.size, temperature, _ptr(out))
    return out


def dot_product(a, b) -> float:
    x, y = _f32(a), _f32(b)
    return float(lib().skvo_dot_product(_ptr(x), _ptr(y), x.size))


def rms_norm_rope_heads_at(x, heads, head_dim, rope_dims, weight, eps, theta, position_offset,
                           style=ROPE_HALVES, position_scale=1.0, frequency_dim=None):
    xa = np.atleast_2d(_f32(x))
    if xa.shape[1] != heads * head_dim:
        raise OracleError(ERR_DIMENSION, "RMSNorm/RoPE heads invalide")
    w = _f32(weight).reshape(-1)
    if w.size != head_dim:
        raise OracleError(ERR_DIMENSION, "RMSNorm/RoPE weight")
    out = np.empty_like(xa)
    _check(lib().skvo_rms_norm_rope_heads_at(_ptr(xa), xa.shape[0], heads, head_dim, rope_dims,
                                             _ptr(w), eps, theta, position_scale,
                                             frequency_dim or rope_dims, position_offset, style,
                                             _ptr(out)), "RMSNorm/RoPE")
    return out


def apply_rope_heads_at(x, heads, head_dim, rope_dims, theta, position_offset, style=ROPE_HALVES,
                        position_scale=1.0, frequency_dim=None):
    xa = np.atleast_2d(_f32(x))
    if xa.shape[1] != heads * head_dim:
        raise OracleError(ERR_DIMENSION, "RoPE heads")
    out = np.empty_like(xa)
    _check(lib().skvo_apply_rope_heads_at(_ptr(xa), xa.shape[0], heads, head_dim, rope_dims, theta,
                                          position_scale, frequency_dim or rope_dims,
                                          position_offset, style, _ptr(out)), "RoPE")
    return out


def split_attention_gate(q_projection, heads, head_dim):
    """split_attention_gate (src/decoder/attention_ops.rs:486-520): ([rows, q_dim] q, gate)."""
    qp = np.atleast_2d(_f32(q_projection))
    q = np.empty((qp.shape[0], heads * head_dim), np.float32)
    gate = np.empty_like(q)
    _check(lib().skvo_split_attention_gate(_ptr(qp), qp.shape[0], qp.shape[1], heads, head_dim,
                                           _ptr(q), _ptr(gate)), "q_proj gated")
    return q, gate


def attention_gate(context, gate):
    """context * sigmoid(gate) (src/decoder/attention_ops.rs:217-219, 522-524)."""
    c, g = _f32(context), _f32(gate)
    if c.shape != g.shape:
        raise OracleError(ERR_DIMENSION, "gate shape")
    out = np.empty_like(c)
    lib().skvo_attention_gate(_ptr(c), _ptr(g), c.size, _ptr(out))
    return out


def attention_layout(q_dim, k_dim, v_dim, q_heads, kv_heads, head_dim=None, rope_dims=None,
                     attn_scalar=None, sliding_window=0) -> Layout:
    out = Layout()
    _check(lib().skvo_attention_layout(q_dim, k_dim, v_dim, q_heads, kv_heads, head_dim or 0,
                                       head_dim is not None, rope_dims or 0, rope_dims is not None,
                                       attn_scalar or 0.0, attn_scalar is not None,
                                       sliding_window, C.byref(out)), "attention layout")
    return out


def sdpa_2pass_blocks(n: int) -> int:
    return lib().skvo_sdpa_2pass_blocks(n)


def window_start(position: int, window: int) -> int:
    return lib().skvo_window_start(position, window)


def resident_capacity(prefill_len: int, max_new_tokens: int, draft_headroom: int) -> int:
    out = C.c_size_t()
    _check(lib().skvo_resident_capacity(prefill_len, max_new_tokens, draft_headroom, C.byref(out)),
           "capacité KV résidente déborde")
    return out.value
