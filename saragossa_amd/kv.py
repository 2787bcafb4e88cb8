"""Host mirror of DecodeResidentState / FullAttentionMetalState over the C ABI.

Method names follow src/decode_resident/attention.rs so that the parity tests
read like src/decode_resident/tests.rs. Host entry points take numpy arrays;
device entry points take raw device pointers (e.g. ``tensor.data_ptr()``) and a
stream handle (e.g. ``torch.cuda.current_stream().cuda_stream``).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from ._lib import DTYPE_BF16, DTYPE_F32, check, lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


class DecodeResidentState:
    """DecodeResidentState::new (src/decoder/resident/setup.rs:237, 675)."""

    def __init__(self, device: int = 0):
        self._l = lib()
        h = C.c_void_p()
        check(self._l.skv_ctx_create(device, C.byref(h)))
        self._h = h

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._l.skv_ctx_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def synchronize(self) -> None:
        check(self._l.skv_ctx_synchronize(self._h))

    def full_attention_with_element(self, capacity, q_heads, kv_heads, head_dim,
                                    dtype=DTYPE_BF16, window=0, rollback_rows=None) -> "FullAttentionState":
        """rollback_rows: rows a ring layer (window > 0) keeps behind its window so that a
        speculative verify of that depth can be rolled back; None = the library's default."""
        h = C.c_void_p()
        if rollback_rows is None:
            check(self._l.skv_layer_create(self._h, capacity, q_heads, kv_heads, head_dim, dtype,
                                           window, C.byref(h)))
        else:
            check(self._l.skv_layer_create_ring(self._h, capacity, q_heads, kv_heads, head_dim, dtype,
                                                window, rollback_rows, C.byref(h)))
        return FullAttentionState(self, h)

    def full_attention(self, capacity, q_heads, kv_heads, head_dim, sampled) -> "FullAttentionState":
        """full_attention (src/decode_resident/attention.rs:26-45): dtype from the KV policy."""
        h = C.c_void_p()
        check(self._l.skv_layer_create_for(self._h, capacity, q_heads, kv_heads, head_dim,
                                           int(sampled), C.byref(h)))
        return FullAttentionState(self, h)

    def rms_norm_rope_decode(self, x, weight, heads, head_dim, rope_dims, position, eps, theta,
                             position_scale=1.0, frequency_dim=0, style=0) -> np.ndarray:
        """DecodeResidentState::rms_norm_rope_decode (src/decode_resident/tests.rs:1168-1172);
        weight None = rotation only."""
        xa = _f32(x).reshape(-1)
        out = np.empty_like(xa)
        w = None if weight is None else _f32(weight).reshape(-1)
        if xa.size != heads * head_dim or (w is not None and w.size != head_dim):
            from ._lib import DimensionError
            raise DimensionError("RMSNorm/RoPE heads invalide")
        check(self._l.skv_rms_norm_rope_decode_host(self._h, _p(xa), None if w is None else _p(w),
                                                    heads, head_dim, rope_dims, frequency_dim,
                                                    position, eps, theta, position_scale, style,
                                                    _p(out)))
        return out

    def encode_rms_norm_rope_rows(self, stream, rope, position_offset, x_ptr, weight_ptr, n_rows, heads,
                                  head_dim, eps, out_ptr) -> None:
        """rms_norm_rope_heads_at for n_rows rows at positions position_offset.. (device in/out)."""
        check(self._l.skv_rms_norm_rope_rows_device(
            self._h, stream, None if rope is None else rope._h, position_offset, x_ptr, weight_ptr,
            n_rows, heads, head_dim, eps, out_ptr))

    def encode_attn_gate(self, stream, ctx_ptr, gate_ptr, gate_head_stride, heads, head_dim,
                         out_ptr) -> None:
        """encode_attn_gate (attn_gate_f32, src/decode_resident/kernels.rs:949-959)."""
        check(self._l.skv_attn_gate_device(self._h, stream, ctx_ptr, gate_ptr, gate_head_stride,
                                           heads, head_dim, out_ptr))

    def check_allocation(self, requested: int, static_cap: int = 0, headroom: int = 0):
        """MemoryGuard::check_allocation (src/memory_guard.rs:365-370) against this device:
        raises MemoryGuardError when the request would pass the ceiling, else returns
        (available, projected)."""
        avail, proj = C.c_uint64(0), C.c_uint64(0)
        check(self._l.skv_check_allocation(self._h, requested, static_cap, headroom, C.byref(avail),
                                           C.byref(proj)))
        return int(avail.value), int(proj.value)

    def encode_probe_empty_launch(self, stream) -> None:
        """Measurement aid: an empty kernel with the decode launch's shape."""
        check(self._l.skv_probe_empty_launch_device(self._h, stream))

    def rope_table(self, max_positions, rope_dims, theta, position_scale=1.0, frequency_dim=0,
                   style=0) -> "RopeTable":
        return RopeTable(self, max_positions, rope_dims, theta, position_scale, frequency_dim, style)

    def full_attention_bf16(self, capacity, q_heads, kv_heads, head_dim, window=0):
        """full_attention_bf16_for_test (attention.rs:47-54)."""
        return self.full_attention_with_element(capacity, q_heads, kv_heads, head_dim,
                                                DTYPE_BF16, window)


    def full_attention_f32(self, capacity, q_heads, kv_heads, head_dim, window=0):
        """The f32 element of full_attention_with_element (attention.rs:56-108): what
        full_attention chooses for greedy decoding."""
        return self.full_attention_with_element(capacity, q_heads, kv_heads, head_dim,
                                                DTYPE_F32, window)


def rope_rotations(position, rope_dims, theta, position_scale=1.0, frequency_dim=0) -> np.ndarray:
    """rope_rotations (src/decoder/attention_ops.rs:848-887) on the host: [rope_dims/2, 2] of
    (cos, sin)."""
    out = np.empty(rope_dims, np.float32)
    check(lib().skv_rope_rotations_host(position, rope_dims, frequency_dim, theta, position_scale,
                                        _p(out)))
    return out.reshape(-1, 2)


class RopeTable:
    """Device table of the rotations of positions 0..max_positions-1 (skv_rope_create)."""

    def __init__(self, ctx, max_positions, rope_dims, theta, position_scale=1.0, frequency_dim=0,
                 style=0):
        self._ctx, self._l = ctx, ctx._l
        h = C.c_void_p()
        check(self._l.skv_rope_create(ctx._h, max_positions, rope_dims, frequency_dim, theta,
                                      position_scale, style, C.byref(h)))
        self._h = h

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._l.skv_rope_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()


class FullAttentionState:
    """FullAttentionMetalState (src/decode_resident/attention.rs:457-1038). Not clonable."""

    def __init__(self, ctx: DecodeResidentState, handle):
        self._ctx = ctx  # keeps the context alive
        self._l = ctx._l
        self._h = handle

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._l.skv_layer_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def __copy__(self):
        raise TypeError("device KV state is not clonable (src/decoder.rs:682-697)")

    __deepcopy__ = __copy__

    # ---- getters (attention.rs:485-548)
    def kv_dim(self): return self._l.skv_kv_dim(self._h)
    def len(self): return self._l.skv_len(self._h)
    def __len__(self): return self.len()
    def capacity(self): return self._l.skv_capacity(self._h)
    def q_heads(self): return self._l.skv_q_heads(self._h)
    def kv_heads(self): return self._l.skv_kv_heads(self._h)
    def head_dim(self): return self._l.skv_head_dim(self._h)
    def window(self): return self._l.skv_window(self._h)
    def pages(self): return self._l.skv_layer_pages(self._h)
    def byte_len(self): return self._l.skv_logical_byte_len(self._h)

    def set_block_table(self, table) -> None:
        t = np.ascontiguousarray(table, dtype=np.int32)
        check(self._l.skv_layer_set_block_table(self._h, _p(t), t.size))

    def truncate(self, n: int) -> None:
        check(self._l.skv_truncate(self._h, n))

    # ---- host entry points
    def seed(self, keys_rows, values_rows, n_rows: int) -> None:
        k, v = _f32(keys_rows).reshape(-1), _f32(values_rows).reshape(-1)
        expected = n_rows * self.kv_dim()
        n_elems = k.size if k.size != expected else v.size  # a wrong length reaches the check
        check(self._l.skv_seed(self._h, _p(k), _p(v), n_elems, n_rows))

    def append_row(self, key, value) -> None:
        k, v = _f32(key).reshape(-1), _f32(value).reshape(-1)
        n = k.size if k.size != self.kv_dim() else v.size  # a wrong length reaches the check
        check(self._l.skv_append_host(self._h, _p(k), _p(v), n))

    def attention_decode(self, q) -> np.ndarray:
        return self.attention_decode_windowed(q, 0)

    def attention_decode_windowed(self, q, window_start: int) -> np.ndarray:
        qa = _f32(q).reshape(-1)
        out = np.empty(self.q_heads() * self.head_dim(), dtype=np.float32)
        check(self._l.skv_attention_host(self._h, _p(qa), qa.size, window_start, _p(out)))
        return out

    def prefill_rows(self, q, k, v) -> np.ndarray:
        """cached_attention_prefill_rows (src/decoder/attention_ops.rs:976-1017): append the
        rows of k/v and attend each new row causally over the cache. Host arrays."""
        qa, ka, va = np.atleast_2d(_f32(q)), np.atleast_2d(_f32(k)), np.atleast_2d(_f32(v))
        n = qa.shape[0]
        if ka.shape != (n, self.kv_dim()) or va.shape != ka.shape or \
                qa.shape[1] != self.q_heads() * self.head_dim():
            from ._lib import DimensionError
            raise DimensionError(f"attention batch cached shapes q={qa.shape}, k={ka.shape}, v={va.shape}")
        out = np.empty_like(qa)
        check(self._l.skv_prefill_chunk_host(self._h, _p(qa), _p(ka), _p(va), n, _p(out)))
        return out

    def encode_prefill_rows(self, stream, q_ptr, k_ptr, v_ptr, n_rows, out_ptr) -> None:
        check(self._l.skv_prefill_chunk_device(self._h, stream, q_ptr, k_ptr, v_ptr, n_rows, out_ptr))

    def read_rows(self, first: int = 0, n: int | None = None):
        """Logical rows as bf16 bit patterns, ([n, kv_dim] uint16, same)."""
        n = self.len() - first if n is None else n
        k = np.empty((n, self.kv_dim()), dtype=np.uint16)
        v = np.empty((n, self.kv_dim()), dtype=np.uint16)
        check(self._l.skv_read_rows(self._h, first, n, _p(k), _p(v)))
        return k, v

    def read_rows_f32(self, first: int = 0, n: int | None = None):
        """Logical rows as f32, for either element type (bf16 rows widen exactly)."""
        n = self.len() - first if n is None else n
        k = np.empty((n, self.kv_dim()), dtype=np.float32)
        v = np.empty((n, self.kv_dim()), dtype=np.float32)
        check(self._l.skv_read_rows_f32(self._h, first, n, _p(k), _p(v)))
        return k, v

    # ---- device entry points (raw pointers + stream handle)
    def encode_append_kv(self, stream, k_ptr, v_ptr) -> None:
        self.encode_append_kv_with_offsets(stream, k_ptr, 0, v_ptr, 0)

    def encode_append_kv_with_offsets(self, stream, k_ptr, k_off, v_ptr, v_off) -> None:
        check(self._l.skv_append_device(self._h, stream, k_ptr, k_off, v_ptr, v_off))

    def encode_append_batch(self, stream, k_ptr, v_ptr, n_rows) -> None:
        check(self._l.skv_append_batch_device(self._h, stream, k_ptr, v_ptr, n_rows))

    def encode_attention_decode(self, stream, q_ptr, out_ptr) -> None:
        self.encode_attention_decode_windowed(stream, q_ptr, out_ptr, 0)

    def encode_attention_decode_windowed(self, stream, q_ptr, out_ptr, window_start) -> None:
        check(self._l.skv_attention_device(self._h, stream, q_ptr, out_ptr, window_start))

    def encode_probe_read_pages(self, stream) -> None:
        """Measurement aid: a launch that only fetches the cached K and V pages, with the
        decode kernel's grid and access pattern."""
        check(self._l.skv_probe_read_pages_device(self._h, stream))

    def encode_probe_read_store_pages(self, stream) -> None:
        """The read-only launch plus a split partial of the decode kernel's size written by every
        workgroup: the least a split-K launch must do."""
        check(self._l.skv_probe_read_store_pages_device(self._h, stream))

    def encode_probe_merge(self, stream, out_ptr) -> None:
        """Measurement aid: the merge launch of a decode step at the current length, over the
        partials the layer's last attention call left."""
        check(self._l.skv_probe_merge_device(self._h, stream, out_ptr))

    def encode_decode_step(self, stream, k_ptr, k_off, v_ptr, v_off, q_ptr, out_ptr) -> None:
        check(self._l.skv_decode_step_device(self._h, stream, k_ptr, k_off, v_ptr, v_off, q_ptr,
                                             out_ptr))

    def encode_decode_step_static(self, stream, k_ptr, k_off, v_ptr, v_off, q_ptr, out_ptr) -> None:
        """encode_decode_step for callers that cannot allocate: the split partials live in the
        library's static device array (skv_decode_step_static_device)."""
        check(self._l.skv_decode_step_static_device(self._h, stream, k_ptr, k_off, v_ptr, v_off,
                                                    q_ptr, out_ptr))

    def encode_decode_step_prekv(self, stream, rope, position, q_ptr, q_off, k_ptr, k_off, v_ptr,
                                 v_off, q_norm_ptr, k_norm_ptr, eps, attn_scalar, out_ptr) -> None:
        """The q/k norms, rotation, query scale, append and attention of
        encode_resident_full_layer (src/decode_resident/layers.rs:214-288) in one call."""
        check(self._l.skv_decode_step_prekv_device(
            self._h, stream, None if rope is None else rope._h, position, q_ptr, q_off, k_ptr,
            k_off, v_ptr, v_off, q_norm_ptr, k_norm_ptr, eps, attn_scalar, out_ptr))

    def encode_decode_step_gated(self, stream, rope, position, qg_ptr, qg_off, k_ptr, k_off, v_ptr,
                                 v_off, q_norm_ptr, k_norm_ptr, eps, attn_scalar, out_ptr) -> None:
        """encode_decode_step_prekv for a layer with an output gate: qg is the gated q
        projection (per head: q then gate) and the context comes out times sigmoid(gate)."""
        check(self._l.skv_decode_step_gated_device(
            self._h, stream, None if rope is None else rope._h, position, qg_ptr, qg_off, k_ptr,
            k_off, v_ptr, v_off, q_norm_ptr, k_norm_ptr, eps, attn_scalar, out_ptr))

    def encode_gather(self, stream, first, n, k_dst_ptr, v_dst_ptr) -> None:
        check(self._l.skv_gather_device(self._h, stream, first, n, k_dst_ptr, v_dst_ptr))


def encode_decode_step_batch(seqs, stream, k_ptrs, v_ptrs, q_ptrs, out_ptrs) -> None:
    """One decode step of the same model layer for several independent sequences in one pair
    of launches (skv_decode_step_batch_device): sequence i appends the kv_dim f32 values at
    k_ptrs[i] / v_ptrs[i], then attends q_ptrs[i] into out_ptrs[i]. Per sequence it is
    FullAttentionState.encode_decode_step (src/decode_resident/layers.rs:259-288)."""
    import ctypes as C
    n = len(seqs)
    if not (len(k_ptrs) == len(v_ptrs) == len(q_ptrs) == len(out_ptrs) == n):
        raise ValueError("one k, v, q and out pointer per sequence")
    arr = C.c_void_p * n
    l = seqs[0]._l if n else None
    if l is None:
        from ._lib import lib
        l = lib()
    check(l.skv_decode_step_batch_device(arr(*[s._h for s in seqs]), n, stream, arr(*k_ptrs),
                                         arr(*v_ptrs), arr(*q_ptrs), arr(*out_ptrs)))
