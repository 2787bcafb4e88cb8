"""ctypes loader for libsaragossa_kv.so. Fails loudly when the library is missing."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libsaragossa_kv.so")

OK, ERR_DIMENSION, ERR_CONFIG, ERR_DEVICE, ERR_MEMORY = 0, 1, 2, 3, 4
DTYPE_F32, DTYPE_BF16 = 0, 1
PAGE_ROWS = 16


class KvError(RuntimeError):
    """InferError of the reference (src/error.rs:12-75)."""

    code = -1


class DimensionError(KvError):
    code = ERR_DIMENSION


class ConfigError(KvError):
    code = ERR_CONFIG


class DeviceError(KvError):
    code = ERR_DEVICE


class MemoryGuardError(KvError):
    """InferError::MemoryGuard (src/error.rs:66-68)."""

    code = ERR_MEMORY


_BY_CODE = {ERR_DIMENSION: DimensionError, ERR_CONFIG: ConfigError, ERR_DEVICE: DeviceError,
            ERR_MEMORY: MemoryGuardError}

_lib = None

_vp, _sz, _i32, _f32p = C.c_void_p, C.c_size_t, C.c_int32, C.POINTER(C.c_float)

# name -> (restype, argtypes); every symbol include/saragossa_kv.h declares
SIGNATURES = {
    "skv_last_error": (C.c_char_p, []),
    "skv_abi_version": (_i32, []),
    "skv_env_flag": (_i32, [C.c_char_p, _i32]),
    "skv_env_flag_value": (_i32, [C.c_char_p]),
    "skv_flag_kv_bf16_for": (_i32, [_i32]),
    "skv_flag_flash_sdpa_enabled": (_i32, []),
    "skv_flag_sdpa_2pass_enabled": (_i32, []),
    "skv_flag_sdpa_2pass_min_len": (_sz, []),
    "skv_sdpa_2pass_blocks": (_sz, [_sz]),
    "skv_effective_split_min_len": (_sz, []),
    "skv_flag_kv_bf16_sim_konly": (_i32, []),
    "skv_flag_kv_bf16_sim_vonly": (_i32, []),
    "skv_flag_attention_par_threshold": (_sz, []),
    "skv_flag_decode_pipeline": (_i32, []),
    "skv_resident_kv_bytes": (_i32, [_sz, _vp, _sz, _sz, C.POINTER(C.c_uint64)]),
    "skv_memory_projection": (_i32, [C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64,
                                     C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "skv_layer_bytes": (_i32, [_sz, _sz, _sz, _sz, _i32, _sz, C.POINTER(C.c_uint64)]),
    "skv_layer_bytes_ring": (_i32, [_sz, _sz, _sz, _sz, _i32, _sz, _sz, C.POINTER(C.c_uint64)]),
    "skv_check_allocation": (_i32, [_vp, C.c_uint64, C.c_uint64, C.c_uint64, C.POINTER(C.c_uint64),
                                    C.POINTER(C.c_uint64)]),
    "skv_decode_step_static_device": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp]),
    "skv_flag_decode_resident_full": (_i32, []),
    "skv_flag_decode_resident": (_i32, []),
    "skv_flag_serve_prefix_cache_enabled": (_i32, []),
    "skv_flag_serve_prefix_block_tokens": (_sz, []),
    "skv_flag_serve_prefix_cache_blocks": (_sz, []),
    "skv_flag_serve_prefix_blocks_per_session": (_sz, []),
    "skv_flag_prefix_cache_enabled": (_i32, []),
    "skv_flag_prefix_cache_capacity": (_sz, []),
    "skv_flag_prefill_chunk": (_sz, []),
    "skv_flag_memory_guard_enabled": (_i32, []),
    "skv_flag_serve_oom_guard_enabled": (_i32, []),
    "skv_flag_memory_static_cap_bytes": (C.c_uint64, []),
    "skv_flag_memory_headroom_bytes": (C.c_uint64, []),
    "skv_flag_serve_memory_static_cap_bytes": (C.c_uint64, []),
    "skv_flag_serve_memory_headroom_bytes": (C.c_uint64, []),
    "skv_flags_reload": (None, []),
    "skv_window_start": (_sz, [_sz, _sz]),
    "skv_resident_capacity": (_i32, [_sz, _sz, _sz, C.POINTER(_sz)]),
    "skv_probe_read_pages_device": (_i32, [_vp, _vp]),
    "skv_probe_read_store_pages_device": (_i32, [_vp, _vp]),
    "skv_probe_merge_device": (_i32, [_vp, _vp, _vp]),
    "skv_probe_empty_launch_device": (_i32, [_vp, _vp]),
    "skv_f32_to_bf16_bits": (C.c_uint16, [C.c_float]),
    "skv_ctx_create": (_i32, [_i32, C.POINTER(_vp)]),
    "skv_ctx_destroy": (None, [_vp]),
    "skv_ctx_synchronize": (_i32, [_vp]),
    "skv_layer_create": (_i32, [_vp, _sz, _sz, _sz, _sz, _i32, _sz, C.POINTER(_vp)]),
    "skv_layer_create_ring": (_i32, [_vp, _sz, _sz, _sz, _sz, _i32, _sz, _sz, C.POINTER(_vp)]),
    "skv_layer_create_for": (_i32, [_vp, _sz, _sz, _sz, _sz, _i32, C.POINTER(_vp)]),
    "skv_layer_destroy": (None, [_vp]),
    "skv_layer_set_block_table": (_i32, [_vp, _vp, _sz]),
    "skv_layer_pages": (_sz, [_vp]),
    "skv_kv_dim": (_sz, [_vp]),
    "skv_len": (_sz, [_vp]),
    "skv_capacity": (_sz, [_vp]),
    "skv_q_heads": (_sz, [_vp]),
    "skv_kv_heads": (_sz, [_vp]),
    "skv_head_dim": (_sz, [_vp]),
    "skv_window": (_sz, [_vp]),
    "skv_logical_byte_len": (_sz, [_vp]),
    "skv_truncate": (_i32, [_vp, _sz]),
    "skv_seed": (_i32, [_vp, _vp, _vp, _sz, _sz]),
    "skv_append_host": (_i32, [_vp, _vp, _vp, _sz]),
    "skv_append_device": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz]),
    "skv_append_batch_device": (_i32, [_vp, _vp, _vp, _vp, _sz]),
    "skv_attention_host": (_i32, [_vp, _vp, _sz, _sz, _vp]),
    "skv_attention_device": (_i32, [_vp, _vp, _vp, _vp, _sz]),
    "skv_decode_step_device": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp]),
    "skv_prefill_chunk_device": (_i32, [_vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "skv_prefill_chunk_host": (_i32, [_vp, _vp, _vp, _vp, _sz, _vp]),
    "skv_rope_rotations_host": (_i32, [_sz, _sz, _sz, C.c_float, C.c_float, _vp]),
    "skv_rope_create": (_i32, [_vp, _sz, _sz, _sz, C.c_float, C.c_float, _i32, C.POINTER(_vp)]),
    "skv_rope_destroy": (None, [_vp]),
    "skv_rms_norm_rope_decode_device": (_i32, [_vp, _vp, _vp, _sz, _vp, _vp, _sz, _sz, C.c_float, _vp]),
    "skv_rms_norm_rope_rows_device": (_i32, [_vp, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _sz, C.c_float, _vp]),
    "skv_rms_norm_rope_decode_host": (_i32, [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, C.c_float,
                                             C.c_float, C.c_float, _i32, _vp]),
    "skv_decode_step_prekv_device": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _vp,
                                            C.c_float, C.c_float, _vp]),
    "skv_decode_step_gated_device": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _vp,
                                            C.c_float, C.c_float, _vp]),
    "skv_attn_gate_device": (_i32, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "skv_decode_step_batch_device": (_i32, [_vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "skv_decode_step_layers_device": (_i32, [_vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "skv_read_rows": (_i32, [_vp, _sz, _sz, _vp, _vp]),
    "skv_read_rows_f32": (_i32, [_vp, _sz, _sz, _vp, _vp]),
    "skv_gather_device": (_i32, [_vp, _vp, _sz, _sz, _vp, _vp]),
    "skv_snapshot_blocks": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, C.POINTER(_vp)]),
    "skv_snapshot_clone": (_i32, [_vp, _vp, _vp, C.POINTER(_vp)]),
    "skv_restore_blocks": (_i32, [_vp, _vp, _vp, _vp, _sz, _vp, _sz]),
    "skv_snapshot_bytes": (_sz, [_vp]),
    "skv_snapshot_free": (None, [_vp]),
    "skv_state_snapshot": (_i32, [_vp, _vp, _vp, _vp, _sz, C.POINTER(_vp)]),
    "skv_state_restore": (_i32, [_vp, _vp, _vp, _vp, _vp, _sz]),
    "skv_hash_root": (None, [_vp]),
    "skv_hash_for_session": (None, [C.c_char_p, _sz, _vp]),
    "skv_hash_chain": (None, [_vp, _vp, _sz, _vp]),
    "skv_prefix_create": (_i32, [_sz, _sz, _sz, C.POINTER(_vp)]),
    "skv_prefix_from_runtime_flags": (_i32, [C.POINTER(_vp)]),
    "skv_prefix_destroy": (None, [_vp]),
    "skv_prefix_block_tokens": (_sz, [_vp]),
    "skv_prefix_capacity": (_sz, [_vp]),
    "skv_prefix_len": (_sz, [_vp]),
    "skv_prefix_bytes": (_sz, [_vp]),
    "skv_prefix_session_block_count": (_sz, [_vp, _vp]),
    "skv_prefix_match": (_i32, [_vp, _vp, _vp, _sz, C.POINTER(_i32), _vp, _vp, _sz]),
    "skv_prefix_insert": (_i32, [_vp, _vp, _vp, _sz, C.c_uint64, _sz, _vp, _sz,
                                 C.POINTER(_sz), C.POINTER(_sz)]),
    "skv_prefix_evict_lru": (_i32, [_vp, C.POINTER(_i32), C.POINTER(C.c_uint64), C.POINTER(_sz)]),
    "skv_prefix_entry": (_i32, [_vp, _sz, _vp, _vp, C.POINTER(_sz), C.POINTER(C.c_uint64),
                                C.POINTER(_sz)]),
    "skv_hot_create": (_i32, [_vp, _sz, _sz, _sz, _sz, _vp, _sz, C.POINTER(_vp)]),
    "skv_hot_destroy": (None, [_vp]),
    "skv_hot_remember": (_i32, [_vp, _vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _sz,
                                C.POINTER(_i32)]),
    "skv_hot_remember_range": (_i32, [_vp, _vp, _vp, _vp, _sz, _sz, _vp, _sz, C.POINTER(_sz)]),
    "skv_hot_match_restore": (_i32, [_vp, _vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _sz,
                                     C.POINTER(_sz), _vp]),
    "skv_hot_evict_lru": (_i32, [_vp, C.POINTER(_i32), C.POINTER(_sz)]),
    "skv_hot_block_tokens": (_sz, [_vp]),
    "skv_hot_len": (_sz, [_vp]),
    "skv_hot_bytes": (_sz, [_vp]),
    "skv_hot_free_blocks": (_sz, [_vp]),
    "skv_hot_pool_blocks": (_sz, [_vp]),
    "skv_hot_block_bytes": (_sz, [_vp]),
    "skv_hot_evictions": (C.c_uint64, [_vp]),
    "skv_hot_skipped": (C.c_uint64, [_vp]),
    "skv_hot_entry": (_i32, [_vp, _sz, _vp, _vp, C.POINTER(_sz), C.POINTER(_sz)]),
    "skv_prompt_cache_create": (_i32, [_vp, _sz, C.POINTER(_vp)]),
    "skv_prompt_cache_from_runtime_flags": (_i32, [_vp, C.POINTER(_vp)]),
    "skv_prompt_cache_destroy": (None, [_vp]),
    "skv_prompt_cache_len": (_sz, [_vp]),
    "skv_prompt_cache_capacity": (_sz, [_vp]),
    "skv_prompt_cache_bytes": (_sz, [_vp]),
    "skv_prompt_cache_entry": (_i32, [_vp, _sz, C.POINTER(_sz), _vp, _sz]),
    "skv_prompt_cache_put": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _sz]),
    "skv_prompt_cache_get": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _sz, C.POINTER(_sz)]),
}


def lib_path() -> str:
    return _LIB


def lib():
    """The loaded library. Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise DeviceError(
                f"{_LIB} is missing: build it with `python -c 'import __graft_entry__ as g; "
                "g.build()'` (hipcc, gfx950). The KV path has no CPU fallback.")
        l = C.CDLL(_LIB)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc: int) -> None:
    if rc != OK:
        msg = lib().skv_last_error().decode("utf-8", "replace")
        raise _BY_CODE.get(rc, KvError)(msg)
