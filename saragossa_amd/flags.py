"""Runtime kill-switches of the KV path (src/runtime_flags.rs; src/decode_resident/utils.rs)."""
from ._lib import lib


def env_flag(name: str, default: bool) -> bool:
    return bool(lib().skv_env_flag(name.encode(), int(default)))


def env_flag_value(value: str):
    v = lib().skv_env_flag_value(value.encode())
    return None if v < 0 else bool(v)


def kv_bf16_for(sampled: bool) -> bool:
    return bool(lib().skv_flag_kv_bf16_for(int(sampled)))


def flash_sdpa_enabled() -> bool:
    return bool(lib().skv_flag_flash_sdpa_enabled())


def sdpa_2pass_enabled() -> bool:
    return bool(lib().skv_flag_sdpa_2pass_enabled())


def sdpa_2pass_min_len() -> int:
    return lib().skv_flag_sdpa_2pass_min_len()


def sdpa_2pass_blocks(n: int) -> int:
    return lib().skv_sdpa_2pass_blocks(n)


def effective_split_min_len() -> int:
    """Rows from which this library splits a decode launch's context (128 unless
    RETI_RUST_SDPA_2PASS_MIN_LEN is set; the reference's own default is sdpa_2pass_min_len())."""
    return lib().skv_effective_split_min_len()


def kv_bf16_sim_konly() -> bool:
    """RETI_RUST_KV_BF16_SIM_KONLY (src/decode_resident/utils.rs:245-248)."""
    return bool(lib().skv_flag_kv_bf16_sim_konly())


def kv_bf16_sim_vonly() -> bool:
    """RETI_RUST_KV_BF16_SIM_VONLY (src/decode_resident/utils.rs:253-256)."""
    return bool(lib().skv_flag_kv_bf16_sim_vonly())


def attention_parallel_threshold() -> int:
    """RETI_RUST_ATTENTION_PAR_THRESHOLD (src/runtime_flags.rs:641-649)."""
    return lib().skv_flag_attention_par_threshold()


def decode_pipeline_enabled() -> bool:
    """RETI_RUST_DECODE_PIPELINE (src/runtime_flags.rs:309-313)."""
    return bool(lib().skv_flag_decode_pipeline())


def decode_resident_full_enabled() -> bool:
    return bool(lib().skv_flag_decode_resident_full())


def decode_resident_enabled() -> bool:
    return bool(lib().skv_flag_decode_resident())


def serve_prefix_cache_enabled() -> bool:
    return bool(lib().skv_flag_serve_prefix_cache_enabled())


def serve_prefix_block_tokens() -> int:
    return lib().skv_flag_serve_prefix_block_tokens()


def serve_prefix_cache_blocks() -> int:
    return lib().skv_flag_serve_prefix_cache_blocks()


def serve_prefix_blocks_per_session() -> int:
    return lib().skv_flag_serve_prefix_blocks_per_session()


def prefix_cache_enabled() -> bool:
    return bool(lib().skv_flag_prefix_cache_enabled())


def prefix_cache_capacity() -> int:
    return lib().skv_flag_prefix_cache_capacity()


def prefill_chunk_size() -> int:
    return lib().skv_flag_prefill_chunk()


def memory_guard_enabled() -> bool:
    """memory_guard_enabled (src/runtime_flags.rs:699-702)."""
    return bool(lib().skv_flag_memory_guard_enabled())


def serve_oom_guard_enabled() -> bool:
    """serve_oom_guard_enabled (src/runtime_flags.rs:693-696)."""
    return bool(lib().skv_flag_serve_oom_guard_enabled())


def memory_static_cap_bytes():
    """memory_static_cap_bytes (src/runtime_flags.rs:705-713): None when unset, unparsable or zero."""
    return lib().skv_flag_memory_static_cap_bytes() or None


def memory_headroom_bytes() -> int:
    return lib().skv_flag_memory_headroom_bytes()


def serve_memory_static_cap_bytes():
    """serve_memory_static_cap_bytes (src/runtime_flags.rs:773-781)."""
    return lib().skv_flag_serve_memory_static_cap_bytes() or None


def serve_memory_headroom_bytes() -> int:
    return lib().skv_flag_serve_memory_headroom_bytes()


def reload() -> None:
    """Re-read the environment (the reference freezes flags at first read). Tests only."""
    lib().skv_flags_reload()


def window_start(position: int, window: int) -> int:
    return lib().skv_window_start(position, window)


def resident_capacity(prefill_len: int, max_new_tokens: int, draft_headroom: int = 0):
    """prefill + max_new + headroom, or None when the sum overflows
    (src/decoder/resident/setup.rs:322-329)."""
    import ctypes
    out = ctypes.c_size_t(0)
    ok = lib().skv_resident_capacity(prefill_len, max_new_tokens, draft_headroom, ctypes.byref(out))
    return int(out.value) if ok else None


def resident_kv_bytes(capacity: int, kv_dims, elem_bytes: int = 4):
    """Sum of 2 * capacity * kv_dim * elem_bytes over the layers, or None when a product
    overflows (check_resident_full_decode_allocation, src/decoder/resident/setup.rs:897-917)."""
    import ctypes
    dims = (ctypes.c_size_t * len(kv_dims))(*kv_dims)
    out = ctypes.c_uint64(0)
    ok = lib().skv_resident_kv_bytes(capacity, dims, len(kv_dims), elem_bytes, ctypes.byref(out))
    return int(out.value) if ok else None


def memory_projection(current: int, reserved: int, requested: int, limit: int):
    """(over_limit, projected, available) of MemoryGuard::projection_with_reserved
    (src/memory_guard.rs:334-362)."""
    import ctypes
    proj, avail = ctypes.c_uint64(0), ctypes.c_uint64(0)
    over = lib().skv_memory_projection(current, reserved, requested, limit, ctypes.byref(proj),
                                       ctypes.byref(avail))
    return bool(over), int(proj.value), int(avail.value)


def layer_bytes(capacity, q_heads, kv_heads, head_dim, dtype, window=0, rollback_rows=None) -> int:
    """Device bytes a layer with these arguments takes (skv_layer_bytes, skv_layer_bytes_ring)."""
    import ctypes
    from ._lib import check
    out = ctypes.c_uint64(0)
    if rollback_rows is None:
        check(lib().skv_layer_bytes(capacity, q_heads, kv_heads, head_dim, dtype, window, ctypes.byref(out)))
    else:
        check(lib().skv_layer_bytes_ring(capacity, q_heads, kv_heads, head_dim, dtype, window, rollback_rows,
                                         ctypes.byref(out)))
    return int(out.value)


def f32_to_bf16_bits(value: float) -> int:
    return lib().skv_f32_to_bf16_bits(value)
