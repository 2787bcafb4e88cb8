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


def f32_to_bf16_bits(value: float) -> int:
    return lib().skv_f32_to_bf16_bits(value)
