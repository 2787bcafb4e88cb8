// Raw FFI binding of include/saragossa_kv.h (libsaragossa_kv.so, the gfx950 KV-cache hot path).
// Written by gen_bindings.py from the header: one declaration per C prototype, nothing else.
// No Rust toolchain exists where this file is produced: it has not been compiled there.
#![allow(non_camel_case_types)]
use std::os::raw::{c_char, c_void};

#[repr(C)] pub struct skv_ctx { _private: [u8; 0] }
#[repr(C)] pub struct skv_hot { _private: [u8; 0] }
#[repr(C)] pub struct skv_layer { _private: [u8; 0] }
#[repr(C)] pub struct skv_prefix { _private: [u8; 0] }
#[repr(C)] pub struct skv_prompt_cache { _private: [u8; 0] }
#[repr(C)] pub struct skv_rope { _private: [u8; 0] }
#[repr(C)] pub struct skv_snapshot { _private: [u8; 0] }

/// PrefixBlockHit with an opaque payload (src/serve/cache.rs:50-60).
#[repr(C)]
#[derive(Clone, Copy)]
pub struct skv_hit { pub tokens: usize, pub hash: [u8; 32], pub payload: u64, pub matched_blocks: usize }

/// A hipStream_t; null is the default stream.
pub type skv_stream = *mut c_void;

pub const SKV_OK: i32 = 0;
pub const SKV_ERR_DIMENSION: i32 = 1;
pub const SKV_ERR_CONFIG: i32 = 2;
pub const SKV_ERR_DEVICE: i32 = 3;
pub const SKV_ERR_MEMORY: i32 = 4;
pub const SKV_DTYPE_F32: i32 = 0;
pub const SKV_DTYPE_BF16: i32 = 1;
pub const SKV_PAGE_ROWS: usize = 16;
pub const SKV_STATIC_SCRATCH_BYTES: usize = 8 << 20;

#[link(name = "saragossa_kv")]
extern "C" {
    pub fn skv_last_error() -> *const c_char;
    pub fn skv_abi_version() -> i32;
    pub fn skv_env_flag(name: *const c_char, default_value: i32) -> i32;
    pub fn skv_env_flag_value(value: *const c_char) -> i32;
    pub fn skv_flag_kv_bf16_for(sampled: i32) -> i32;
    pub fn skv_flag_flash_sdpa_enabled() -> i32;
    pub fn skv_flag_sdpa_2pass_enabled() -> i32;
    pub fn skv_flag_sdpa_2pass_min_len() -> usize;
    pub fn skv_sdpa_2pass_blocks(len: usize) -> usize;
    pub fn skv_effective_split_min_len() -> usize;
    pub fn skv_flag_kv_bf16_sim_konly() -> i32;
    pub fn skv_flag_kv_bf16_sim_vonly() -> i32;
    pub fn skv_flag_attention_par_threshold() -> usize;
    pub fn skv_flag_decode_pipeline() -> i32;
    pub fn skv_flag_decode_resident_full() -> i32;
    pub fn skv_flag_decode_resident() -> i32;
    pub fn skv_flag_serve_prefix_cache_enabled() -> i32;
    pub fn skv_flag_serve_prefix_block_tokens() -> usize;
    pub fn skv_flag_serve_prefix_cache_blocks() -> usize;
    pub fn skv_flag_serve_prefix_blocks_per_session() -> usize;
    pub fn skv_flag_prefix_cache_enabled() -> i32;
    pub fn skv_flag_prefix_cache_capacity() -> usize;
    pub fn skv_flag_prefill_chunk() -> usize;
    pub fn skv_flag_memory_guard_enabled() -> i32;
    pub fn skv_flag_serve_oom_guard_enabled() -> i32;
    pub fn skv_flag_memory_static_cap_bytes() -> u64;
    pub fn skv_flag_memory_headroom_bytes() -> u64;
    pub fn skv_flag_serve_memory_static_cap_bytes() -> u64;
    pub fn skv_flag_serve_memory_headroom_bytes() -> u64;
    pub fn skv_flags_reload();
    pub fn skv_window_start(position: usize, window: usize) -> usize;
    pub fn skv_resident_capacity(prefill_len: usize, max_new_tokens: usize, draft_headroom: usize, capacity: *mut usize) -> i32;
    pub fn skv_resident_kv_bytes(capacity: usize, kv_dims: *const usize, n_layers: usize, elem_bytes: usize, bytes: *mut u64) -> i32;
    pub fn skv_memory_projection(current: u64, reserved: u64, requested: u64, limit: u64, projected: *mut u64, available: *mut u64) -> i32;
    pub fn skv_f32_to_bf16_bits(value: f32) -> u16;
    pub fn skv_ctx_create(device: i32, out: *mut *mut skv_ctx) -> i32;
    pub fn skv_ctx_destroy(ctx: *mut skv_ctx);
    pub fn skv_ctx_synchronize(ctx: *mut skv_ctx) -> i32;
    pub fn skv_layer_create(ctx: *mut skv_ctx, capacity: usize, q_heads: usize, kv_heads: usize, head_dim: usize, dtype: i32, window: usize, out: *mut *mut skv_layer) -> i32;
    pub fn skv_layer_create_ring(ctx: *mut skv_ctx, capacity: usize, q_heads: usize, kv_heads: usize, head_dim: usize, dtype: i32, window: usize, rollback_rows: usize, out: *mut *mut skv_layer) -> i32;
    pub fn skv_layer_create_for(ctx: *mut skv_ctx, capacity: usize, q_heads: usize, kv_heads: usize, head_dim: usize, sampled: i32, out: *mut *mut skv_layer) -> i32;
    pub fn skv_layer_destroy(layer: *mut skv_layer);
    pub fn skv_layer_bytes(capacity: usize, q_heads: usize, kv_heads: usize, head_dim: usize, dtype: i32, window: usize, bytes: *mut u64) -> i32;
    pub fn skv_layer_bytes_ring(capacity: usize, q_heads: usize, kv_heads: usize, head_dim: usize, dtype: i32, window: usize, rollback_rows: usize, bytes: *mut u64) -> i32;
    pub fn skv_check_allocation(ctx: *mut skv_ctx, requested: u64, static_cap: u64, headroom: u64, available: *mut u64, projected: *mut u64) -> i32;
    pub fn skv_layer_set_block_table(layer: *mut skv_layer, table: *const i32, n: usize) -> i32;
    pub fn skv_layer_pages(layer: *const skv_layer) -> usize;
    pub fn skv_kv_dim(layer: *const skv_layer) -> usize;
    pub fn skv_len(layer: *const skv_layer) -> usize;
    pub fn skv_capacity(layer: *const skv_layer) -> usize;
    pub fn skv_q_heads(layer: *const skv_layer) -> usize;
    pub fn skv_kv_heads(layer: *const skv_layer) -> usize;
    pub fn skv_head_dim(layer: *const skv_layer) -> usize;
    pub fn skv_window(layer: *const skv_layer) -> usize;
    pub fn skv_logical_byte_len(layer: *const skv_layer) -> usize;
    pub fn skv_truncate(layer: *mut skv_layer, len: usize) -> i32;
    pub fn skv_seed(layer: *mut skv_layer, keys: *const f32, values: *const f32, n_elems: usize, n_rows: usize) -> i32;
    pub fn skv_append_host(layer: *mut skv_layer, key: *const f32, value: *const f32, n_elems: usize) -> i32;
    pub fn skv_append_device(layer: *mut skv_layer, stream: skv_stream, k_dev: *const c_void, k_off: usize, v_dev: *const c_void, v_off: usize) -> i32;
    pub fn skv_append_batch_device(layer: *mut skv_layer, stream: skv_stream, k_dev: *const c_void, v_dev: *const c_void, n_rows: usize) -> i32;
    pub fn skv_attention_host(layer: *mut skv_layer, q: *const f32, n_elems: usize, window_start: usize, out: *mut f32) -> i32;
    pub fn skv_attention_device(layer: *mut skv_layer, stream: skv_stream, q_dev: *const f32, out_dev: *mut f32, window_start: usize) -> i32;
    pub fn skv_decode_step_device(layer: *mut skv_layer, stream: skv_stream, k_dev: *const c_void, k_off: usize, v_dev: *const c_void, v_off: usize, q_dev: *const f32, out_dev: *mut f32) -> i32;
    pub fn skv_decode_step_static_device(layer: *mut skv_layer, stream: skv_stream, k_dev: *const c_void, k_off: usize, v_dev: *const c_void, v_off: usize, q_dev: *const f32, out_dev: *mut f32) -> i32;
    pub fn skv_prefill_chunk_device(layer: *mut skv_layer, stream: skv_stream, q_dev: *const f32, k_dev: *const c_void, v_dev: *const c_void, n_rows: usize, out_dev: *mut f32) -> i32;
    pub fn skv_prefill_chunk_host(layer: *mut skv_layer, q: *const f32, k: *const f32, v: *const f32, n_rows: usize, out: *mut f32) -> i32;
    pub fn skv_rope_rotations_host(position: usize, rope_dims: usize, frequency_dim: usize, theta: f32, position_scale: f32, cos_sin_out: *mut f32) -> i32;
    pub fn skv_rope_create(ctx: *mut skv_ctx, max_positions: usize, rope_dims: usize, frequency_dim: usize, theta: f32, position_scale: f32, style: i32, out: *mut *mut skv_rope) -> i32;
    pub fn skv_rope_destroy(rope: *mut skv_rope);
    pub fn skv_rms_norm_rope_decode_device(ctx: *mut skv_ctx, stream: skv_stream, rope: *const skv_rope, position: usize, x_dev: *const f32, weight_dev: *const f32, heads: usize, head_dim: usize, eps: f32, out_dev: *mut f32) -> i32;
    pub fn skv_rms_norm_rope_rows_device(ctx: *mut skv_ctx, stream: skv_stream, rope: *const skv_rope, position_offset: usize, x_dev: *const f32, weight_dev: *const f32, n_rows: usize, heads: usize, head_dim: usize, eps: f32, out_dev: *mut f32) -> i32;
    pub fn skv_rms_norm_rope_decode_host(ctx: *mut skv_ctx, x: *const f32, weight: *const f32, heads: usize, head_dim: usize, rope_dims: usize, frequency_dim: usize, position: usize, eps: f32, theta: f32, position_scale: f32, style: i32, out: *mut f32) -> i32;
    pub fn skv_decode_step_prekv_device(layer: *mut skv_layer, stream: skv_stream, rope: *const skv_rope, position: usize, q_dev: *const c_void, q_off: usize, k_dev: *const c_void, k_off: usize, v_dev: *const c_void, v_off: usize, q_norm_w: *const f32, k_norm_w: *const f32, eps: f32, attn_scalar: f32, out_dev: *mut f32) -> i32;
    pub fn skv_decode_step_gated_device(layer: *mut skv_layer, stream: skv_stream, rope: *const skv_rope, position: usize, qg_dev: *const c_void, qg_off: usize, k_dev: *const c_void, k_off: usize, v_dev: *const c_void, v_off: usize, q_norm_w: *const f32, k_norm_w: *const f32, eps: f32, attn_scalar: f32, out_dev: *mut f32) -> i32;
    pub fn skv_attn_gate_device(ctx: *mut skv_ctx, stream: skv_stream, ctx_dev: *const f32, gate_dev: *const f32, gate_head_stride: usize, heads: usize, head_dim: usize, out_dev: *mut f32) -> i32;
    pub fn skv_decode_step_batch_device(seqs: *const *mut skv_layer, n_seq: usize, stream: skv_stream, k_dev: *const *const c_void, v_dev: *const *const c_void, q_dev: *const *const f32, out_dev: *const *mut f32) -> i32;
    pub fn skv_decode_step_layers_device(layers: *const *mut skv_layer, n_layers: usize, stream: skv_stream, k_dev: *const *const c_void, v_dev: *const *const c_void, q_dev: *const *const f32, out_dev: *const *mut f32) -> i32;
    pub fn skv_read_rows(layer: *mut skv_layer, first: usize, n: usize, k_out: *mut u16, v_out: *mut u16) -> i32;
    pub fn skv_read_rows_f32(layer: *mut skv_layer, first: usize, n: usize, k_out: *mut f32, v_out: *mut f32) -> i32;
    pub fn skv_gather_device(layer: *mut skv_layer, stream: skv_stream, first: usize, n: usize, k_dst_dev: *mut c_void, v_dst_dev: *mut c_void) -> i32;
    pub fn skv_probe_read_pages_device(layer: *mut skv_layer, stream: skv_stream) -> i32;
    pub fn skv_probe_read_store_pages_device(layer: *mut skv_layer, stream: skv_stream) -> i32;
    pub fn skv_probe_merge_device(layer: *mut skv_layer, stream: skv_stream, out_dev: *mut f32) -> i32;
    pub fn skv_probe_empty_launch_device(ctx: *mut skv_ctx, stream: skv_stream) -> i32;
    pub fn skv_snapshot_blocks(ctx: *mut skv_ctx, stream: skv_stream, layers: *const *mut skv_layer, n_layers: usize, block_ids: *const usize, n_blocks: usize, out: *mut *mut skv_snapshot) -> i32;
    pub fn skv_snapshot_clone(ctx: *mut skv_ctx, stream: skv_stream, snapshot: *const skv_snapshot, out: *mut *mut skv_snapshot) -> i32;
    pub fn skv_restore_blocks(ctx: *mut skv_ctx, stream: skv_stream, snapshot: *const skv_snapshot, layers: *const *mut skv_layer, n_layers: usize, dst_block_ids: *const usize, n_blocks: usize) -> i32;
    pub fn skv_snapshot_bytes(snapshot: *const skv_snapshot) -> usize;
    pub fn skv_snapshot_free(snapshot: *mut skv_snapshot);
    pub fn skv_state_snapshot(ctx: *mut skv_ctx, stream: skv_stream, dev_ptrs: *const *const c_void, bytes: *const usize, n: usize, out: *mut *mut skv_snapshot) -> i32;
    pub fn skv_state_restore(ctx: *mut skv_ctx, stream: skv_stream, snapshot: *const skv_snapshot, dev_ptrs: *const *mut c_void, bytes: *const usize, n: usize) -> i32;
    pub fn skv_hash_root(out: *mut u8);
    pub fn skv_hash_for_session(key: *const c_char, key_len: usize, out: *mut u8);
    pub fn skv_hash_chain(previous: *const u8, tokens: *const u64, n: usize, out: *mut u8);
    pub fn skv_prefix_create(block_tokens: usize, capacity: usize, blocks_per_session: usize, out: *mut *mut skv_prefix) -> i32;
    pub fn skv_prefix_from_runtime_flags(out: *mut *mut skv_prefix) -> i32;
    pub fn skv_prefix_destroy(cache: *mut skv_prefix);
    pub fn skv_prefix_block_tokens(cache: *const skv_prefix) -> usize;
    pub fn skv_prefix_capacity(cache: *const skv_prefix) -> usize;
    pub fn skv_prefix_len(cache: *const skv_prefix) -> usize;
    pub fn skv_prefix_bytes(cache: *const skv_prefix) -> usize;
    pub fn skv_prefix_session_block_count(cache: *const skv_prefix, session: *const u8) -> usize;
    pub fn skv_prefix_match(cache: *mut skv_prefix, root: *const u8, tokens: *const u64, n: usize, found: *mut i32, hit: *mut skv_hit, chain_payloads: *mut u64, chain_cap: usize) -> i32;
    pub fn skv_prefix_insert(cache: *mut skv_prefix, session: *const u8, hash: *const u8, tokens: usize, payload: u64, bytes: usize, dropped: *mut u64, dropped_cap: usize, n_dropped: *mut usize, bytes_out: *mut usize) -> i32;
    pub fn skv_prefix_evict_lru(cache: *mut skv_prefix, found: *mut i32, payload: *mut u64, bytes: *mut usize) -> i32;
    pub fn skv_prefix_entry(cache: *const skv_prefix, index: usize, session: *mut u8, hash: *mut u8, tokens: *mut usize, payload: *mut u64, bytes: *mut usize) -> i32;
    pub fn skv_hot_create(ctx: *mut skv_ctx, block_tokens: usize, capacity_blocks: usize, blocks_per_session: usize, pool_blocks: usize, layers: *const *mut skv_layer, n_layers: usize, out: *mut *mut skv_hot) -> i32;
    pub fn skv_hot_destroy(hot: *mut skv_hot);
    pub fn skv_hot_remember(hot: *mut skv_hot, stream: skv_stream, session: *const u8, hash: *const u8, tokens: usize, layers: *const *mut skv_layer, n_layers: usize, state_ptrs: *const *const c_void, state_bytes: *const usize, n_states: usize, cached: *mut i32) -> i32;
    pub fn skv_hot_remember_range(hot: *mut skv_hot, stream: skv_stream, session: *const u8, hashes: *const u8, first_tokens: usize, n_blocks: usize, layers: *const *mut skv_layer, n_layers: usize, n_cached: *mut usize) -> i32;
    pub fn skv_hot_match_restore(hot: *mut skv_hot, stream: skv_stream, root: *const u8, tokens: *const u64, n_tokens: usize, layers: *const *mut skv_layer, n_layers: usize, state_ptrs: *const *mut c_void, state_bytes: *const usize, n_states: usize, reused_tokens: *mut usize, hash_out: *mut u8) -> i32;
    pub fn skv_hot_evict_lru(hot: *mut skv_hot, found: *mut i32, bytes: *mut usize) -> i32;
    pub fn skv_hot_block_tokens(hot: *const skv_hot) -> usize;
    pub fn skv_hot_len(hot: *const skv_hot) -> usize;
    pub fn skv_hot_bytes(hot: *const skv_hot) -> usize;
    pub fn skv_hot_free_blocks(hot: *const skv_hot) -> usize;
    pub fn skv_hot_pool_blocks(hot: *const skv_hot) -> usize;
    pub fn skv_hot_block_bytes(hot: *const skv_hot) -> usize;
    pub fn skv_hot_evictions(hot: *const skv_hot) -> u64;
    pub fn skv_hot_skipped(hot: *const skv_hot) -> u64;
    pub fn skv_hot_entry(hot: *const skv_hot, index: usize, session: *mut u8, hash: *mut u8, tokens: *mut usize, bytes: *mut usize) -> i32;
    pub fn skv_prompt_cache_create(ctx: *mut skv_ctx, capacity: usize, out: *mut *mut skv_prompt_cache) -> i32;
    pub fn skv_prompt_cache_from_runtime_flags(ctx: *mut skv_ctx, out: *mut *mut skv_prompt_cache) -> i32;
    pub fn skv_prompt_cache_destroy(cache: *mut skv_prompt_cache);
    pub fn skv_prompt_cache_len(cache: *const skv_prompt_cache) -> usize;
    pub fn skv_prompt_cache_capacity(cache: *const skv_prompt_cache) -> usize;
    pub fn skv_prompt_cache_bytes(cache: *const skv_prompt_cache) -> usize;
    pub fn skv_prompt_cache_entry(cache: *const skv_prompt_cache, index: usize, n_tokens: *mut usize, tokens_out: *mut u64, tokens_cap: usize) -> i32;
    pub fn skv_prompt_cache_put(cache: *mut skv_prompt_cache, stream: skv_stream, tokens: *const u64, n_tokens: usize, layers: *const *mut skv_layer, n_layers: usize, state_ptrs: *const *const c_void, state_bytes: *const usize, n_states: usize) -> i32;
    pub fn skv_prompt_cache_get(cache: *mut skv_prompt_cache, stream: skv_stream, prompt: *const u64, n_prompt: usize, layers: *const *mut skv_layer, n_layers: usize, state_ptrs: *const *mut c_void, state_bytes: *const usize, n_states: usize, cached_tokens: *mut usize) -> i32;
}
