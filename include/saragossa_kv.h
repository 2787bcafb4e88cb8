/*
 * saragossa_kv.h — C ABI of the MI355X (gfx950) KV-cache hot path.
 *
 * Every entry point names the reference interface it stands in for
 * (paths relative to the reference repository root). Plain pointers and sizes
 * only; no torch types. Handles are opaque, owned by exactly one holder, not
 * clonable (src/decoder.rs:434-446, 682-697) and thread-affine: one decode at a
 * time per handle, no internal locking (src/decode_resident.rs:21-24).
 *
 * Status codes mirror InferError (src/error.rs:12-75): what the reference raises
 * as Dimension / Config / Metal comes back as SKV_ERR_DIMENSION / SKV_ERR_CONFIG /
 * SKV_ERR_DEVICE. Nothing here aborts the process on a fallible path; the text
 * of the last error on the calling thread is skv_last_error().
 *
 * Layout: the cache of one layer is a pool of 16-token pages reached through a
 * block table; logical row r of the reference's contiguous cache is
 * (block_table[r / 16], r % 16) here. A layer's elements are bf16, rounded from
 * f32 with the reference's integer formula (src/decode_resident/utils.rs:55-60),
 * or f32 kept verbatim (GpuElement, src/decode_resident/attention.rs:26-45).
 */
#ifndef SARAGOSSA_KV_H
#define SARAGOSSA_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SKV_OK 0
#define SKV_ERR_DIMENSION 1 /* InferError::Dimension: shapes, overflow at capacity, empty KV/window */
#define SKV_ERR_CONFIG 2    /* InferError::Config: zero dimension, bad GQA ratio, unsupported option */
#define SKV_ERR_DEVICE 3    /* InferError::Metal: device/runtime failure, null pointer, wrong element */
#define SKV_ERR_MEMORY 4    /* InferError::MemoryGuard: an allocation would pass the memory ceiling */

#define SKV_DTYPE_F32 0  /* GpuElement::F32: rows kept as they arrive */
#define SKV_DTYPE_BF16 1 /* GpuElement::Bf16 */

#define SKV_PAGE_ROWS 16

typedef struct skv_ctx skv_ctx;
typedef struct skv_layer skv_layer;
typedef struct skv_snapshot skv_snapshot;
typedef struct skv_prefix skv_prefix;
typedef struct skv_hot skv_hot;

/* A stream argument is a hipStream_t passed as void*; NULL is the default stream.
 * The *_device entry points only queue work on that stream: they neither wait for the
 * device nor switch devices, so the stream must belong to the context's device and that
 * device must be current on the calling thread (the *_host entry points and the create /
 * destroy calls make it current themselves). Two exceptions allocate, after a device
 * synchronisation: a chunked-prefill call whose split partials need more scratch than any
 * call before it on the same context and stream (one buffer per stream, which only grows: calls
 * on different streams never share partials), and the first attention call of a
 * layer on the plain kernel (RETI_RUST_FLASH_SDPA=0), which creates its score buffer. Host-side bookkeeping (len, ring position)
 * advances when the call returns, before the device has run the work, exactly like the
 * reference's encode-time `len += 1` (src/decode_resident/attention.rs:993); buffers handed
 * to a *_device call must stay valid until the stream has passed that work. */
typedef void *skv_stream;

/* ---- errors, version ---------------------------------------------------- */

/* Text of the last error raised on this thread ("" if none). InferError's Display. */
const char *skv_last_error(void);
int32_t skv_abi_version(void);

/* ---- runtime flags (src/runtime_flags.rs, src/decode_resident/utils.rs) -- */

/* env_flag (src/runtime_flags.rs:25-44): 1/true/on and 0/false/off, case- and
 * space-insensitive; anything else gives `default_value`. */
int32_t skv_env_flag(const char *name, int32_t default_value);
/* env_flag_value: 1, 0, or -1 for None. */
int32_t skv_env_flag_value(const char *value);
/* kv_bf16_for (src/decode_resident/utils.rs:202-221): RETI_RUST_KV_BF16 wins, else bf16 iff sampled. */
int32_t skv_flag_kv_bf16_for(int32_t sampled);
int32_t skv_flag_flash_sdpa_enabled(void);        /* RETI_RUST_FLASH_SDPA, utils.rs:182-185 */
int32_t skv_flag_sdpa_2pass_enabled(void);        /* RETI_RUST_SDPA_2PASS, utils.rs:260-263 */
size_t skv_flag_sdpa_2pass_min_len(void);         /* RETI_RUST_SDPA_2PASS_MIN_LEN, utils.rs:270-278 */
size_t skv_sdpa_2pass_blocks(size_t len);         /* utils.rs:282-286 */
/* Rows from which this library splits the context of a decode launch: RETI_RUST_SDPA_2PASS_MIN_LEN
 * when it is set (the reference's parse, default 2048 when unparsable), else 128. The reference's
 * own default (2048, utils.rs:270-278) is what skv_flag_sdpa_2pass_min_len reports; it was tuned
 * for another GPU, and one workgroup per kv head would leave this one idle. */
size_t skv_effective_split_min_len(void);
int32_t skv_flag_kv_bf16_sim_konly(void);         /* RETI_RUST_KV_BF16_SIM_KONLY, utils.rs:245-248; honoured by skv_seed */
int32_t skv_flag_kv_bf16_sim_vonly(void);         /* RETI_RUST_KV_BF16_SIM_VONLY, utils.rs:253-256; honoured by skv_seed */
/* RETI_RUST_ATTENTION_PAR_THRESHOLD (runtime_flags.rs:641-649, default 128): cache length from
 * which the CPU path spreads the query heads over threads (src/decoder/attention_ops.rs:926).
 * The device path has no use for it; a host that keeps a CPU fallback reads it here. */
size_t skv_flag_attention_par_threshold(void);
/* RETI_RUST_DECODE_PIPELINE (runtime_flags.rs:309-313, default on): whether the host keeps
 * several tokens in flight (src/decoder/generation.rs:831). Every *_device entry point only
 * queues work, so both settings are served; the getter is for the host's loop. */
int32_t skv_flag_decode_pipeline(void);
int32_t skv_flag_decode_resident_full(void);      /* RETI_RUST_DECODE_RESIDENT_FULL, runtime_flags.rs:283-286 */
int32_t skv_flag_decode_resident(void);           /* RETI_RUST_DECODE_RESIDENT, runtime_flags.rs:266-269 */
int32_t skv_flag_serve_prefix_cache_enabled(void);   /* RETI_SERVE_PREFIX_CACHE, runtime_flags.rs:681-684 */
size_t skv_flag_serve_prefix_block_tokens(void);     /* runtime_flags.rs:727-736 */
size_t skv_flag_serve_prefix_cache_blocks(void);     /* runtime_flags.rs:739-747 */
size_t skv_flag_serve_prefix_blocks_per_session(void); /* runtime_flags.rs:750-758 */
int32_t skv_flag_prefix_cache_enabled(void);      /* RETI_RUST_PREFIX_CACHE, runtime_flags.rs:665-668 */
size_t skv_flag_prefix_cache_capacity(void);      /* RETI_RUST_PREFIX_CACHE_CAP, runtime_flags.rs:670-678 */
size_t skv_flag_prefill_chunk(void);              /* RETI_RUST_PREFILL_CHUNK (alias _STEP_SIZE), runtime_flags.rs:414-423 */
/* The switches and limits of the memory guard that drives prefix-block eviction
 * (src/serve/state.rs:226-238, 287-306, 627-635): a host feeds them to skv_check_allocation /
 * skv_memory_projection. A cap of 0 = none set (the reference's None; a zero in the
 * environment is filtered out). */
int32_t skv_flag_memory_guard_enabled(void);          /* RETI_MEMORY_GUARD, runtime_flags.rs:699-702 */
int32_t skv_flag_serve_oom_guard_enabled(void);       /* memory guard && RETI_SERVE_OOM_GUARD, runtime_flags.rs:693-696 */
uint64_t skv_flag_memory_static_cap_bytes(void);      /* RETI_MEMORY_CAP_BYTES, runtime_flags.rs:705-713 */
uint64_t skv_flag_memory_headroom_bytes(void);        /* RETI_MEMORY_HEADROOM_BYTES, default 2 GiB, runtime_flags.rs:716-724 */
uint64_t skv_flag_serve_memory_static_cap_bytes(void);   /* RETI_SERVE_MEMORY_CAP_BYTES, runtime_flags.rs:773-781 */
uint64_t skv_flag_serve_memory_headroom_bytes(void);     /* RETI_SERVE_MEMORY_HEADROOM_BYTES, default 2 GiB, runtime_flags.rs:784-792 */
/* The reference freezes each flag at first read (OnceLock). This re-reads the
 * environment; it exists for tests only. */
void skv_flags_reload(void);
/* window_start of a sliding layer (src/decoder/resident/types.rs:13-18); window 0 = none. */
size_t skv_window_start(size_t position, size_t window);
/* Rows a resident cache is created with: prefill_len + max_new_tokens + draft_headroom with
 * checked additions (setup_resident_full_decode_with_slot, src/decoder/resident/setup.rs:322-329).
 * Returns 1 and writes *capacity, or 0 when the sum overflows (the reference's
 * "capacité KV résidente déborde"). A capacity of 0 means there is nothing to set up. */
int32_t skv_resident_capacity(size_t prefill_len, size_t max_new_tokens, size_t draft_headroom,
                              size_t *capacity);
/* The KV part of check_resident_full_decode_allocation (src/decoder/resident/setup.rs:897-917):
 * sum over the layers of 2 * capacity * kv_dims[i] * elem_bytes (the reference counts
 * size_of::<f32>() = 4), each product checked, the sum saturating. Returns 1 and writes *bytes,
 * or 0 when a product overflows ("KV résident déborde"). */
int32_t skv_resident_kv_bytes(size_t capacity, const size_t *kv_dims, size_t n_layers, size_t elem_bytes,
                              uint64_t *bytes);
/* MemoryGuard::projection_with_reserved / projection_over_limit (src/memory_guard.rs:334-362):
 * projected = current + reserved + requested (saturating), available = limit - (current +
 * reserved), floored at 0. Returns 1 when projected > limit, else 0. Pure arithmetic. */
int32_t skv_memory_projection(uint64_t current, uint64_t reserved, uint64_t requested, uint64_t limit,
                              uint64_t *projected, uint64_t *available);
/* f32 -> bf16 bits, the reference's formula (src/decode_resident/utils.rs:55-60). Host helper. */
uint16_t skv_f32_to_bf16_bits(float value);

/* ---- context ------------------------------------------------------------ */

/* DecodeResidentState::new(device) (src/decoder/resident/setup.rs:237, 675). */
int32_t skv_ctx_create(int32_t device, skv_ctx **out);
/* Waits for the device, gives back the device memory the context itself holds and ends the
 * caller's use of `ctx`. Layers, rope tables, snapshots and hot caches made from it stay valid
 * until their own destroy call (the order of the destroy calls is free, as with finalisers of a
 * garbage-collected binding); making new objects from a destroyed context is an error of the
 * caller. */
void skv_ctx_destroy(skv_ctx *ctx);
/* Blocks until everything queued on the context's own stream has finished. */
int32_t skv_ctx_synchronize(skv_ctx *ctx);

/* ---- one layer's cache: FullAttentionMetalState -------------------------- */

/* DecodeResidentState::full_attention_with_element (src/decode_resident/attention.rs:56-108).
 * Rejects a zero dimension and q_heads % kv_heads != 0 with SKV_ERR_CONFIG.
 * `window` > 0 makes the layer a ring buffer that keeps the last `window` rows plus
 * SKV_RING_SLACK_ROWS (environment, default 32) rows behind them, rounded up to whole pages:
 * the slack is what lets a speculative verify of up to that many rows be rolled back with
 * skv_truncate (the reference keeps the whole cache and rolls back freely,
 * src/decoder/attention_cache.rs:72-100); 0 keeps all `capacity` rows in pages.
 * `dtype` is what the pages hold: SKV_DTYPE_BF16 (rows rounded to nearest even at append,
 * pages of kv_heads * P * 32 bytes per tensor, P = head_dim rounded up to a power of two) or
 * SKV_DTYPE_F32 (rows verbatim; pages twice the bytes). head_dim up to 512 in both. Every
 * entry point below serves both; where they differ it says so. */
int32_t skv_layer_create(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads,
                         size_t head_dim, int32_t dtype, size_t window, skv_layer **out);
/* skv_layer_create with the rollback depth of a ring layer as an argument: the ring keeps
 * `window` + `rollback_rows` rows (rounded up to whole pages, never more than `capacity`), so a
 * host whose speculative draft is deeper than the default 32 rows (or that never rolls back:
 * 0) says so here instead of through the environment. The reference keeps the whole cache and
 * truncates freely (src/decoder/attention_cache.rs:72-100; rollback in
 * src/decoder/generation.rs:924-1026); a rollback deeper than the ring kept is reported by
 * the next attention call. SIZE_MAX = the default (SKV_RING_SLACK_ROWS, else 32); ignored when
 * `window` is 0. */
int32_t skv_layer_create_ring(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads, size_t head_dim,
                              int32_t dtype, size_t window, size_t rollback_rows, skv_layer **out);
/* full_attention(capacity, q_heads, kv_heads, head_dim, sampled) (attention.rs:26-45):
 * element type from skv_flag_kv_bf16_for(sampled). */
int32_t skv_layer_create_for(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads,
                             size_t head_dim, int32_t sampled, skv_layer **out);
void skv_layer_destroy(skv_layer *layer);
/* Device bytes skv_layer_create will take for these arguments (pools of whole pages, block
 * table, split partials, staging rows), after the same checks: what a host adds up before it
 * creates a model's layers, where the reference adds up 2 * capacity * kv_dim * 4 per layer
 * (check_resident_full_decode_allocation, src/decoder/resident/setup.rs:897-962). A bf16
 * layer takes about half of an f32 one; a ring layer's size follows its window, not capacity. */
int32_t skv_layer_bytes(size_t capacity, size_t q_heads, size_t kv_heads, size_t head_dim, int32_t dtype,
                        size_t window, uint64_t *bytes);
/* The same for skv_layer_create_ring (no counterpart in the reference, whose caches are never rings). */
int32_t skv_layer_bytes_ring(size_t capacity, size_t q_heads, size_t kv_heads, size_t head_dim, int32_t dtype,
                             size_t window, size_t rollback_rows, uint64_t *bytes);
/* MemoryGuard::check_allocation (src/memory_guard.rs:365-370) against the context's device:
 * current = device memory in use minus what the context's own arena holds for reuse, limit =
 * device memory - headroom, further capped by static_cap when that is not 0. SKV_ERR_MEMORY
 * when current + requested > limit; *available and *projected (either may be null) as in
 * MemoryProjection. */
int32_t skv_check_allocation(skv_ctx *ctx, uint64_t requested, uint64_t static_cap, uint64_t headroom,
                             uint64_t *available, uint64_t *projected);

/* Replace the block table (logical block -> physical page) with a permutation of
 * [0, skv_layer_pages). Only while the layer is empty. No reference counterpart:
 * the reference cache is contiguous. */
int32_t skv_layer_set_block_table(skv_layer *layer, const int32_t *table, size_t n);
size_t skv_layer_pages(const skv_layer *layer);

/* kv_dim / len / capacity / q_heads / kv_heads / head_dim (attention.rs:485-548). */
size_t skv_kv_dim(const skv_layer *layer);
size_t skv_len(const skv_layer *layer);
size_t skv_capacity(const skv_layer *layer);
size_t skv_q_heads(const skv_layer *layer);
size_t skv_kv_heads(const skv_layer *layer);
size_t skv_head_dim(const skv_layer *layer);
size_t skv_window(const skv_layer *layer);
/* keys().byte_len() of the reference for the same capacity (tests.rs:446): capacity*kv_dim*2. */
size_t skv_logical_byte_len(const skv_layer *layer);
/* truncate(len) (attention.rs:496-505): error if len > capacity. */
int32_t skv_truncate(skv_layer *layer, size_t len);

/* seed(keys_rows, values_rows, n_rows) (attention.rs:550-602): host f32 rows
 * [n_rows, kv_dim] written from row 0, len = n_rows. `n_elems` is the length of
 * each slice and must equal n_rows*kv_dim. Synchronous. */
int32_t skv_seed(skv_layer *layer, const float *keys, const float *values, size_t n_elems,
                 size_t n_rows);
/* append_row(key, value) (attention.rs:611-644): host f32 slices of `n_elems` ==
 * kv_dim; SKV_ERR_DIMENSION at capacity. Synchronous. */
int32_t skv_append_host(skv_layer *layer, const float *key, const float *value, size_t n_elems);
/* encode_append_kv_with_offsets (attention.rs:959-995): device f32 buffers plus
 * byte offsets; len advances on the host at call time; the copy runs on `stream`. */
int32_t skv_append_device(skv_layer *layer, skv_stream stream, const void *k_dev, size_t k_off,
                          const void *v_dev, size_t v_off);
/* Batched device append of n_rows rows ([n_rows, kv_dim] f32 each): the device
 * twin of LayerKvCache::append_batch (src/decoder/attention_cache.rs:38-70). */
int32_t skv_append_batch_device(skv_layer *layer, skv_stream stream, const void *k_dev,
                                const void *v_dev, size_t n_rows);

/* attention_decode / attention_decode_windowed (attention.rs:660-717): host q of
 * `n_elems` == q_heads*head_dim in, raw context [q_dim] out, rows
 * window_start..len. Synchronous. */
int32_t skv_attention_host(skv_layer *layer, const float *q, size_t n_elems, size_t window_start,
                           float *out);
/* encode_attention_decode_windowed (attention.rs:738-835): device q and out, async on `stream`. */
int32_t skv_attention_device(skv_layer *layer, skv_stream stream, const float *q_dev,
                             float *out_dev, size_t window_start);
/* append + attention of one token in one call (layers.rs:259-288 does the two
 * encodes back to back). window_start is derived from the layer's window. On the GPU it is one
 * launch pair (the attention kernel stores the new row itself) for bf16 layers up to head_dim
 * 512 and for f32 layers up to head_dim 256 with at most 16 query heads per kv head; other
 * f32 shapes, and every shape with RETI_RUST_FLASH_SDPA=0, take an append launch first (the
 * f32 kernel for wide heads has no registers to spare: with the append built into it the step
 * takes 48.7 us against 44.1 us at 4096 rows of q16/kv8/hd512, 260 against 253 us at 32768). */
int32_t skv_decode_step_device(skv_layer *layer, skv_stream stream, const void *k_dev,
                               size_t k_off, const void *v_dev, size_t v_off, const float *q_dev,
                               float *out_dev);

/* skv_decode_step_device for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same
 * arguments, same result; the launch's split-K partials live in a static device array of
 * SKV_STATIC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends,
 * instead of the layer's own buffers, and the call makes no allocation and frees nothing.
 * SKV_ERR_DIMENSION when the partials of the launch (q_heads * splits * (head_dim + 2) * 4
 * bytes; splits follow the context length, 256 workgroups at most) would not fit,
 * SKV_ERR_CONFIG with RETI_RUST_FLASH_SDPA=0 (the plain kernel allocates its score buffer).
 * The array keeps the last call's contents and needs no clearing (every partial a launch reads
 * it has written itself), but all calls on one GPU share it: calls that overlap on one GPU,
 * on different streams or from different threads, race. */
#define SKV_STATIC_SCRATCH_BYTES ((size_t)8 << 20)
int32_t skv_decode_step_static_device(skv_layer *layer, skv_stream stream, const void *k_dev,
                                      size_t k_off, const void *v_dev, size_t v_off,
                                      const float *q_dev, float *out_dev);

/* Chunked prefill over the cache: appends n_rows rows (k_dev, v_dev: [n_rows, kv_dim] f32)
 * and computes, for every new row i, attention of q_dev[i] over rows 0..len_before+i through
 * the layer's sliding window: cached_attention_prefill_rows
 * (src/decoder/attention_ops.rs:976-1017) as one launch on the matrix cores instead of
 * the reference's per-row loop (src/decode_resident/layers.rs:1113-1118). out_dev is
 * [n_rows, q_dim] f32. */
int32_t skv_prefill_chunk_device(skv_layer *layer, skv_stream stream, const float *q_dev,
                                 const void *k_dev, const void *v_dev, size_t n_rows,
                                 float *out_dev);
/* Same with host buffers; synchronous. */
int32_t skv_prefill_chunk_host(skv_layer *layer, const float *q, const float *k, const float *v,
                               size_t n_rows, float *out);

/* ---- The step before the cache: per-head RMSNorm + rotation at the token's position ----
 * rope_rotations (src/decoder/attention_ops.rs:848-887): cos and sin of
 * (position * position_scale) / theta^(2*pair / frequency_dim) for every pair, computed
 * on the host in f32 with libm exactly as the reference's CPU path does; cos_sin_out
 * receives rope_dims floats, (cos, sin) per pair. frequency_dim 0 = rope_dims. */
int32_t skv_rope_rotations_host(size_t position, size_t rope_dims, size_t frequency_dim, float theta,
                                float position_scale, float *cos_sin_out);

/* The same rotations for positions 0..max_positions-1 as a device table, built once per
 * (theta, scale, rope_dims) of a model; it replaces the reference's process-global memo of
 * rope_rotations. style: 0 = RopeStyle::Halves, 1 = RopeStyle::Interleaved
 * (src/decoder.rs:70-76). */
typedef struct skv_rope skv_rope;
int32_t skv_rope_create(skv_ctx *ctx, size_t max_positions, size_t rope_dims, size_t frequency_dim,
                        float theta, float position_scale, int32_t style, skv_rope **out);
void skv_rope_destroy(skv_rope *rope);

/* encode_rms_norm_rope_decode[_with_offset] (src/decode_resident/layers.rs:214-227, kernel
 * rms_norm_rope_heads_decode_f32, src/decode_resident/kernels.rs:975-1027): out = per-head
 * RMSNorm(x) * weight, then the rotation of `position` on the first rope_dims dims of each
 * head. weight_dev null = no norm (apply_rope_heads_at, attention_ops.rs:779-834); rope
 * null = no rotation. Same arithmetic, in the same order, as rms_norm_rope_heads_at
 * (attention_ops.rs:682-777). */
int32_t skv_rms_norm_rope_decode_device(skv_ctx *ctx, skv_stream stream, const skv_rope *rope,
                                        size_t position, const float *x_dev, const float *weight_dev,
                                        size_t heads, size_t head_dim, float eps, float *out_dev);
/* The same for n_rows consecutive rows (a prefill chunk): row r, contiguous after row r-1,
 * is rotated at position_offset + r, as rms_norm_rope_heads_at does for a [seq, dim] tensor
 * (src/decoder/attention_ops.rs:682-777, position_offset + pos at lines 736-739). */
int32_t skv_rms_norm_rope_rows_device(skv_ctx *ctx, skv_stream stream, const skv_rope *rope,
                                      size_t position_offset, const float *x_dev, const float *weight_dev,
                                      size_t n_rows, size_t heads, size_t head_dim, float eps,
                                      float *out_dev);
/* DecodeResidentState::rms_norm_rope_decode (src/decode_resident/tests.rs:1168-1172, 1883):
 * host in, host out, synchronous; the rotations of `position` are computed on the host. */
int32_t skv_rms_norm_rope_decode_host(skv_ctx *ctx, const float *x, const float *weight, size_t heads,
                                      size_t head_dim, size_t rope_dims, size_t frequency_dim,
                                      size_t position, float eps, float theta, float position_scale,
                                      int32_t style, float *out);

/* encode_resident_full_layer from the q/k norms to the attention context
 * (src/decode_resident/layers.rs:214-288) in one launch pair: RMSNorm + rotation of the raw
 * q (q_heads*head_dim f32 at q_dev + q_off) and of the raw k row, the query scale
 * sqrt(head_dim / attn_scalar) (encode_query_attention_scale, layers.rs:7-33; an invalid
 * attn_scalar is SKV_ERR_CONFIG), append of (k, v) and attention through the layer's
 * window. q_norm_w / k_norm_w: device f32[head_dim], null = that norm is skipped. The
 * finished q is not written back; the appended k row is the CPU path's row bit for bit.
 * (One launch pair on bf16 layers of any head_dim and on f32 layers up to head_dim 256, at
 * most 16 query heads per kv head; on f32 layers with wider heads, or more heads per group,
 * the norm and rotation, the append and the attention are separate launches with the same
 * result. Measured on one MI355X at q16/kv8/hd512: an f32 layer's step as those four launches
 * takes 61 us at 4096 cached rows and 267 us at 32768, its attention launches alone 41 us and
 * 254 us; a bf16 layer's one launch pair takes 31 us and 112 us, the same step as separate
 * launches 44 us and 123 us.) */
int32_t skv_decode_step_prekv_device(skv_layer *layer, skv_stream stream, const skv_rope *rope,
                                     size_t position, const void *q_dev, size_t q_off,
                                     const void *k_dev, size_t k_off, const void *v_dev, size_t v_off,
                                     const float *q_norm_w, const float *k_norm_w, float eps,
                                     float attn_scalar, float *out_dev);

/* The same step for a layer with an output gate (attn_output_gate, Qwen3.5/3.6 full-attention
 * layers): qg_dev + qg_off is the gated q projection, per head head_dim query values then
 * head_dim gate values (split_q_gate_f32, src/decode_resident/kernels.rs:931-946;
 * split_attention_gate, src/decoder/attention_ops.rs:486-520), read in place; the context
 * leaves the kernel already multiplied by sigmoid(gate) (attn_gate_f32, kernels.rs:949-959;
 * attention_ops.rs:217-219, 522-524), ready for the o projection. */
int32_t skv_decode_step_gated_device(skv_layer *layer, skv_stream stream, const skv_rope *rope,
                                     size_t position, const void *qg_dev, size_t qg_off,
                                     const void *k_dev, size_t k_off, const void *v_dev, size_t v_off,
                                     const float *q_norm_w, const float *k_norm_w, float eps,
                                     float attn_scalar, float *out_dev);
/* encode_attn_gate (attn_gate_f32, src/decode_resident/kernels.rs:949-959) on its own:
 * out[h][c] = ctx[h][c] * sigmoid(gate[h * gate_head_stride + c]); stride 0 = head_dim;
 * out may be ctx. */
int32_t skv_attn_gate_device(skv_ctx *ctx, skv_stream stream, const float *ctx_dev, const float *gate_dev,
                             size_t gate_head_stride, size_t heads, size_t head_dim, float *out_dev);

/* One decode step of the SAME model layer for n_seq independent sequences (each its own
 * handle, block table and length): for sequence i, append k_dev[i]/v_dev[i] (kv_dim f32
 * each) then attention of q_dev[i] into out_dev[i], all in one pair of launches. The
 * reference decodes one sequence at a time (encode_resident_full_layer,
 * src/decode_resident/layers.rs:259-288, once per sequence); this is that call applied to
 * a batch, with the same result per sequence. All handles must share the head geometry,
 * the element, the window and the context, and be distinct; nothing is modified when one of
 * them is at capacity. (One launch pair on either element up to 16 query heads per kv head,
 * f32 layers up to head_dim 256; other shapes run a launch pair per sequence.) */
int32_t skv_decode_step_batch_device(skv_layer *const *seqs, size_t n_seq, skv_stream stream,
                                     const void *const *k_dev, const void *const *v_dev,
                                     const float *const *q_dev, float *const *out_dev);

/* The KV path of one token over several layers: for each layer i, append
 * k_dev[i]/v_dev[i] (kv_dim f32 each) then attention of q_dev[i] into out_dev[i].
 * It is the per-layer loop of enqueue_decode_token_resident
 * (src/decoder/resident/decode.rs:183-458) restricted to the append and attention
 * encodes, issued from native code so that a host in another language pays one
 * FFI crossing per token instead of two per layer. */
int32_t skv_decode_step_layers_device(skv_layer *const *layers, size_t n_layers, skv_stream stream,
                                      const void *const *k_dev, const void *const *v_dev,
                                      const float *const *q_dev, float *const *out_dev);

/* Reads logical rows [first, first+n) through the block table as bf16 bits,
 * row-major [n, kv_dim]: the stand-in for reading keys()/values() back
 * (tests.rs:423-428, 469-476). Synchronous. bf16 layers only (SKV_ERR_CONFIG on an f32 one). */
int32_t skv_read_rows(skv_layer *layer, size_t first, size_t n, uint16_t *k_out, uint16_t *v_out);
/* The same rows as f32, for layers of either element type (bf16 rows widen exactly). */
int32_t skv_read_rows_f32(skv_layer *layer, size_t first, size_t n, float *k_out, float *v_out);
/* Same gather, device to device, async on `stream`; the destination rows have the layer's
 * element type (bf16 bits or f32). */
int32_t skv_gather_device(skv_layer *layer, skv_stream stream, size_t first, size_t n,
                          void *k_dst_dev, void *v_dst_dev);

/* ---- measurement aids (no counterpart in the reference; used by bench.py) ---- */

/* Reads every K and V page of the layer's first `len` rows once, through the block table, with
 * the decode kernel's grid and access pattern (256 workgroups of 8 wavefronts by default, 16-byte
 * non-temporal loads of whole tiles) and does nothing with them: what a launch that only
 * had to fetch the cache would cost. Async on `stream`. */
int32_t skv_probe_read_pages_device(skv_layer *layer, skv_stream stream);
/* The same launch, each workgroup also writing a split partial of the decode kernel's size
 * (heads-per-group * head_dim f32, non-temporal stores) into the layer's partial buffer once
 * its last page has arrived: the least a split-K launch must do before a merge can run. The
 * layer's partials are overwritten (the next attention call rewrites them anyway). */
int32_t skv_probe_read_store_pages_device(skv_layer *layer, skv_stream stream);
/* The merge launch of a decode step at the layer's current length, over whatever split
 * partials the layer's buffers hold (those of its last attention call), into out_dev
 * (q_heads * head_dim f32): behind skv_probe_read_pages_device it is what a decode launch pair
 * costs when nothing is multiplied. Nothing is launched when the step would take one split. */
int32_t skv_probe_merge_device(skv_layer *layer, skv_stream stream, float *out_dev);
/* An empty kernel with the decode launch's shape: the cost of a launch alone. */
int32_t skv_probe_empty_launch_device(skv_ctx *ctx, skv_stream stream);

/* ---- block snapshots: snapshot/copy/restore_prompt_state_metal ------------- */

/* Deep copy of logical blocks (16-row pages) `block_ids` of every layer into storage the
 * snapshot owns: the block-paged form of snapshot_prompt_state_metal
 * (src/decoder/generation.rs:2834-2849). Async on `stream`. */
int32_t skv_snapshot_blocks(skv_ctx *ctx, skv_stream stream, skv_layer *const *layers,
                            size_t n_layers, const size_t *block_ids, size_t n_blocks,
                            skv_snapshot **out);
/* copy_prompt_state_metal_snapshot (generation.rs:2856-2871): an independent copy, so that
 * restoring never aliases the cached entry (src/serve/state.rs:580-584). */
int32_t skv_snapshot_clone(skv_ctx *ctx, skv_stream stream, const skv_snapshot *snapshot,
                           skv_snapshot **out);
/* restore_prompt_state_metal (generation.rs:2878-2892): block i of the snapshot goes to
 * logical block dst_block_ids[i] of every layer; SKV_ERR_DIMENSION when the layer count
 * or shapes differ (generation.rs:3086-3092). The caller sets the length with skv_truncate. */
int32_t skv_restore_blocks(skv_ctx *ctx, skv_stream stream, const skv_snapshot *snapshot,
                           skv_layer *const *layers, size_t n_layers, const size_t *dst_block_ids,
                           size_t n_blocks);
/* estimated_bytes (src/decoder.rs:273-289). */
size_t skv_snapshot_bytes(const skv_snapshot *snapshot);
void skv_snapshot_free(skv_snapshot *snapshot);
/* snapshot_linear_attn_states / restore (src/metal_backend/linear_attention.rs:3027-3067,
 * 3163-3198): n device buffers (conv and ssm state of every linear-attention layer)
 * copied in one launch. Pointers must be 16-byte aligned. */
int32_t skv_state_snapshot(skv_ctx *ctx, skv_stream stream, const void *const *dev_ptrs,
                           const size_t *bytes, size_t n, skv_snapshot **out);
int32_t skv_state_restore(skv_ctx *ctx, skv_stream stream, const skv_snapshot *snapshot,
                          void *const *dev_ptrs, const size_t *bytes, size_t n);

/* ---- prefix hot cache, host index: BlockHash + BlockAwarePrefixCache -------- */

/* BlockHash::root / for_session / chain (src/serve/cache.rs:10-47). A null or empty key
 * gives the root; tokens are hashed as u64 little-endian after the previous digest. */
void skv_hash_root(uint8_t out[32]);
void skv_hash_for_session(const char *key, size_t key_len, uint8_t out[32]);
void skv_hash_chain(const uint8_t previous[32], const uint64_t *tokens, size_t n, uint8_t out[32]);

/* PrefixBlockHit (src/serve/cache.rs:50-60) with an opaque payload in place of the state. */
typedef struct skv_hit {
    size_t tokens;
    uint8_t hash[32];
    uint64_t payload;
    size_t matched_blocks;
} skv_hit;

/* with_blocks_per_session / from_runtime_flags (src/serve/cache.rs:83-112); block_tokens 0 -> 1. */
int32_t skv_prefix_create(size_t block_tokens, size_t capacity, size_t blocks_per_session,
                          skv_prefix **out);
int32_t skv_prefix_from_runtime_flags(skv_prefix **out);
void skv_prefix_destroy(skv_prefix *cache);
size_t skv_prefix_block_tokens(const skv_prefix *cache);
size_t skv_prefix_capacity(const skv_prefix *cache);
size_t skv_prefix_len(const skv_prefix *cache);
/* estimated_bytes (src/serve/cache.rs:202-204). */
size_t skv_prefix_bytes(const skv_prefix *cache);
size_t skv_prefix_session_block_count(const skv_prefix *cache, const uint8_t session[32]);
/* match_prefix (src/serve/cache.rs:121-151). *found = 1 and *hit filled on a hit;
 * chain_payloads (optional, chain_cap entries) receives the payload of every matched
 * block in chain order. */
int32_t skv_prefix_match(skv_prefix *cache, const uint8_t root[32], const uint64_t *tokens, size_t n,
                         int32_t *found, skv_hit *hit, uint64_t *chain_payloads, size_t chain_cap);
/* insert (src/serve/cache.rs:154-193). Payloads that leave the index (an equal key that was
 * replaced, the session's least recent block, the global least recent block, or the new
 * payload itself when capacity is 0) are written to `dropped` (at least 4 places) so the
 * caller can release what they stand for. *bytes_out is insert's return value. */
int32_t skv_prefix_insert(skv_prefix *cache, const uint8_t session[32], const uint8_t hash[32],
                          size_t tokens, uint64_t payload, size_t bytes, uint64_t *dropped,
                          size_t dropped_cap, size_t *n_dropped, size_t *bytes_out);
/* evict_lru_block (src/serve/cache.rs:196-198). */
int32_t skv_prefix_evict_lru(skv_prefix *cache, int32_t *found, uint64_t *payload, size_t *bytes);
/* Entry `index` in recency order (0 = most recent): the tests' view of `cache.entries`. */
int32_t skv_prefix_entry(const skv_prefix *cache, size_t index, uint8_t session[32], uint8_t hash[32],
                         size_t *tokens, uint64_t *payload, size_t *bytes);

/* ---- prefix hot cache on the GPU: page pool + index --------------------------- */

/* A pool of `pool_blocks` prefix blocks (each block_tokens/16 page slots holding K and V
 * of every layer) indexed like BlockAwarePrefixCache. `layers` fixes the shapes the pool
 * is laid out for; any set of layers with the same shapes can be used afterwards.
 * Copies into and out of the pool are ordered only by the streams they are queued on: use
 * one stream for all calls on a hot cache (the reference's server is single-threaded,
 * src/serve/state.rs:560-646), or order the streams yourself, because an evicted block's
 * slots are reused by the next remember without waiting for the device. */
int32_t skv_hot_create(skv_ctx *ctx, size_t block_tokens, size_t capacity_blocks,
                       size_t blocks_per_session, size_t pool_blocks, skv_layer *const *layers,
                       size_t n_layers, skv_hot **out);
void skv_hot_destroy(skv_hot *hot);
/* remember_prefix_block (src/serve/state.rs:613-639) for the block of rows
 * [tokens - block_tokens, tokens): evicts least-recent blocks while the pool is full,
 * copies the pages (and, if n_states > 0, the recurrent-state buffers) and inserts.
 * *cached = 0 when nothing was left to evict or the cache is disabled (no error). */
int32_t skv_hot_remember(skv_hot *hot, skv_stream stream, const uint8_t session[32],
                         const uint8_t hash[32], size_t tokens, skv_layer *const *layers,
                         size_t n_layers, const void *const *state_ptrs, const size_t *state_bytes,
                         size_t n_states, int32_t *cached);
/* remember_prefix_block for n_blocks consecutive boundaries (first_tokens, first_tokens +
 * block_tokens, ...) keyed by hashes[i] (n_blocks x 32 bytes): the same evictions and
 * insertions in the same order as separate calls, with the page copies queued together. What
 * the block-boundary loop of prefill_prompt_state (src/serve/state.rs:595-602) does after a
 * chunk that spans several blocks. No recurrent state. *n_cached counts the blocks kept. */
int32_t skv_hot_remember_range(skv_hot *hot, skv_stream stream, const uint8_t session[32],
                               const uint8_t *hashes, size_t first_tokens, size_t n_blocks,
                               skv_layer *const *layers, size_t n_layers, size_t *n_cached);
/* The hit branch of prefill_prompt_state (src/serve/state.rs:574-584): longest cached
 * chain for `tokens` under `root`, its pages gathered into rows [0, *reused_tokens) of the
 * layers, the last block's recurrent state copied to state_ptrs, each layer's len set to
 * *reused_tokens. *reused_tokens = 0 on a miss (layers untouched). The copies of the first
 * matched blocks are queued while the rest of the chain is still being hashed: an error found
 * after that (a chain longer than a layer's capacity, state buffers that do not match) leaves
 * every layer empty (len 0), never with its old length over overwritten rows. */
int32_t skv_hot_match_restore(skv_hot *hot, skv_stream stream, const uint8_t root[32],
                              const uint64_t *tokens, size_t n_tokens, skv_layer *const *layers,
                              size_t n_layers, void *const *state_ptrs, const size_t *state_bytes,
                              size_t n_states, size_t *reused_tokens, uint8_t hash_out[32]);
/* evict_prefix_block (src/serve/state.rs:644-646). */
int32_t skv_hot_evict_lru(skv_hot *hot, int32_t *found, size_t *bytes);
size_t skv_hot_block_tokens(const skv_hot *hot);
size_t skv_hot_len(const skv_hot *hot);
/* prefix_cache_bytes (src/serve/state.rs:640-642). */
size_t skv_hot_bytes(const skv_hot *hot);
size_t skv_hot_free_blocks(const skv_hot *hot);
size_t skv_hot_pool_blocks(const skv_hot *hot);
size_t skv_hot_block_bytes(const skv_hot *hot);
uint64_t skv_hot_evictions(const skv_hot *hot);
uint64_t skv_hot_skipped(const skv_hot *hot);
int32_t skv_hot_entry(const skv_hot *hot, size_t index, uint8_t session[32], uint8_t hash[32],
                      size_t *tokens, size_t *bytes);

/* ---- the decoder's own whole-prompt cache: prefix_cache_get / prefix_cache_put ------------ */

/* A few whole prompts, most recent first, each with the K/V rows of every layer and the model's
 * opaque state buffers (final hidden state, recurrent states) as device snapshots
 * (PrefixCacheEntry, src/decoder/generation.rs:175-188). capacity 0 = disabled: put is a no-op. */
typedef struct skv_prompt_cache skv_prompt_cache;
int32_t skv_prompt_cache_create(skv_ctx *ctx, size_t capacity, skv_prompt_cache **out);
/* capacity = RETI_RUST_PREFIX_CACHE_CAP (default 4), or 0 when RETI_RUST_PREFIX_CACHE=0
 * (src/runtime_flags.rs:665-678). */
int32_t skv_prompt_cache_from_runtime_flags(skv_ctx *ctx, skv_prompt_cache **out);
void skv_prompt_cache_destroy(skv_prompt_cache *cache);
size_t skv_prompt_cache_len(const skv_prompt_cache *cache);
size_t skv_prompt_cache_capacity(const skv_prompt_cache *cache);
size_t skv_prompt_cache_bytes(const skv_prompt_cache *cache);
/* Entry `index` in recency order (0 = most recent): *n_tokens and, if tokens_out is not null,
 * its first min(tokens_cap, *n_tokens) tokens. The tests' view of the entries. */
int32_t skv_prompt_cache_entry(const skv_prompt_cache *cache, size_t index, size_t *n_tokens,
                               uint64_t *tokens_out, size_t tokens_cap);
/* prefix_cache_put (generation.rs:3105-3139): a deep copy of rows [0, n_tokens) of every layer
 * (each layer's len must be n_tokens) and of the n_states state buffers, keyed by the prompt's
 * tokens; an entry with the same tokens is replaced, the new entry is the most recent, the
 * least recent ones beyond the capacity are dropped. Async on `stream`; dropping an entry waits
 * for the device before its memory is freed. Of a ring layer (window > 0) whose prompt is
 * longer than the ring, the entry holds the pages the ring still holds (the reference clones
 * the whole cache, but its sliding layers never attend the older rows again); a hit restores
 * them into ring layers only, with the oldest kept row as the layer's floor. */
int32_t skv_prompt_cache_put(skv_prompt_cache *cache, skv_stream stream, const uint64_t *tokens,
                             size_t n_tokens, skv_layer *const *layers, size_t n_layers,
                             const void *const *state_ptrs, const size_t *state_bytes, size_t n_states);
/* prefix_cache_get (generation.rs:2998-3025) up to the point where the model runs: the longest
 * entry whose tokens `prompt` starts with (longest_prefix_entry_index, generation.rs:190-204)
 * becomes the most recent one, its rows are copied into rows [0, *cached_tokens) of the layers
 * (len set to it), its state buffers into state_ptrs. *cached_tokens = 0 on a miss (layers
 * untouched). When *cached_tokens < n_prompt the caller extends the layers with the suffix and
 * puts the whole prompt (generation.rs:3016-3019). Every check precedes the first copy. */
int32_t skv_prompt_cache_get(skv_prompt_cache *cache, skv_stream stream, const uint64_t *prompt,
                             size_t n_prompt, skv_layer *const *layers, size_t n_layers,
                             void *const *state_ptrs, const size_t *state_bytes, size_t n_states,
                             size_t *cached_tokens);

#ifdef __cplusplus
}
#endif
#endif /* SARAGOSSA_KV_H */
