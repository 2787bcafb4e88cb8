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
 * (block_table[r / 16], r % 16) here. Elements are bf16, rounded from f32 with
 * the reference's integer formula (src/decode_resident/utils.rs:55-60).
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

#define SKV_DTYPE_F32 0  /* GpuElement::F32 — not built; skv_layer_create rejects it */
#define SKV_DTYPE_BF16 1 /* GpuElement::Bf16 */

#define SKV_PAGE_ROWS 16

typedef struct skv_ctx skv_ctx;
typedef struct skv_layer skv_layer;
typedef struct skv_snapshot skv_snapshot;
typedef struct skv_prefix skv_prefix;
typedef struct skv_hot skv_hot;

/* A stream argument is a hipStream_t passed as void*; NULL is the default stream. */
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
int32_t skv_flag_decode_resident_full(void);      /* RETI_RUST_DECODE_RESIDENT_FULL, runtime_flags.rs:283-286 */
int32_t skv_flag_decode_resident(void);           /* RETI_RUST_DECODE_RESIDENT, runtime_flags.rs:266-269 */
int32_t skv_flag_serve_prefix_cache_enabled(void);   /* RETI_SERVE_PREFIX_CACHE, runtime_flags.rs:681-684 */
size_t skv_flag_serve_prefix_block_tokens(void);     /* runtime_flags.rs:727-736 */
size_t skv_flag_serve_prefix_cache_blocks(void);     /* runtime_flags.rs:739-747 */
size_t skv_flag_serve_prefix_blocks_per_session(void); /* runtime_flags.rs:750-758 */
int32_t skv_flag_prefix_cache_enabled(void);      /* RETI_RUST_PREFIX_CACHE, runtime_flags.rs:665-668 */
size_t skv_flag_prefix_cache_capacity(void);      /* RETI_RUST_PREFIX_CACHE_CAP, runtime_flags.rs:670-678 */
size_t skv_flag_prefill_chunk(void);              /* RETI_RUST_PREFILL_CHUNK (alias _STEP_SIZE), runtime_flags.rs:414-423 */
/* The reference freezes each flag at first read (OnceLock). This re-reads the
 * environment; it exists for tests only. */
void skv_flags_reload(void);
/* window_start of a sliding layer (src/decoder/resident/types.rs:13-18); window 0 = none. */
size_t skv_window_start(size_t position, size_t window);
/* f32 -> bf16 bits, the reference's formula (src/decode_resident/utils.rs:55-60). Host helper. */
uint16_t skv_f32_to_bf16_bits(float value);

/* ---- context ------------------------------------------------------------ */

/* DecodeResidentState::new(device) (src/decoder/resident/setup.rs:237, 675). */
int32_t skv_ctx_create(int32_t device, skv_ctx **out);
void skv_ctx_destroy(skv_ctx *ctx);
/* Blocks until everything queued on the context's own stream has finished. */
int32_t skv_ctx_synchronize(skv_ctx *ctx);

/* ---- one layer's cache: FullAttentionMetalState -------------------------- */

/* DecodeResidentState::full_attention_with_element (src/decode_resident/attention.rs:56-108).
 * Rejects a zero dimension and q_heads % kv_heads != 0 with SKV_ERR_CONFIG.
 * `window` > 0 makes the layer a ring buffer that keeps the last `window` rows
 * (rounded up to whole pages); 0 keeps all `capacity` rows in pages. */
int32_t skv_layer_create(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads,
                         size_t head_dim, int32_t dtype, size_t window, skv_layer **out);
/* full_attention(capacity, q_heads, kv_heads, head_dim, sampled) (attention.rs:26-45):
 * element type from skv_flag_kv_bf16_for(sampled). */
int32_t skv_layer_create_for(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads,
                             size_t head_dim, int32_t sampled, skv_layer **out);
void skv_layer_destroy(skv_layer *layer);

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
 * encodes back to back). window_start is derived from the layer's window. */
int32_t skv_decode_step_device(skv_layer *layer, skv_stream stream, const void *k_dev,
                               size_t k_off, const void *v_dev, size_t v_off, const float *q_dev,
                               float *out_dev);

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
 * (tests.rs:423-428, 469-476). Synchronous. */
int32_t skv_read_rows(skv_layer *layer, size_t first, size_t n, uint16_t *k_out, uint16_t *v_out);
/* Same gather, device to device, async on `stream`. */
int32_t skv_gather_device(skv_layer *layer, skv_stream stream, size_t first, size_t n,
                          void *k_dst_dev, void *v_dst_dev);

#ifdef __cplusplus
}
#endif
#endif /* SARAGOSSA_KV_H */
