/*
 * CPU oracle for the KV-cache hot path: a plain-C restatement of the
 * reference's CPU algorithms, built with strict IEEE flags
 * (-O2 -ffp-contract=off -fno-fast-math).
 *
 * THIS IS TEST INFRASTRUCTURE. Only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may load it. The product library never
 * links, loads or calls anything in this file.
 *
 * Every function cites the reference file:line it follows. The reference is
 * Rust; f32::{exp,powf,sin,cos,sqrt} lower to the platform libm, which is the
 * same expf/powf/sinf/cosf/sqrtf called here, and rustc neither contracts nor
 * re-associates float operations, so sums below are kept strictly sequential.
 *
 * Pinning status of each function (what the tests check it against):
 *   skvo_f32_to_bf16_bits / skvo_bf16_round   closed form + reference known answers
 *                                             (src/decoder/tests.rs:13-25) + torch bfloat16
 *   skvo_cache_*                               reference fixtures with explicit arithmetic data
 *                                             (src/decode_resident/tests.rs:380-525)
 *   skvo_softmax_in_place, skvo_softmax        closed forms (uniform fallback, single key)
 *   skvo_cached_attention_one                  two-key closed form, window == truncated cache,
 *                                             len 1 == V row, fp64 textbook attention, torch SDPA
 *   skvo_causal_attention                      equality with the cached path row by row, fp64 bound
 *   skvo_cached_attention_prefill_rows         definitionally append + attention per row
 *   skvo_rms_norm_rope_heads_at / apply_rope   MLX-captured constants (src/decoder/tests.rs:998-1113)
 *   skvo_split_attention_gate, skvo_attention_gate   index identity against a reshape; sigmoid(0) = 1/2,
 *                                             sigmoid(x) + sigmoid(-x) = 1, fp64 formula to one ulp
 *   skvo_sdpa_2pass_blocks, skvo_window_start  integer closed forms from the reference's comments
 * The last-ulp value of the float functions on large random inputs is pinned
 * only by the same-libm/no-contraction argument above: parity unpinned beyond
 * the checks listed.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>

#define SKVO_OK 0
#define SKVO_ERR_DIMENSION 1
#define SKVO_ERR_CONFIG 2

#define SKVO_ROPE_HALVES 0
#define SKVO_ROPE_INTERLEAVED 1

/* ---- bf16 rounding ------------------------------------------------------ */

/* src/decode_resident/utils.rs:55-60 — round-to-nearest-even on the raw bits,
 * wrapping add, no NaN special case. */
uint16_t skvo_f32_to_bf16_bits(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    uint32_t lsb = (bits >> 16) & 1u;
    uint32_t rounded = bits + (0x7fffu + lsb); /* unsigned add wraps */
    return (uint16_t)(rounded >> 16);
}

/* src/decode_resident/utils.rs:230-232 and src/decoder.rs:1629-1633 */
float skvo_bf16_round(float value) {
    uint32_t bits = ((uint32_t)skvo_f32_to_bf16_bits(value)) << 16;
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

void skvo_bf16_round_array(const float *in, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = skvo_bf16_round(in[i]);
}

void skvo_f32_to_bf16_bits_array(const float *in, uint16_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = skvo_f32_to_bf16_bits(in[i]);
}

/* ---- LayerKvCache (src/decoder.rs:671-697) ------------------------------ */

typedef struct skvo_cache {
    float *keys;
    float *values;
    size_t keys_len;   /* elements, like Vec::len */
    size_t values_len;
    size_t cap;        /* allocated elements for each of keys / values */
    int has_kv_dim;    /* Option<usize> */
    size_t kv_dim;
    int round_k;       /* oracle mode BF16R: round at append, the reference's */
    int round_v;       /* own bf16 convention (src/decode_resident/tests.rs:1462-1472) */
} skvo_cache;

skvo_cache *skvo_cache_new(void) {
    return (skvo_cache *)calloc(1, sizeof(skvo_cache));
}

void skvo_cache_free(skvo_cache *c) {
    if (!c) return;
    free(c->keys);
    free(c->values);
    free(c);
}

/* Mode BF16R switch: K and/or V elements pass through bf16_round when appended
 * (same effect as RETI_RUST_KV_BF16_SIM_KONLY / _VONLY at seed,
 * src/decode_resident/utils.rs:245-256, extended to both tensors). */
void skvo_cache_set_bf16_round(skvo_cache *c, int round_k, int round_v) {
    c->round_k = round_k;
    c->round_v = round_v;
}

/* Clone for LayerKvCache (src/decoder.rs:686-697): deep copy of both vectors. */
skvo_cache *skvo_cache_clone(const skvo_cache *c) {
    skvo_cache *n = skvo_cache_new();
    if (!n) return NULL;
    *n = *c;
    n->cap = c->keys_len > c->values_len ? c->keys_len : c->values_len;
    n->keys = NULL;
    n->values = NULL;
    if (n->cap) {
        n->keys = (float *)malloc(n->cap * sizeof(float));
        n->values = (float *)malloc(n->cap * sizeof(float));
        if (!n->keys || !n->values) {
            skvo_cache_free(n);
            return NULL;
        }
        memcpy(n->keys, c->keys, c->keys_len * sizeof(float));
        memcpy(n->values, c->values, c->values_len * sizeof(float));
    }
    return n;
}

static int skvo_cache_reserve(skvo_cache *c, size_t extra) {
    size_t need = c->keys_len + extra;
    if (need <= c->cap) return 0;
    size_t cap = c->cap ? c->cap : 1024;
    while (cap < need) cap *= 2; /* amortised growth, like Vec */
    float *k = (float *)realloc(c->keys, cap * sizeof(float));
    if (!k) return -1;
    c->keys = k;
    float *v = (float *)realloc(c->values, cap * sizeof(float));
    if (!v) return -1;
    c->values = v;
    c->cap = cap;
    return 0;
}

static int skvo_cache_extend(skvo_cache *c, const float *key, const float *value, size_t n) {
    if (skvo_cache_reserve(c, n)) return SKVO_ERR_CONFIG;
    if (c->round_k) skvo_bf16_round_array(key, c->keys + c->keys_len, n);
    else memcpy(c->keys + c->keys_len, key, n * sizeof(float));
    if (c->round_v) skvo_bf16_round_array(value, c->values + c->values_len, n);
    else memcpy(c->values + c->values_len, value, n * sizeof(float));
    c->keys_len += n;
    c->values_len += n;
    return SKVO_OK;
}

/* LayerKvCache::append (src/decoder/attention_cache.rs:7-36). */
int skvo_cache_append(skvo_cache *c, const float *key, size_t key_rows, size_t key_dim,
                      const float *value, size_t value_rows, size_t value_dim,
                      size_t kv_heads, size_t head_dim) {
    size_t expected_dim = kv_heads * head_dim;
    if (key_rows != 1 || value_rows != 1 || key_dim != expected_dim || value_dim != expected_dim)
        return SKVO_ERR_DIMENSION;
    if (c->has_kv_dim) {
        if (c->kv_dim != expected_dim) return SKVO_ERR_DIMENSION;
    } else {
        c->has_kv_dim = 1;
        c->kv_dim = expected_dim;
    }
    return skvo_cache_extend(c, key, value, expected_dim);
}

/* LayerKvCache::append_batch (src/decoder/attention_cache.rs:38-70). */
int skvo_cache_append_batch(skvo_cache *c, const float *key, size_t key_rows, size_t key_dim,
                            const float *value, size_t value_rows, size_t value_dim,
                            size_t kv_heads, size_t head_dim) {
    size_t expected_dim = kv_heads * head_dim;
    if (key_rows == 0 || key_rows != value_rows || key_dim != expected_dim ||
        value_dim != expected_dim)
        return SKVO_ERR_DIMENSION;
    if (c->has_kv_dim) {
        if (c->kv_dim != expected_dim) return SKVO_ERR_DIMENSION;
    } else {
        c->has_kv_dim = 1;
        c->kv_dim = expected_dim;
    }
    return skvo_cache_extend(c, key, value, key_rows * expected_dim);
}

/* LayerKvCache::len (src/decoder/attention_cache.rs:72-77). */
size_t skvo_cache_len(const skvo_cache *c) {
    if (c->has_kv_dim && c->kv_dim > 0) return c->keys_len / c->kv_dim;
    return 0;
}

/* LayerKvCache::truncate (src/decoder/attention_cache.rs:79-100). */
int skvo_cache_truncate(skvo_cache *c, size_t len) {
    if (!c->has_kv_dim) return len == 0 ? SKVO_OK : SKVO_ERR_DIMENSION;
    size_t new_len;
    if (__builtin_mul_overflow(len, c->kv_dim, &new_len)) return SKVO_ERR_DIMENSION;
    if (new_len > c->keys_len || new_len > c->values_len) return SKVO_ERR_DIMENSION;
    c->keys_len = new_len;
    c->values_len = new_len;
    return SKVO_OK;
}

const float *skvo_cache_keys(const skvo_cache *c) { return c->keys; }
const float *skvo_cache_values(const skvo_cache *c) { return c->values; }
size_t skvo_cache_kv_dim(const skvo_cache *c) { return c->has_kv_dim ? c->kv_dim : 0; }
int skvo_cache_has_kv_dim(const skvo_cache *c) { return c->has_kv_dim; }
/* estimated_cpu_bytes of one layer (src/decoder.rs:725-737), KV part. */
size_t skvo_cache_estimated_bytes(const skvo_cache *c) {
    return (c->keys_len + c->values_len) * sizeof(float);
}

/* ---- attention ---------------------------------------------------------- */

/* AttentionLayout (src/decoder/attention_ops.rs:526-585). sliding_window 0 == None
 * (the reference filters window > 0). */
typedef struct skvo_layout {
    size_t num_attention_heads;
    size_t num_key_value_heads;
    size_t head_dim;
    size_t rope_dims;
    float attn_scalar;
    size_t sliding_window;
} skvo_layout;

/* attention_layout (src/decoder/attention_ops.rs:526-585): head_dim 0 means
 * "not given" (derive from q_dim); rope_dims 0 means "not given" (= head_dim);
 * attn_scalar <= 0 means "not given" (= head_dim). explicit_zero_head_dim
 * reproduces Some(0). */
int skvo_attention_layout(size_t q_dim, size_t k_dim, size_t v_dim, size_t q_heads,
                          size_t kv_heads, size_t head_dim_opt, int head_dim_given,
                          size_t rope_dims_opt, int rope_dims_given, float attn_scalar_opt,
                          int attn_scalar_given, size_t sliding_window, skvo_layout *out) {
    if (q_heads == 0 || kv_heads == 0) return SKVO_ERR_DIMENSION;
    if (q_heads % kv_heads != 0) return SKVO_ERR_DIMENSION;
    size_t head_dim;
    if (head_dim_given) {
        if (head_dim_opt == 0) return SKVO_ERR_DIMENSION;
        head_dim = head_dim_opt;
    } else {
        head_dim = q_dim / q_heads;
    }
    if (q_dim != q_heads * head_dim) return SKVO_ERR_DIMENSION;
    size_t expected_kv_dim = kv_heads * head_dim;
    if (k_dim != expected_kv_dim || v_dim != expected_kv_dim) return SKVO_ERR_DIMENSION;
    size_t rope_dims = rope_dims_given ? rope_dims_opt : head_dim;
    if (rope_dims == 0 || rope_dims > head_dim || rope_dims % 2 != 0) return SKVO_ERR_DIMENSION;
    out->num_attention_heads = q_heads;
    out->num_key_value_heads = kv_heads;
    out->head_dim = head_dim;
    out->rope_dims = rope_dims;
    out->attn_scalar = attn_scalar_given ? attn_scalar_opt : (float)head_dim;
    out->sliding_window = sliding_window;
    return SKVO_OK;
}

/* attention_parallel_threshold (src/runtime_flags.rs:641-649), default 128. */
static size_t g_par_threshold = 128;
void skvo_set_attention_parallel_threshold(size_t t) { g_par_threshold = t; }
size_t skvo_attention_parallel_threshold(void) { return g_par_threshold; }

/* dot_product (src/decoder/attention_ops.rs:1040-1046): index loop, separate
 * multiply and add. */
float skvo_dot_product(const float *left, const float *right, size_t n) {
    float sum = 0.0f;
    for (size_t idx = 0; idx < n; ++idx) sum += left[idx] * right[idx];
    return sum;
}

/* f32::max(a, b): returns the non-NaN operand if one is NaN. */
static inline float rust_f32_max(float a, float b) { return fmaxf(a, b); }

/* softmax_in_place (src/decoder/attention_ops.rs:1019-1038). */
void skvo_softmax_in_place(float *values, size_t n, float temperature) {
    temperature = rust_f32_max(temperature, 0.0001f);
    float max = -INFINITY;
    for (size_t i = 0; i < n; ++i) max = rust_f32_max(max, values[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        values[i] = expf((values[i] - max) / temperature);
        sum += values[i];
    }
    if (sum <= FLT_EPSILON) {
        float uniform = 1.0f / (float)n;
        for (size_t i = 0; i < n; ++i) values[i] = uniform;
        return;
    }
    for (size_t i = 0; i < n; ++i) values[i] /= sum;
}

/* softmax (src/sampling.rs:133-153): same arithmetic, out of place. */
void skvo_softmax(const float *logits, size_t n, float temperature, float *out) {
    temperature = rust_f32_max(temperature, 0.0001f);
    float max = -INFINITY;
    for (size_t i = 0; i < n; ++i) max = rust_f32_max(max, logits[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        float value = expf((logits[i] - max) / temperature);
        sum += value;
        out[i] = value;
    }
    if (sum <= FLT_EPSILON) {
        for (size_t i = 0; i < n; ++i) out[i] = 1.0f / (float)n;
        return;
    }
    for (size_t i = 0; i < n; ++i) out[i] /= sum;
}

/* One query head of cached_attention_one: the closure body at
 * src/decoder/attention_ops.rs:931-949 (and the serial twin at 955-971). */
static void attention_one_head(const float *q_row, const float *keys, const float *values,
                               const skvo_layout *layout, size_t q_head, size_t window_start,
                               size_t window_len, float inv_scale, float *scores,
                               float *out_head) {
    size_t head_dim = layout->head_dim;
    size_t expected_kv_dim = layout->num_key_value_heads * head_dim;
    size_t kv_group = layout->num_attention_heads / layout->num_key_value_heads;
    size_t kv_head = q_head / kv_group;
    size_t q_start = q_head * head_dim;
    size_t k_start = kv_head * head_dim;
    const float *q_slice = q_row + q_start;
    for (size_t offset = 0; offset < window_len; ++offset) {
        size_t key_start = (window_start + offset) * expected_kv_dim + k_start;
        scores[offset] = skvo_dot_product(q_slice, keys + key_start, head_dim) * inv_scale;
    }
    skvo_softmax_in_place(scores, window_len, 1.0f);
    for (size_t offset = 0; offset < window_len; ++offset) {
        float prob = scores[offset];
        size_t value_start = (window_start + offset) * expected_kv_dim + k_start;
        const float *v_slice = values + value_start;
        for (size_t col = 0; col < head_dim; ++col) out_head[col] += prob * v_slice[col];
    }
}

/* cached_attention_one (src/decoder/attention_ops.rs:889-974). `threads` is the
 * size of the worker pool used once cache_len reaches the parallel threshold
 * (rayon par_chunks_mut per head in the reference); the result does not depend
 * on it because each head is computed by exactly one worker. */
int skvo_cached_attention_one(const float *q, size_t q_rows, size_t q_dim, const skvo_cache *cache,
                              const skvo_layout *layout, float *out, int threads) {
    size_t expected_q_dim = layout->num_attention_heads * layout->head_dim;
    size_t expected_kv_dim = layout->num_key_value_heads * layout->head_dim;
    if (q_rows != 1 || q_dim != expected_q_dim || !cache->has_kv_dim ||
        cache->kv_dim != expected_kv_dim)
        return SKVO_ERR_DIMENSION;
    size_t cache_len = skvo_cache_len(cache);
    if (cache_len == 0 || cache->keys_len != cache->values_len) return SKVO_ERR_DIMENSION;

    float inv_scale = 1.0f / sqrtf(layout->attn_scalar);
    size_t window_start = 0;
    if (layout->sliding_window > 0)
        window_start = cache_len > layout->sliding_window ? cache_len - layout->sliding_window : 0;
    size_t window_len = cache_len - window_start;
    size_t heads = layout->num_attention_heads;
    for (size_t i = 0; i < expected_q_dim; ++i) out[i] = 0.0f;

    if (cache_len >= g_par_threshold && threads > 1) {
        int failed = 0;
#pragma omp parallel num_threads(threads)
        {
            float *scores = (float *)malloc(window_len * sizeof(float));
            if (!scores) {
#pragma omp atomic write
                failed = 1;
            }
#pragma omp barrier
            if (!failed) {
#pragma omp for schedule(dynamic, 1)
                for (long q_head = 0; q_head < (long)heads; ++q_head)
                    attention_one_head(q, cache->keys, cache->values, layout, (size_t)q_head,
                                       window_start, window_len, inv_scale, scores,
                                       out + (size_t)q_head * layout->head_dim);
            }
            free(scores);
        }
        return failed ? SKVO_ERR_CONFIG : SKVO_OK;
    }
    float *scores = (float *)malloc(window_len * sizeof(float));
    if (!scores) return SKVO_ERR_CONFIG;
    for (size_t q_head = 0; q_head < heads; ++q_head)
        attention_one_head(q, cache->keys, cache->values, layout, q_head, window_start,
                           window_len, inv_scale, scores, out + q_head * layout->head_dim);
    free(scores);
    return SKVO_OK;
}

/* cached_attention_prefill_rows (src/decoder/attention_ops.rs:976-1017), CPU
 * branch: for each row append then cached_attention_one. */
int skvo_cached_attention_prefill_rows(const float *q, const float *k, const float *v, size_t seq,
                                       size_t q_dim, size_t k_dim, size_t v_dim, skvo_cache *cache,
                                       const skvo_layout *layout, float *out, int threads) {
    size_t expected_q_dim = layout->num_attention_heads * layout->head_dim;
    size_t expected_kv_dim = layout->num_key_value_heads * layout->head_dim;
    if (seq == 0 || q_dim != expected_q_dim || k_dim != expected_kv_dim ||
        v_dim != expected_kv_dim)
        return SKVO_ERR_DIMENSION;
    for (size_t pos = 0; pos < seq; ++pos) {
        int rc = skvo_cache_append(cache, k + pos * k_dim, 1, k_dim, v + pos * v_dim, 1, v_dim,
                                   layout->num_key_value_heads, layout->head_dim);
        if (rc) return rc;
        rc = skvo_cached_attention_one(q + pos * q_dim, 1, q_dim, cache, layout,
                                       out + pos * expected_q_dim, threads);
        if (rc) return rc;
    }
    return SKVO_OK;
}

/* causal_attention (src/decoder/attention_ops.rs:1052-1116): first-chunk prefill.
 * Divides by sqrt(attn_scalar) where the cached path multiplies by the
 * reciprocal, and uses the out-of-place softmax of src/sampling.rs. */
int skvo_causal_attention(const float *q, const float *k, const float *v, size_t seq,
                          size_t q_dim, size_t k_dim, size_t v_dim, const skvo_layout *layout,
                          float *out) {
    size_t head_dim = layout->head_dim;
    size_t expected_q_dim = layout->num_attention_heads * head_dim;
    size_t expected_kv_dim = layout->num_key_value_heads * head_dim;
    if (q_dim != expected_q_dim || k_dim != expected_kv_dim || v_dim != expected_kv_dim)
        return SKVO_ERR_DIMENSION;
    float scale = sqrtf(layout->attn_scalar);
    size_t kv_group = layout->num_attention_heads / layout->num_key_value_heads;
    for (size_t i = 0; i < seq * expected_q_dim; ++i) out[i] = 0.0f;
    float *scores = (float *)malloc((seq ? seq : 1) * sizeof(float));
    float *probs = (float *)malloc((seq ? seq : 1) * sizeof(float));
    if (!scores || !probs) {
        free(scores);
        free(probs);
        return SKVO_ERR_CONFIG;
    }
    for (size_t pos = 0; pos < seq; ++pos) {
        const float *q_row = q + pos * q_dim;
        size_t window_start = 0;
        if (layout->sliding_window > 0)
            window_start = (pos + 1) > layout->sliding_window ? (pos + 1) - layout->sliding_window : 0;
        for (size_t q_head = 0; q_head < layout->num_attention_heads; ++q_head) {
            size_t kv_head = q_head / kv_group;
            size_t q_start = q_head * head_dim;
            const float *q_slice = q_row + q_start;
            size_t n = 0;
            for (size_t row = window_start; row <= pos; ++row) {
                const float *k_slice = k + row * k_dim + kv_head * head_dim;
                /* iter().zip().map(a*b).sum::<f32>() folds from 0.0 in order */
                float dot = 0.0f;
                for (size_t c = 0; c < head_dim; ++c) dot += q_slice[c] * k_slice[c];
                scores[n++] = dot / scale;
            }
            skvo_softmax(scores, n, 1.0f, probs);
            for (size_t offset = 0; offset < n; ++offset) {
                const float *v_slice = v + (window_start + offset) * v_dim + kv_head * head_dim;
                float prob = probs[offset];
                float *o = out + pos * expected_q_dim + q_start;
                for (size_t col = 0; col < head_dim; ++col) o[col] += prob * v_slice[col];
            }
        }
    }
    free(scores);
    free(probs);
    return SKVO_OK;
}

/* ---- RMSNorm + RoPE ----------------------------------------------------- */

/* rope_rotations (src/decoder/attention_ops.rs:848-887), without the memo
 * (a pure cache keyed on all inputs). */
static void rope_rotations(size_t position, size_t rope_dims, float theta, float position_scale,
                           size_t frequency_dim, float *cos_out, float *sin_out) {
    size_t pairs = rope_dims / 2;
    float scaled_position = (float)position * position_scale;
    for (size_t pair = 0; pair < pairs; ++pair) {
        float exponent = (float)(2 * pair) / (float)frequency_dim;
        float angle = scaled_position / powf(theta, exponent);
        cos_out[pair] = cosf(angle);
        sin_out[pair] = sinf(angle);
    }
}

static void rotate_head(float *out, size_t head_start, size_t pairs, const float *cosv,
                        const float *sinv, int style) {
    if (style == SKVO_ROPE_INTERLEAVED) {
        for (size_t pair = 0; pair < pairs; ++pair) {
            float even = out[head_start + 2 * pair];
            float odd = out[head_start + 2 * pair + 1];
            out[head_start + 2 * pair] = even * cosv[pair] - odd * sinv[pair];
            out[head_start + 2 * pair + 1] = even * sinv[pair] + odd * cosv[pair];
        }
    } else {
        for (size_t pair = 0; pair < pairs; ++pair) {
            size_t first_index = head_start + pair;
            size_t second_index = head_start + pairs + pair;
            float first = out[first_index];
            float second = out[second_index];
            out[first_index] = first * cosv[pair] - second * sinv[pair];
            out[second_index] = first * sinv[pair] + second * cosv[pair];
        }
    }
}

/* rms_norm_rope_heads_at (src/decoder/attention_ops.rs:682-777). */
int skvo_rms_norm_rope_heads_at(const float *x, size_t seq, size_t heads, size_t head_dim,
                                size_t rope_dims, const float *weight, float eps, float theta,
                                float position_scale, size_t frequency_dim,
                                size_t position_offset, int style, float *out) {
    if (heads == 0 || head_dim == 0) return SKVO_ERR_DIMENSION;
    if (rope_dims == 0 || rope_dims > head_dim || rope_dims % 2 != 0) return SKVO_ERR_DIMENSION;
    size_t dim = heads * head_dim;
    size_t pairs = rope_dims / 2;
    float *cosv = (float *)malloc(pairs * sizeof(float));
    float *sinv = (float *)malloc(pairs * sizeof(float));
    if (!cosv || !sinv) {
        free(cosv);
        free(sinv);
        return SKVO_ERR_CONFIG;
    }
    for (size_t pos = 0; pos < seq; ++pos) {
        rope_rotations(position_offset + pos, rope_dims, theta, position_scale, frequency_dim,
                       cosv, sinv);
        size_t row_start = pos * dim;
        for (size_t head = 0; head < heads; ++head) {
            size_t head_start = row_start + head * head_dim;
            const float *xs = x + head_start;
            float sum = 0.0f;
            for (size_t c = 0; c < head_dim; ++c) sum += xs[c] * xs[c];
            float mean_square = sum / (float)head_dim;
            float inv_rms = 1.0f / sqrtf(mean_square + eps);
            for (size_t col = 0; col < head_dim; ++col)
                out[head_start + col] = xs[col] * inv_rms * weight[col];
            rotate_head(out, head_start, pairs, cosv, sinv, style);
        }
    }
    free(cosv);
    free(sinv);
    return SKVO_OK;
}

/* apply_rope_heads_at (src/decoder/attention_ops.rs:779-834). */
int skvo_apply_rope_heads_at(const float *x, size_t seq, size_t heads, size_t head_dim,
                             size_t rope_dims, float theta, float position_scale,
                             size_t frequency_dim, size_t position_offset, int style, float *out) {
    if (theta <= 0.0f) return SKVO_ERR_DIMENSION;
    size_t dim = heads * head_dim;
    size_t pairs = rope_dims / 2;
    float *cosv = (float *)malloc((pairs ? pairs : 1) * sizeof(float));
    float *sinv = (float *)malloc((pairs ? pairs : 1) * sizeof(float));
    if (!cosv || !sinv) {
        free(cosv);
        free(sinv);
        return SKVO_ERR_CONFIG;
    }
    memcpy(out, x, seq * dim * sizeof(float));
    for (size_t pos = 0; pos < seq; ++pos) {
        rope_rotations(position_offset + pos, rope_dims, theta, position_scale, frequency_dim,
                       cosv, sinv);
        for (size_t head = 0; head < heads; ++head)
            rotate_head(out, pos * dim + head * head_dim, pairs, cosv, sinv, style);
    }
    free(cosv);
    free(sinv);
    return SKVO_OK;
}

/* ---- output gate --------------------------------------------------------- */

/* split_attention_gate (src/decoder/attention_ops.rs:486-520): the gated q projection
 * holds, per head, head_dim query values then head_dim gate values. */
int skvo_split_attention_gate(const float *q_projection, size_t rows, size_t cols, size_t heads,
                              size_t head_dim, float *q, float *gate) {
    size_t q_dim = heads * head_dim;
    if (heads == 0 || head_dim == 0 || cols != 2 * q_dim) return SKVO_ERR_DIMENSION;
    for (size_t row = 0; row < rows; ++row) {
        const float *source = q_projection + row * cols;
        for (size_t head = 0; head < heads; ++head) {
            size_t start = head * 2 * q_dim / heads;
            memcpy(q + row * q_dim + head * head_dim, source + start, head_dim * sizeof(float));
            memcpy(gate + row * q_dim + head * head_dim, source + start + head_dim,
                   head_dim * sizeof(float));
        }
    }
    return SKVO_OK;
}

/* sigmoid_scalar (src/decoder/attention_ops.rs:522-524). */
float skvo_sigmoid(float value) { return 1.0f / (1.0f + expf(-value)); }

/* context.mul_elementwise(gate.map(sigmoid_scalar)) (src/decoder/attention_ops.rs:217-219). */
void skvo_attention_gate(const float *context, const float *gate, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) out[i] = context[i] * skvo_sigmoid(gate[i]);
}

/* ---- integer policy helpers --------------------------------------------- */

/* sdpa_2pass_blocks (src/decode_resident/utils.rs:282-286). */
size_t skvo_sdpa_2pass_blocks(size_t len) {
    size_t raw = len / 128;
    if (raw < 1) raw = 1;
    size_t rounded = (raw + 31) / 32 * 32;
    if (rounded < 32) rounded = 32;
    if (rounded > 1024) rounded = 1024;
    return rounded;
}

/* resident_windowed_full_attn_layer_dims (src/decoder/resident/types.rs:13-18):
 * window_start = (position + 1).saturating_sub(window); window 0 == no window. */
size_t skvo_window_start(size_t position, size_t window) {
    if (window == 0) return 0;
    return (position + 1) > window ? (position + 1) - window : 0;
}

/* Resident capacity rule (src/decoder/resident/setup.rs:322-329); returns
 * SKVO_ERR_DIMENSION on overflow. */
int skvo_resident_capacity(size_t prefill_len, size_t max_new_tokens, size_t draft_headroom,
                           size_t *out) {
    size_t a, b;
    if (__builtin_add_overflow(prefill_len, max_new_tokens, &a)) return SKVO_ERR_DIMENSION;
    if (__builtin_add_overflow(a, draft_headroom, &b)) return SKVO_ERR_DIMENSION;
    *out = b;
    return SKVO_OK;
}

/* ---- CPU baseline helpers (timed by the benchmark's cpu_baseline leg) ---- */

/* One decode step of the reference CPU path for one layer: append one row,
 * then cached_attention_one (src/decoder/attention_ops.rs:223-322 calls
 * attention_cache.rs:7-36 then attention_ops.rs:889-974). */
int skvo_decode_step(skvo_cache *cache, const float *k_row, const float *v_row, const float *q,
                     const skvo_layout *layout, float *out, int threads) {
    size_t kv_dim = layout->num_key_value_heads * layout->head_dim;
    size_t q_dim = layout->num_attention_heads * layout->head_dim;
    int rc = skvo_cache_append(cache, k_row, 1, kv_dim, v_row, 1, kv_dim,
                               layout->num_key_value_heads, layout->head_dim);
    if (rc) return rc;
    return skvo_cached_attention_one(q, 1, q_dim, cache, layout, out, threads);
}
