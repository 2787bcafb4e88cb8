/* A plain C11 client of include/saragossa_kv.h, linked against libsaragossa_kv.so the way a
 * foreign-function binding would be: no C++, no Python, no torch. It seeds a paged cache
 * through a permuted block table, appends rows from host memory, reads the contents back
 * (bit-exact against the reference's f32 -> bf16 formula) and checks decode attention,
 * with and without a window start, against a double-precision softmax attention computed
 * here over the same bf16-rounded rows (textbook formula of cached_attention_one,
 * src/decoder/attention_ops.rs:889-974). Error paths: overflow at capacity, empty window,
 * a bad GQA ratio. Then the same on a layer with the f32 element, whose rows come back
 * verbatim. Prints "ok" and exits 0 when everything holds. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "saragossa_kv.h"

#define CHECK(cond, ...)                                                      \
    do {                                                                      \
        if (!(cond)) {                                                        \
            fprintf(stderr, "kv_c_client: " __VA_ARGS__);                     \
            fprintf(stderr, " [last error: %s]\n", skv_last_error());         \
            return 1;                                                         \
        }                                                                     \
    } while (0)

static float bf16_value(uint16_t bits) {
    uint32_t u = (uint32_t)bits << 16;
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

static uint32_t lcg(uint32_t *s) { return *s = *s * 1664525u + 1013904223u; }
/* roughly normal: sum of four uniforms, centred and scaled */
static float noise(uint32_t *s) {
    float acc = 0.0f;
    for (int i = 0; i < 4; ++i) acc += (float)(lcg(s) >> 8) / 16777216.0f;
    return (acc - 2.0f) * 1.7320508f;
}

static double attention_error(const float *q, const float *k, const float *v, const float *got,
                              size_t first, size_t len, size_t q_heads, size_t kv_heads, size_t hd) {
    const size_t kv_dim = kv_heads * hd, gqa = q_heads / kv_heads;
    double worst = 0.0;
    double *p = (double *)malloc(len * sizeof(double));
    for (size_t h = 0; h < q_heads; ++h) {
        const size_t kvh = h / gqa;
        double mx = -INFINITY;
        for (size_t r = first; r < len; ++r) {
            double s = 0.0;
            for (size_t d = 0; d < hd; ++d) s += (double)q[h * hd + d] * k[r * kv_dim + kvh * hd + d];
            p[r] = s / sqrt((double)hd);
            if (p[r] > mx) mx = p[r];
        }
        double sum = 0.0;
        for (size_t r = first; r < len; ++r) sum += (p[r] = exp(p[r] - mx));
        for (size_t d = 0; d < hd; ++d) {
            double o = 0.0;
            for (size_t r = first; r < len; ++r) o += p[r] / sum * v[r * kv_dim + kvh * hd + d];
            const double e = fabs(o - (double)got[h * hd + d]);
            if (e > worst) worst = e;
        }
    }
    free(p);
    return worst;
}

int main(void) {
    const size_t q_heads = 8, kv_heads = 2, hd = 64, capacity = 80, seeded = 45;
    const size_t kv_dim = kv_heads * hd, q_dim = q_heads * hd;
    uint32_t rng = 12345u;

    skv_ctx *ctx = NULL;
    CHECK(skv_ctx_create(0, &ctx) == SKV_OK, "ctx_create");
    skv_layer *bad = NULL;
    CHECK(skv_layer_create(ctx, capacity, 8, 3, hd, SKV_DTYPE_BF16, 0, &bad) == SKV_ERR_CONFIG && bad == NULL,
          "a GQA ratio of 8/3 must be a Config error");
    CHECK(strlen(skv_last_error()) > 0, "an error leaves a message");

    skv_layer *kv = NULL;
    CHECK(skv_layer_create(ctx, capacity, q_heads, kv_heads, hd, SKV_DTYPE_BF16, 0, &kv) == SKV_OK, "layer_create");
    CHECK(skv_capacity(kv) == capacity && skv_kv_dim(kv) == kv_dim && skv_len(kv) == 0, "geometry");
    const size_t n_pages = skv_layer_pages(kv);
    CHECK(n_pages == (capacity + SKV_PAGE_ROWS - 1) / SKV_PAGE_ROWS, "page count");
    int32_t *table = (int32_t *)malloc(n_pages * sizeof(int32_t));
    for (size_t i = 0; i < n_pages; ++i) table[i] = (int32_t)((i * 3 + 1) % n_pages); /* 3 and 5 pages: a permutation */
    CHECK(skv_layer_set_block_table(kv, table, n_pages) == SKV_OK, "set_block_table");

    float *keys = (float *)malloc(capacity * kv_dim * sizeof(float));
    float *values = (float *)malloc(capacity * kv_dim * sizeof(float));
    for (size_t i = 0; i < capacity * kv_dim; ++i) {
        keys[i] = noise(&rng);
        values[i] = noise(&rng);
    }
    CHECK(skv_seed(kv, keys, values, seeded * kv_dim, seeded) == SKV_OK && skv_len(kv) == seeded, "seed");
    for (size_t r = seeded; r < capacity; ++r)
        CHECK(skv_append_host(kv, keys + r * kv_dim, values + r * kv_dim, kv_dim) == SKV_OK, "append row %zu", r);
    CHECK(skv_len(kv) == capacity, "len after appends");
    CHECK(skv_append_host(kv, keys, values, kv_dim) == SKV_ERR_DIMENSION && skv_len(kv) == capacity,
          "an append at capacity must be a Dimension error that changes nothing");

    uint16_t *kb = (uint16_t *)malloc(capacity * kv_dim * sizeof(uint16_t));
    uint16_t *vb = (uint16_t *)malloc(capacity * kv_dim * sizeof(uint16_t));
    CHECK(skv_read_rows(kv, 0, capacity, kb, vb) == SKV_OK, "read_rows");
    for (size_t i = 0; i < capacity * kv_dim; ++i)
        CHECK(kb[i] == skv_f32_to_bf16_bits(keys[i]) && vb[i] == skv_f32_to_bf16_bits(values[i]),
              "contents differ from the bf16 rounding of the input at element %zu", i);

    /* the same rows as f32 (bf16 widened: exact) */
    float *kf = (float *)malloc(capacity * kv_dim * sizeof(float));
    float *vf = (float *)malloc(capacity * kv_dim * sizeof(float));
    CHECK(skv_read_rows_f32(kv, 0, capacity, kf, vf) == SKV_OK, "read_rows_f32");
    for (size_t i = 0; i < capacity * kv_dim; ++i)
        CHECK(kf[i] == bf16_value(kb[i]) && vf[i] == bf16_value(vb[i]), "widened row element %zu", i);

    float *q = (float *)malloc(q_dim * sizeof(float));
    float *out = (float *)malloc(q_dim * sizeof(float));
    for (size_t i = 0; i < q_dim; ++i) q[i] = noise(&rng);
    const size_t starts[3] = {0, 17, capacity - 1};
    for (int w = 0; w < 3; ++w) {
        CHECK(skv_attention_host(kv, q, q_dim, starts[w], out) == SKV_OK, "attention from row %zu", starts[w]);
        const double err = attention_error(q, kf, vf, out, starts[w], capacity, q_heads, kv_heads, hd);
        CHECK(err <= 1e-4, "attention from row %zu: max-abs error %g > 1e-4", starts[w], err);
    }
    CHECK(skv_attention_host(kv, q, q_dim, capacity, out) == SKV_ERR_DIMENSION, "an empty window must be a Dimension error");

    /* rollback then re-append: the rows after the cut are replaced */
    CHECK(skv_truncate(kv, 30) == SKV_OK && skv_len(kv) == 30, "truncate");
    CHECK(skv_append_host(kv, keys, values, kv_dim) == SKV_OK, "append after truncate");
    CHECK(skv_read_rows(kv, 30, 1, kb, vb) == SKV_OK, "read row 30");
    for (size_t i = 0; i < kv_dim; ++i)
        CHECK(kb[i] == skv_f32_to_bf16_bits(keys[i]) && vb[i] == skv_f32_to_bf16_bits(values[i]), "row 30 after rollback");

    /* the f32 element: rows are kept verbatim, bf16 bits are refused */
    skv_layer *kv32 = NULL;
    CHECK(skv_layer_create(ctx, capacity, q_heads, kv_heads, hd, SKV_DTYPE_F32, 0, &kv32) == SKV_OK, "f32 layer_create");
    CHECK(skv_logical_byte_len(kv32) == 2 * skv_logical_byte_len(kv), "f32 rows are twice the bytes");
    CHECK(skv_layer_set_block_table(kv32, table, n_pages) == SKV_OK, "f32 set_block_table");
    CHECK(skv_seed(kv32, keys, values, seeded * kv_dim, seeded) == SKV_OK, "f32 seed");
    for (size_t r = seeded; r < capacity; ++r)
        CHECK(skv_append_host(kv32, keys + r * kv_dim, values + r * kv_dim, kv_dim) == SKV_OK, "f32 append row %zu", r);
    CHECK(skv_read_rows(kv32, 0, 1, kb, vb) == SKV_ERR_CONFIG, "bf16 bits of an f32 layer must be a Config error");
    CHECK(skv_read_rows_f32(kv32, 0, capacity, kf, vf) == SKV_OK, "f32 read_rows_f32");
    CHECK(memcmp(kf, keys, capacity * kv_dim * sizeof(float)) == 0 &&
              memcmp(vf, values, capacity * kv_dim * sizeof(float)) == 0, "f32 rows differ from the input");
    for (int w = 0; w < 3; ++w) {
        CHECK(skv_attention_host(kv32, q, q_dim, starts[w], out) == SKV_OK, "f32 attention from row %zu", starts[w]);
        const double err = attention_error(q, keys, values, out, starts[w], capacity, q_heads, kv_heads, hd);
        CHECK(err <= 1e-4, "f32 attention from row %zu: max-abs error %g > 1e-4", starts[w], err);
    }
    skv_layer_destroy(kv32);

    skv_layer_destroy(kv);
    skv_ctx_destroy(ctx);
    free(table); free(keys); free(values); free(kb); free(vb); free(kf); free(vf); free(q); free(out);
    printf("ok\n");
    return 0;
}
