/* What a native host pays for remember_prefix_block (src/serve/state.rs:613-639) on the
 * GPU hot cache, one block boundary per call: the 4096-token prefix of BASELINE configs[3]
 * (256 blocks of 16 tokens over 36 layers of kv8/hd128 bf16 KV), hash chain included.
 * Plain C11 through the C ABI, no interpreter in the loop. Prints one JSON line:
 * host_us = the 256 calls returned, total_us = the GPU has finished the copies
 * (median of seven passes). Exit status 0 = every block was cached. */
#define _POSIX_C_SOURCE 199309L
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "saragossa_kv.h"

#define CHECK(cond, what)                                                        \
    do {                                                                         \
        if (!(cond)) {                                                           \
            fprintf(stderr, "FAIL %s (line %d): %s\n", what, __LINE__, skv_last_error()); \
            return 1;                                                            \
        }                                                                        \
    } while (0)

enum { LAYERS = 36, ROWS = 4096, KV_HEADS = 8, HEAD_DIM = 128, BLOCK = 16, PASSES = 7 };

static double now_us(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec * 1e6 + (double)t.tv_nsec * 1e-3;
}
static int by_value(const void *a, const void *b) {
    const double x = *(const double *)a, y = *(const double *)b;
    return (x > y) - (x < y);
}

int main(void) {
    const size_t kv_dim = (size_t)KV_HEADS * HEAD_DIM, n_blocks = ROWS / BLOCK;
    skv_ctx *ctx = NULL;
    CHECK(skv_ctx_create(0, &ctx) == SKV_OK, "ctx_create");
    float *rows = (float *)malloc((size_t)ROWS * kv_dim * sizeof(float));
    uint32_t rng = 2463534242u;
    for (size_t i = 0; i < (size_t)ROWS * kv_dim; ++i) {
        rng ^= rng << 13; rng ^= rng >> 17; rng ^= rng << 5;
        rows[i] = (float)(rng >> 8) * (1.0f / 8388608.0f) - 1.0f;
    }
    skv_layer *layers[LAYERS];
    for (int l = 0; l < LAYERS; ++l) {
        CHECK(skv_layer_create(ctx, ROWS + 64, 32, KV_HEADS, HEAD_DIM, SKV_DTYPE_BF16, 0, &layers[l]) == SKV_OK, "layer_create");
        CHECK(skv_seed(layers[l], rows, rows, (size_t)ROWS * kv_dim, ROWS) == SKV_OK, "seed");
    }
    skv_hot *hot = NULL;
    CHECK(skv_hot_create(ctx, BLOCK, 4096, 4096, 1024, layers, LAYERS, &hot) == SKV_OK, "hot_create");
    uint64_t *tokens = (uint64_t *)malloc(ROWS * sizeof(uint64_t));
    for (size_t i = 0; i < ROWS; ++i) {
        rng ^= rng << 13; rng ^= rng >> 17; rng ^= rng << 5;
        tokens[i] = rng % 151936u;
    }
    uint8_t root[32];
    skv_hash_root(root);
    double host[PASSES], total[PASSES];
    size_t kept = 0;
    for (int pass = 0; pass < PASSES; ++pass) {
        int32_t found = 1;
        size_t bytes = 0;
        while (found) CHECK(skv_hot_evict_lru(hot, &found, &bytes) == SKV_OK, "evict");
        CHECK(skv_ctx_synchronize(ctx) == SKV_OK, "synchronize");
        uint8_t h[32], next[32];
        memcpy(h, root, 32);
        kept = 0;
        const double t0 = now_us();
        for (size_t b = 0; b < n_blocks; ++b) {
            int32_t cached = 0;
            skv_hash_chain(h, tokens + b * BLOCK, BLOCK, next);
            memcpy(h, next, 32);
            CHECK(skv_hot_remember(hot, NULL, root, h, (b + 1) * BLOCK, layers, LAYERS, NULL, NULL, 0, &cached) == SKV_OK,
                  "hot_remember");
            kept += cached != 0;
        }
        const double t1 = now_us();
        CHECK(skv_ctx_synchronize(ctx) == SKV_OK, "synchronize");
        const double t2 = now_us();
        host[pass] = t1 - t0;
        total[pass] = t2 - t0;
    }
    qsort(host, PASSES, sizeof(double), by_value);
    qsort(total, PASSES, sizeof(double), by_value);
    printf("{\"calls\": %zu, \"cached\": %zu, \"host_us\": %.1f, \"total_us\": %.1f, \"host_us_per_call\": %.2f}\n",
           n_blocks, kept, host[PASSES / 2], total[PASSES / 2], host[PASSES / 2] / (double)n_blocks);
    skv_hot_destroy(hot);
    for (int l = 0; l < LAYERS; ++l) skv_layer_destroy(layers[l]);
    skv_ctx_destroy(ctx);
    free(rows);
    free(tokens);
    return kept == n_blocks ? 0 : 2;
}
