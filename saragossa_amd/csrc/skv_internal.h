// Internal declarations shared by the host side and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

#include "../../include/saragossa_kv.h"

namespace skv {

// ---- errors -------------------------------------------------------------------
void set_error(const std::string &msg);
int32_t fail(int32_t code, const std::string &msg);
int32_t fail_hip(hipError_t e, const char *what);

#define SKV_HIP(expr)                                            \
    do {                                                         \
        hipError_t e__ = (expr);                                 \
        if (e__ != hipSuccess) return ::skv::fail_hip(e__, #expr); \
    } while (0)

// ---- geometry of one layer's pages ---------------------------------------------
//
// A page holds 16 rows of K (or V) for every kv head. Inside a page the elements
// are stored in the order the gfx950 matrix instructions read them, so that a
// wavefront fetches one (page, kv head) tile with 16-byte loads from consecutive
// addresses:
//
//   K tile [P/8 groups][16 rows][8 dims]            element (row r, dim d) at
//          ((d/8)*16 + r)*8 + d%8
//   V tile [P/32][4 row-quads][16 cols][2][4 rows]  element (row r, dim d) at
//          ((((d/32)*4 + r/4)*16 + d%16)*2 + (d%32)/16)*4 + r%4
//
// P is head_dim rounded up to 32, 64, 128, 256 or 512; dims in [head_dim, P) stay zero.
struct Geom {
    int q_heads;
    int kv_heads;
    int head_dim;
    int P;          // padded head dim
    int gqa;        // q_heads / kv_heads
    int tile_elems; // P * 16: one (page, kv head) tile
    int page_elems; // kv_heads * tile_elems
    int ring_rows;  // 0 = full cache; else rows kept by the ring (multiple of 16)
};

__host__ __device__ inline int k_index(int P, int r, int d) {
    (void)P;
    return (((d >> 3) * 16 + r) << 3) + (d & 7);
}
__host__ __device__ inline int v_index(int P, int r, int d) {
    (void)P;
    return ((((((d >> 5) * 4 + (r >> 2)) * 16 + (d & 15)) * 2 + ((d >> 4) & 1))) << 2) + (r & 3);
}

// Rows are addressed by position; a ring layer keeps position p in slot p % ring_rows.
__host__ __device__ inline long slot_of(long pos, int ring_rows) {
    return ring_rows > 0 ? pos % ring_rows : pos;
}

// ---- launch argument blocks ------------------------------------------------------
struct AppendArgs {
    const float *k_src; // [n_rows, kv_dim] f32
    const float *v_src;
    uint16_t *k_pool;
    uint16_t *v_pool;
    const int32_t *table;
    long first_pos; // position of the first appended row
    int n_rows;
    Geom g;
};

struct GatherArgs {
    const uint16_t *k_pool;
    const uint16_t *v_pool;
    const int32_t *table;
    uint16_t *k_dst; // [n_rows, kv_dim] bf16 bits
    uint16_t *v_dst;
    long first_pos;
    int n_rows;
    Geom g;
};

struct DecodeArgs {
    const float *q;  // [n_queries][q_heads*head_dim] f32
    float *out;      // [n_queries][q_heads*head_dim] f32
    const uint16_t *k_pool;
    const uint16_t *v_pool;
    const int32_t *table;
    float *part_o;   // [kv_heads][splits][n_queries*gqa][head_dim]
    float *part_m;   // [kv_heads][splits][n_queries*gqa]   (log2 domain)
    float *part_l;   // [kv_heads][splits][n_queries*gqa]
    int len;          // rows valid: positions 0..len
    int n_queries;    // 1 = decode; C = chunked prefill, query i attends positions <= len-C+i
    int window;       // sliding window applied per query (0 = none)
    int window_start; // first position attended (lower bound for every query)
    int ring_base;    // ring layers: (len-1) - (len-1) % ring_rows
    int ring_t;       // ring layers: (len-1) % ring_rows
    int page_first;   // first logical page scanned
    int n_pages;      // logical pages scanned
    int splits;
    int waves;        // wavefronts per workgroup: 4 or 8
    float qscale;     // (1/sqrt(head_dim)) * log2(e)
    // fused append of the row at position len-1 (k_new null = none)
    const float *k_new; // [kv_dim] f32
    const float *v_new;
    uint16_t *k_pool_w;
    uint16_t *v_pool_w;
    int new_slot;     // slot that receives the row
    Geom g;
};

// One decode step of the same model layer for several independent sequences.
constexpr int SKV_MAX_BATCH = 16;
struct DecodeBatchArgs {
    DecodeArgs seq[SKV_MAX_BATCH];
};
static_assert(sizeof(DecodeBatchArgs) <= 4096, "kernel arguments are limited to 4 KiB");

struct NaiveArgs {
    const float *q;
    float *out;
    const uint16_t *k_pool;
    const uint16_t *v_pool;
    const int32_t *table;
    float *scores; // [q_heads][n_keys]
    long len;
    long window_start;
    float inv_scale; // 1/sqrt(head_dim)
    Geom g;
};

// ---- launchers (kernels.hip) ------------------------------------------------------
hipError_t launch_append(const AppendArgs &a, hipStream_t s);
hipError_t launch_gather(const GatherArgs &a, hipStream_t s);
hipError_t launch_decode(const DecodeArgs &a, hipStream_t s);
hipError_t launch_decode_batch(const DecodeBatchArgs &b, int n_seq, hipStream_t s);
hipError_t launch_naive(const NaiveArgs &a, hipStream_t s);
int decode_max_splits();

} // namespace skv
