// Internal declarations shared by the host side and the kernel launchers.
#pragma once

#include <atomic>
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <exception>
#include <new>
#include <string>

#include "../../include/saragossa_kv.h"

namespace skv {

// ---- errors -------------------------------------------------------------------
void set_error(const std::string &msg);
int32_t fail(int32_t code, const std::string &msg);
// Called from the catch-all of an entry point: the exception in flight becomes a status code
// and a message (nothing C++ crosses the C boundary; the reference never panics on a
// fallible path either).
inline int32_t fail_exception() {
    try {
        throw;
    } catch (const std::bad_alloc &) {
        return fail(SKV_ERR_DEVICE, "mémoire hôte épuisée");
    } catch (const std::exception &e) {
        return fail(SKV_ERR_DEVICE, std::string("exception: ") + e.what());
    } catch (...) {
        return fail(SKV_ERR_DEVICE, "exception inconnue");
    }
}
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
    int tile_elems; // one (page, kv head) tile in 16-bit units: P * 16 (bf16), P * 32 (f32)
    int page_elems; // kv_heads * tile_elems
    int ring_rows;  // 0 = full cache; else rows kept by the ring (multiple of 16)
    int f32;        // 1 = the tiles hold f32 (kernels_f32.hip), 0 = bf16
};

__host__ __device__ inline int k_index(int P, int r, int d) {
    (void)P;
    return (((d >> 3) * 16 + r) << 3) + (d & 7);
}
__host__ __device__ inline int v_index(int P, int r, int d) {
    (void)P;
    return ((((((d >> 5) * 4 + (r >> 2)) * 16 + (d & 15)) * 2 + ((d >> 4) & 1))) << 2) + (r & 3);
}

// The f32 element's tiles (kernels_f32.hip), in floats from the tile's start.
__host__ __device__ inline int k_index_f32(int r, int d) {
    return (((d >> 4) * 64 + ((d >> 2) & 3) * 16 + r) << 2) + (d & 3);
}
__host__ __device__ inline int v_index_f32(int r, int d) {
    return (((d >> 4) * 64 + (r >> 2) * 16 + (d & 15)) << 2) + (r & 3);
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
    // rows [v_grp_first, v_grp_first + v_grp_rows) of the batch start at a position that is a
    // multiple of 4 and come in whole groups of 4: their V elements are written as 16-byte
    // units of the transposed tile (4 rows x 2 dims) instead of 2-byte stores
    int v_grp_first;
    int v_grp_rows;
    // batches: row items are numbered page by page with the row inside the page fastest, so
    // that sixteen neighbouring threads write 256 contiguous bytes of a K tile
    int by_page;
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
    int n_queries;    // 1 = decode; C = chunked prefill, query i sits at position q_pos0 + i
    int q_pos0;       // position of query row 0 (len - n_queries unless the chunk is attended in two phases)
    int limit_cap;    // no query attends beyond this position (INT_MAX = only its own causal limit)
    int split_base;   // this launch writes partials [split_base, split_base + splits) of splits_total
    int splits_total; // partial sets the merge will see; 1 = the launch writes the context itself
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
    int new_slot;     // slot that receives the row
    int new_page;     // physical page of that slot (the host knows its block table)
    // fused pre-KV step (pre != 0): q and the appended k row arrive raw and get the per-head
    // RMSNorm (weights null = none) and the rotation of this position before they are used
    int pre;
    int rope_dims;          // rotated leading dims of each head (even, <= head_dim; 0 = none)
    int rope_style;         // 0 = halves (i, i + rope_dims/2), 1 = interleaved (2i, 2i+1)
    float eps;
    const float *rope;      // [rope_dims/2][2]: (cos, sin) of this position
    const float *q_norm_w;  // [head_dim]
    const float *k_norm_w;  // [head_dim]
    // decode only: head h of q starts at q + h * q_head_stride (0 = head_dim), and the
    // context of head h is multiplied by sigmoid(gate[h * q_head_stride + col]) (null = none)
    const float *gate;
    int q_head_stride;
    int q_vec;              // q is 16-byte aligned and head_dim a multiple of 8: 16-byte loads
    int tiles2;             // prefill tile kernel: two 16-slot query tiles per wavefront
    int xchg_off;           // split kernel: byte offset in LDS of the wavefronts' exchange area (0 = it reuses the staging area); set by the launcher
    Geom g;
};
static_assert(sizeof(DecodeArgs) <= 256, "sixteen of them must fit the kernel argument block");

// Standalone per-head RMSNorm + rotation of one row (the same arithmetic as the fused step).
struct NormRopeArgs {
    const float *x;      // [heads][head_dim]
    float *out;          // [heads][head_dim]
    const float *weight; // [head_dim] or null
    const float *rope;   // [rope_dims/2][2] or null
    int heads, head_dim, rope_dims, rope_style;
    float eps;
    int x_head_stride; // elements between the heads of x (0 = head_dim)
    // several rows at consecutive positions (grid y): row r of x and out is heads * head_dim
    // further (contiguous rows) and uses the rotation of the position r further in the table
    int n_rows;
};

// out[h][c] = ctx[h][c] * sigmoid(gate[h * gate_head_stride + c])
struct GateArgs {
    const float *ctx;
    const float *gate;
    float *out;
    int heads, head_dim, gate_head_stride;
};
hipError_t launch_gate(const GateArgs &a, hipStream_t s);
hipError_t launch_iota(int32_t *dst, int n, hipStream_t s);

// Measurement aids (a read-only walk of the cache with the decode kernel's pattern; an empty launch).
struct ProbeArgs {
    const uint16_t *k_pool;
    const uint16_t *v_pool;
    const int32_t *table;
    uint32_t *sink;
    float *part;     // null = read only; else every workgroup also writes part_floats floats (a multiple of 4)
    int part_floats;
    int n_pages;
    int splits;
    Geom g;
};
hipError_t launch_probe_read(const ProbeArgs &a, hipStream_t s);
hipError_t launch_probe_empty(hipStream_t s);
hipError_t launch_norm_rope(const NormRopeArgs &a, hipStream_t s);

// Raises a kernel's dynamic LDS limit to the 160 KiB of a gfx950 compute unit, once per
// device and kernel (`done` is a per-kernel bit mask over device ids; the attribute belongs to
// the current device's copy of the code object).
inline hipError_t allow_full_lds(const void *kernel, std::atomic<uint64_t> &done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

#ifdef __HIPCC__
// max / sum over the four 16-lane rows of a wavefront (lanes l, l^16, l^32, l^48), every
// lane receiving the result: two row swaps in the vector unit instead of two exchanges
// through LDS.
__device__ __forceinline__ float rows_max(float v) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
// sigmoid_scalar (src/decoder/attention_ops.rs:522-524)
__device__ __forceinline__ float sigmoid_gate(float g) { return 1.0f / (1.0f + expf(-g)); }
// The arithmetic of rms_norm_rope_heads_at (src/decoder/attention_ops.rs:682-777), operation
// for operation and without contraction, so that the device row equals the CPU row bit for
// bit when the (cos, sin) table comes from the host's libm.
// (The contraction pragma matters: the __f*_rn intrinsics are plain operators here and
// would be fused into FMAs otherwise.)
__device__ __forceinline__ float head_inv_rms(const float *row, int head_dim, float eps) {
#pragma clang fp contract(off)
    float sum = 0.0f;
    for (int c = 0; c < head_dim; ++c) {
        const float sq = row[c] * row[c];
        sum = sum + sq;
    }
    const float mean_square = sum / (float)head_dim;
    return 1.0f / sqrtf(mean_square + eps);
}
// The same from the squares, already taken (x * x, rounded) and padded with zeros to a
// multiple of 16 entries at a 16-byte aligned address: the adds stay in index order, the
// loads come sixteen values at a time.
__device__ __forceinline__ float head_inv_rms_sq(const float *sq, int padded, int head_dim, float eps) {
#pragma clang fp contract(off)
    typedef __attribute__((ext_vector_type(4))) float f4;
    const f4 *p = reinterpret_cast<const f4 *>(sq);
    float sum = 0.0f;
    for (int c = 0; c < padded / 4; c += 4) {
        const f4 v0 = p[c], v1 = p[c + 1], v2 = p[c + 2], v3 = p[c + 3];
        sum = sum + v0.x; sum = sum + v0.y; sum = sum + v0.z; sum = sum + v0.w;
        sum = sum + v1.x; sum = sum + v1.y; sum = sum + v1.z; sum = sum + v1.w;
        sum = sum + v2.x; sum = sum + v2.y; sum = sum + v2.z; sum = sum + v2.w;
        sum = sum + v3.x; sum = sum + v3.y; sum = sum + v3.z; sum = sum + v3.w;
    }
    const float mean_square = sum / (float)head_dim;
    return 1.0f / sqrtf(mean_square + eps);
}
// Element c of the head after norm (inv, w; w null = 1) and rotation (rope null = none).
__device__ __forceinline__ float norm_rope_elem(const float *row, int c, float inv, const float *w,
                                                const float *rope, int rope_dims, int style) {
#pragma clang fp contract(off)
    auto normed = [&](int i) {
#pragma clang fp contract(off)
        const float scaled = row[i] * inv;
        return w ? scaled * w[i] : scaled;
    };
    if (!rope || c >= rope_dims) return normed(c);
    const int pairs = rope_dims >> 1;
    int pair, i0, i1;
    bool is_first;
    if (style == 1) {
        pair = c >> 1;
        i0 = 2 * pair;
        i1 = i0 + 1;
        is_first = (c & 1) == 0;
    } else {
        is_first = c < pairs;
        pair = is_first ? c : c - pairs;
        i0 = pair;
        i1 = pair + pairs;
    }
    const float cs = rope[2 * pair], sn = rope[2 * pair + 1];
    const float first = normed(i0), second = normed(i1);
    const float fc = first * cs, ss = second * sn, fs = first * sn, sc = second * cs;
    return is_first ? fc - ss : fs + sc;
}
#endif

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
// f32 storage mode: rows in and out (k_dst / v_dst of GatherArgs then point at f32 rows), and
// the split launch for one query row or a chunk (the caller merges as for bf16)
hipError_t launch_append_f32(const AppendArgs &a, hipStream_t s);
hipError_t launch_gather_f32(const GatherArgs &a, hipStream_t s);
hipError_t launch_f32_split(const DecodeArgs &a, hipStream_t s);
bool f32_decode_kernel_serves(const DecodeArgs &a); // the launch takes the kernel that can also append the row
hipError_t launch_decode(const DecodeArgs &a, hipStream_t s);
hipError_t launch_decode_batch(const DecodeBatchArgs &b, int n_seq, hipStream_t s);
hipError_t launch_f32_split_batch(const DecodeBatchArgs &b, int n_seq, int max_splits, hipStream_t s);
hipError_t launch_merge(const DecodeArgs &a, hipStream_t s);        // split-K partials -> context
hipError_t launch_prefill_tiles(const DecodeArgs &a, hipStream_t s); // chunked prefill, no merge
int prefill_tile_slots(int P, bool two_tiles);
bool prefill_two_tiles_possible(int P);
hipError_t launch_merge_rows(const DecodeArgs &a, hipStream_t s);    // the same merge for many query slots
hipError_t launch_naive(const NaiveArgs &a, hipStream_t s);
int decode_max_splits();

} // namespace skv
