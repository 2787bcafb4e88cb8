// gfx950 kernels of the KV hot path, part 1: append into paged bf16 tiles, gather back
// to rows, and the plain three-phase attention kernel kept behind the
// RETI_RUST_FLASH_SDPA kill-switch.
#include "skv_internal.h"

namespace skv {

// f32 -> bf16 bits: round to nearest even on the raw bits with a wrapping add and
// no NaN special case, the reference's formula (src/decode_resident/utils.rs:55-60).
__device__ __forceinline__ uint16_t bf16_bits(float v) {
    uint32_t b = __float_as_uint(v);
    uint32_t lsb = (b >> 16) & 1u;
    return (uint16_t)((b + 0x7fffu + lsb) >> 16);
}
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}

// ------------------------------------------------------------------------------------
// append: f32 rows -> bf16 tiles. One thread per (row, kv head, 8-dim group): a 16-byte
// store into the K tile, eight 2-byte stores into the transposed V tile. In a batch, the
// rows that form whole position-aligned groups of four take a second kind of work item for
// V instead: one thread per (row group, kv head, 32-dim block, column) gathers 4 rows x 2
// dims and writes the 16 contiguous bytes they occupy in the tile.
// Stands in for copy_at_f32_to_bf16 (src/decode_resident/kernels.rs:1036-1044).
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void append_kernel(AppendArgs a) {
    const Geom g = a.g;
    const int groups = (g.head_dim + 7) >> 3;
    const long per_row = (long)g.kv_heads * groups;
    const long page0 = a.first_pos >> 4; // first page of positions the batch touches
    const long n_blk = ((a.first_pos + a.n_rows + 15) >> 4) - page0;
    const long total_rows = a.by_page ? n_blk * per_row * 16 : per_row * a.n_rows;
    const int kv_dim = g.kv_heads * g.head_dim;
    const int per_grp = g.kv_heads * (g.P >> 5) * 16;
    const long total = total_rows + (long)(a.v_grp_rows >> 2) * per_grp;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total;
         t += (long)gridDim.x * blockDim.x) {
        if (t >= total_rows) {
            // V of one aligned group of four rows: columns c and c + 16 of a 32-dim block
            const long u = t - total_rows;
            const int grp4 = (int)(u / per_grp);
            int rem = (int)(u - (long)grp4 * per_grp);
            const int kvh = rem / ((g.P >> 5) * 16);
            rem -= kvh * ((g.P >> 5) * 16);
            const int db = rem >> 4, c = rem & 15;
            const int row0 = a.v_grp_first + grp4 * 4;
            const long slot = slot_of(a.first_pos + row0, g.ring_rows); // a multiple of 4
            const int page = a.table[slot >> 4];
            const long tile = (long)page * g.page_elems + (long)kvh * g.tile_elems;
            const int d0 = db * 32 + c, d1 = d0 + 16;
            const float *vs = a.v_src + (long)row0 * kv_dim + kvh * g.head_dim;
            uint16_t lo[4], hi[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                lo[r] = d0 < g.head_dim ? bf16_bits(vs[(long)r * kv_dim + d0]) : (uint16_t)0;
                hi[r] = d1 < g.head_dim ? bf16_bits(vs[(long)r * kv_dim + d1]) : (uint16_t)0;
            }
            uint4 pk;
            pk.x = lo[0] | ((uint32_t)lo[1] << 16);
            pk.y = lo[2] | ((uint32_t)lo[3] << 16);
            pk.z = hi[0] | ((uint32_t)hi[1] << 16);
            pk.w = hi[2] | ((uint32_t)hi[3] << 16);
            *reinterpret_cast<uint4 *>(a.v_pool + tile + v_index(g.P, (int)(slot & 15), d0)) = pk;
            continue;
        }
        int row, kvh, grp;
        if (a.by_page) {
            const long blk = t / (per_row * 16);
            const int rem = (int)(t - blk * per_row * 16);
            const long pos = (page0 + blk) * 16 + (rem & 15);
            if (pos < a.first_pos || pos >= a.first_pos + a.n_rows) continue;
            row = (int)(pos - a.first_pos);
            grp = (rem >> 4) % groups;
            kvh = (rem >> 4) / groups;
        } else {
            row = (int)(t / per_row);
            const int rem = (int)(t - (long)row * per_row);
            kvh = rem / groups;
            grp = rem - kvh * groups;
        }
        const long slot = slot_of(a.first_pos + row, g.ring_rows);
        const int page = a.table[slot >> 4];
        const int r = (int)(slot & 15);
        const long tile = (long)page * g.page_elems + (long)kvh * g.tile_elems;
        const float *ks = a.k_src + (long)row * kv_dim + kvh * g.head_dim + grp * 8;
        const float *vs = a.v_src + (long)row * kv_dim + kvh * g.head_dim + grp * 8;
        const int d0 = grp * 8;
        const int nd = min(8, g.head_dim - d0);
        uint16_t kb[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) kb[e] = e < nd ? bf16_bits(ks[e]) : (uint16_t)0;
        uint4 pk;
        pk.x = kb[0] | ((uint32_t)kb[1] << 16);
        pk.y = kb[2] | ((uint32_t)kb[3] << 16);
        pk.z = kb[4] | ((uint32_t)kb[5] << 16);
        pk.w = kb[6] | ((uint32_t)kb[7] << 16);
        *reinterpret_cast<uint4 *>(a.k_pool + tile + k_index(g.P, r, d0)) = pk;
        if (row >= a.v_grp_first && row < a.v_grp_first + a.v_grp_rows) continue; // V by groups
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (e < nd) a.v_pool[tile + v_index(g.P, r, d0 + e)] = bf16_bits(vs[e]);
    }
}

hipError_t launch_append(const AppendArgs &a, hipStream_t s) {
    const int groups = (a.g.head_dim + 7) >> 3;
    const long n_blk = ((a.first_pos + a.n_rows + 15) >> 4) - (a.first_pos >> 4);
    const long row_items = a.by_page ? n_blk * 16 : (long)a.n_rows;
    const long total = (long)a.g.kv_heads * groups * row_items +
                       (long)(a.v_grp_rows >> 2) * a.g.kv_heads * (a.g.P >> 5) * 16;
    if (total <= 0) return hipSuccess;
    long blocks = (total + 255) / 256;
    if (blocks > 65535 * 4) blocks = 65535 * 4;
    hipLaunchKernelGGL(append_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    return hipGetLastError();
}

// Identity block table of a fresh layer, written on the device (no host-to-device copy).
__global__ __launch_bounds__(256) void iota_kernel(int32_t *dst, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = i;
}

hipError_t launch_iota(int32_t *dst, int n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(iota_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, dst, n);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------
// Measurement aids: a launch that only fetches the cache the way the decode kernel does
// (grid (splits, kv heads), eight wavefronts, each walking its share of the pages and loading
// the K and V tile of its kv head with 16-byte non-temporal loads, 1 KiB per instruction), and
// an empty launch of the same shape.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(512) void probe_read_kernel(ProbeArgs a) {
    // the wavefront's number as a scalar: the block-table entries then come through the scalar
    // unit and do not queue behind the other wavefronts' tile loads
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int split = blockIdx.x, kvh = blockIdx.y;
    const int pb0 = (int)(((long)split * a.n_pages) / a.splits);
    const int pb1 = (int)(((long)(split + 1) * a.n_pages) / a.splits);
    const int units = a.g.tile_elems >> 3; // 16-byte units of one tile
    uint32_t acc = 0;
    for (int pb = pb0 + wave; pb < pb1; pb += 8) {
        const int page = __builtin_amdgcn_readfirstlane(a.table[pb]);
        const long tile = (long)page * a.g.page_elems + (long)kvh * a.g.tile_elems;
        typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
        const u32x4_t *kp = reinterpret_cast<const u32x4_t *>(a.k_pool + tile);
        const u32x4_t *vp = reinterpret_cast<const u32x4_t *>(a.v_pool + tile);
        for (int u = lane; u < units; u += 64 * 8) {
            u32x4_t k[8], v[8];
            if ((units & 511) == 0) {
                // whole rounds of 512 units: constant offsets from one address per tile
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    k[i] = __builtin_nontemporal_load(kp + u + i * 64);
                    v[i] = __builtin_nontemporal_load(vp + u + i * 64);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int at = min(u + i * 64, units - 1);
                    k[i] = __builtin_nontemporal_load(kp + at);
                    v[i] = __builtin_nontemporal_load(vp + at);
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) acc ^= k[i].x ^ k[i].w ^ v[i].y ^ v[i].z;
        }
    }
    if (acc == 0x9e3779b9u && a.sink) a.sink[0] = acc; // keeps the loads alive
    if (a.part) {
        // what a split launch has to leave behind: a partial of the decode kernel's size per
        // workgroup, written after the last page has arrived, with the same non-temporal stores
        typedef float f32x4_t __attribute__((ext_vector_type(4)));
        const float x = (float)(acc & 1u);
        f32x4_t *dst = reinterpret_cast<f32x4_t *>(a.part) + (size_t)(kvh * a.splits + split) * (size_t)(a.part_floats >> 2);
        for (int u = threadIdx.x; u < (a.part_floats >> 2); u += 512) __builtin_nontemporal_store(f32x4_t{x, x, x, x}, dst + u);
    }
}

__global__ __launch_bounds__(512) void probe_empty_kernel(uint32_t *sink) {
    if (sink && threadIdx.x == 0xffff) sink[0] = 1;
}

hipError_t launch_probe_read(const ProbeArgs &a, hipStream_t s) {
    if (a.n_pages <= 0 || a.splits <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)a.splits, (unsigned)a.g.kv_heads), dim3(512), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_probe_empty(hipStream_t s) {
    hipLaunchKernelGGL(probe_empty_kernel, dim3(256), dim3(512), 0, s, (uint32_t *)nullptr);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------
// gather: tiles -> row-major bf16 rows [n_rows, kv_dim], through the block table.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gather_kernel(GatherArgs a) {
    const Geom g = a.g;
    const int groups = (g.head_dim + 7) >> 3;
    const long per_row = (long)g.kv_heads * groups;
    const long total = per_row * a.n_rows;
    const int kv_dim = g.kv_heads * g.head_dim;
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total;
         t += (long)gridDim.x * blockDim.x) {
        const int row = (int)(t / per_row);
        const int rem = (int)(t - (long)row * per_row);
        const int kvh = rem / groups;
        const int grp = rem - kvh * groups;
        const long slot = slot_of(a.first_pos + row, g.ring_rows);
        const int page = a.table[slot >> 4];
        const int r = (int)(slot & 15);
        const long tile = (long)page * g.page_elems + (long)kvh * g.tile_elems;
        const int d0 = grp * 8;
        const int nd = min(8, g.head_dim - d0);
        const long dst = (long)row * kv_dim + kvh * g.head_dim + d0;
        const uint4 pk = *reinterpret_cast<const uint4 *>(a.k_pool + tile + k_index(g.P, r, d0));
        const uint32_t w[4] = {pk.x, pk.y, pk.z, pk.w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (e < nd) {
                if (a.k_dst) a.k_dst[dst + e] = (uint16_t)(w[e >> 1] >> ((e & 1) * 16));
                if (a.v_dst) a.v_dst[dst + e] = a.v_pool[tile + v_index(g.P, r, d0 + e)];
            }
    }
}

hipError_t launch_gather(const GatherArgs &a, hipStream_t s) {
    const int groups = (a.g.head_dim + 7) >> 3;
    const long total = (long)a.g.kv_heads * groups * a.n_rows;
    if (total <= 0) return hipSuccess;
    long blocks = (total + 255) / 256;
    if (blocks > 65535 * 4) blocks = 65535 * 4;
    hipLaunchKernelGGL(gather_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------
// Plain three-phase attention, one workgroup per query head: scores with a strictly
// sequential dot product (separate multiply and add, like the CPU path), softmax,
// then a sequential weighted sum over the rows. It stands in for
// attention_decode_naive_bf16 (src/decode_resident/kernels.rs:90-164) behind
// RETI_RUST_FLASH_SDPA=0 and serves as an independent check of the matrix-core kernel.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void naive_kernel(NaiveArgs a) {
    // the __f*_rn intrinsics are plain operators here: without this they fuse into FMAs
#pragma clang fp contract(off)
    const Geom g = a.g;
    const int h = blockIdx.x;
    const int kvh = h / g.gqa;
    const int tid = threadIdx.x;
    const long nkeys = a.len - a.window_start;
    float *scores = a.scores + (long)h * nkeys;
    const float *q = a.q + (long)h * g.head_dim;
    __shared__ float red[256];

    float mx = -INFINITY;
    for (long i = tid; i < nkeys; i += 256) {
        const long slot = slot_of(a.window_start + i, g.ring_rows);
        const int page = a.table[slot >> 4];
        const int r = (int)(slot & 15);
        const uint16_t *kt = a.k_pool + (long)page * g.page_elems + (long)kvh * g.tile_elems;
        const float *ktf = reinterpret_cast<const float *>(kt);
        float dot = 0.0f;
        for (int d = 0; d < g.head_dim; ++d)
            dot = __fadd_rn(dot, __fmul_rn(q[d], g.f32 ? ktf[k_index_f32(r, d)] : bf16_to_f32(kt[k_index(g.P, r, d)])));
        const float sc = __fmul_rn(dot, a.inv_scale);
        scores[i] = sc;
        mx = fmaxf(mx, sc);
    }
    red[tid] = mx;
    __syncthreads();
    for (int off = 128; off >= 1; off >>= 1) {
        if (tid < off) red[tid] = fmaxf(red[tid], red[tid + off]);
        __syncthreads();
    }
    mx = red[0];
    __syncthreads();
    float sum = 0.0f;
    for (long i = tid; i < nkeys; i += 256) {
        const float e = expf(scores[i] - mx);
        scores[i] = e;
        sum += e;
    }
    red[tid] = sum;
    __syncthreads();
    for (int off = 128; off >= 1; off >>= 1) {
        if (tid < off) red[tid] += red[tid + off];
        __syncthreads();
    }
    sum = red[0];
    const bool uniform = sum <= 1.1920929e-07f; // f32::EPSILON fallback of softmax_in_place
    for (int d = tid; d < g.head_dim; d += 256) {
        float acc = 0.0f;
        for (long i = 0; i < nkeys; ++i) {
            const long slot = slot_of(a.window_start + i, g.ring_rows);
            const int page = a.table[slot >> 4];
            const int r = (int)(slot & 15);
            const uint16_t *vt = a.v_pool + (long)page * g.page_elems + (long)kvh * g.tile_elems;
            const float pr = uniform ? 1.0f / (float)nkeys : scores[i] / sum;
            const float val = g.f32 ? reinterpret_cast<const float *>(vt)[v_index_f32(r, d)] : bf16_to_f32(vt[v_index(g.P, r, d)]);
            acc = __fadd_rn(acc, __fmul_rn(pr, val));
        }
        a.out[(long)h * g.head_dim + d] = acc;
    }
}

hipError_t launch_naive(const NaiveArgs &a, hipStream_t s) {
    hipLaunchKernelGGL(naive_kernel, dim3((unsigned)a.g.q_heads), dim3(256), 0, s, a);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------
// Per-head RMSNorm + rotation of one row, one workgroup per head
// (rms_norm_rope_heads_decode_f32, src/decode_resident/kernels.rs:975-1027). The sum of
// squares is taken in index order by one lane, like the CPU path, so the row is the CPU
// row bit for bit.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void norm_rope_kernel(NormRopeArgs a) {
    __shared__ float row[512];
    __shared__ float w[512];
    __shared__ float rope[512];
    __shared__ float inv_s;
    const int head = blockIdx.x;
    const int r = blockIdx.y; // row (position_offset + r)
    const int tid = threadIdx.x;
    const long row_elems = (long)a.heads * a.head_dim;
    const float *x = a.x + r * row_elems + (long)head * (a.x_head_stride > 0 ? a.x_head_stride : a.head_dim);
    const float *rope_row = a.rope ? a.rope + (long)r * a.rope_dims : nullptr;
    for (int c = tid; c < a.head_dim; c += 256) {
        row[c] = x[c];
        w[c] = a.weight ? a.weight[c] : 1.0f;
        rope[c] = (rope_row && c < a.rope_dims) ? rope_row[c] : 0.0f;
    }
    __syncthreads();
    if (tid == 0) inv_s = a.weight ? head_inv_rms(row, a.head_dim, a.eps) : 1.0f;
    __syncthreads();
    const float inv = inv_s;
    for (int c = tid; c < a.head_dim; c += 256)
        a.out[r * row_elems + (long)head * a.head_dim + c] =
            norm_rope_elem(row, c, inv, a.weight ? w : nullptr, a.rope ? rope : nullptr, a.rope_dims,
                           a.rope_style);
}

// The same for many rows (a prefill chunk): one workgroup per ROWS_PAIRS (row, head) pairs.
// Their raw values are staged in LDS with coalesced loads (pair stride head_dim + 1: lane i
// walking pair i is conflict-free), lane i of the first wavefront takes the sum of squares of
// pair i in index order, exactly as above, and all threads then produce the outputs with
// coalesced stores, weight and rotations read from LDS. One workgroup per pair, as for a
// single row, leaves 255 of 256 lanes waiting for the ordered sum: 24.6 us for 512 rows of
// 32 heads x 128 against 14.5 us this way, 89.8 against 32.8 us for 2048 rows. Sixteen pairs
// per workgroup are best up to head_dim 128, eight above (measured).
template <int ROWS_PAIRS>
__global__ __launch_bounds__(256) void norm_rope_rows_kernel(NormRopeArgs a) {
    // [pairs][head_dim + 1] values | [pairs] inverse rms | [head_dim] weight | [rows][rope_dims] rotations
    extern __shared__ float rows_lds[];
    const int hd = a.head_dim;
    const int stride = hd + 1;
    float *inv_s = rows_lds + ROWS_PAIRS * stride;
    float *w_s = inv_s + ROWS_PAIRS;
    float *rope_s = w_s + hd;
    const int lane = threadIdx.x; // 0..255; the ordered sums use the first ROWS_PAIRS
    const long n_pairs = (long)a.n_rows * a.heads;
    const long pair0 = (long)blockIdx.x * ROWS_PAIRS;
    const int here = (int)min((long)ROWS_PAIRS, n_pairs - pair0);
    const long row_elems = (long)a.heads * hd;
    const int hstride = a.x_head_stride > 0 ? a.x_head_stride : hd;
    // threads per pair: a power of two that covers head_dim in at most two passes, so that a
    // thread's (pair, column) comes from shifts and masks, not divisions
    const int tpp_log = hd > 128 ? 8 : hd > 64 ? 7 : 6;
    const int tpp = 1 << tpp_log, ppi = 256 >> tpp_log;
    const int sub = lane >> tpp_log, c0 = lane & (tpp - 1);
    // eight pairs' loads are issued before the first is stored (unconditional, from clamped
    // indices): the staging is then a few memory round trips instead of one per pair
    constexpr int U = 8;
    for (int pb = sub; pb < here; pb += ppi * U) {
        float v0[U], v1[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int pair = (int)pair0 + min(pb + u * ppi, here - 1);
            const int r = pair / a.heads;
            const int h = pair - r * a.heads;
            const float *src = a.x + (long)r * row_elems + (long)h * hstride;
            v0[u] = src[min(c0, hd - 1)];
            v1[u] = src[min(c0 + tpp, hd - 1)];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int p = pb + u * ppi;
            if (p < here) {
                if (c0 < hd) rows_lds[p * stride + c0] = v0[u];
                if (c0 + tpp < hd) rows_lds[p * stride + c0 + tpp] = v1[u];
            }
        }
    }
    // the weight and the rotations of the rows this workgroup touches: read per element below,
    // from LDS instead of one dependent global load each
    const long r_first = pair0 / a.heads;
    const int n_r = (int)((pair0 + here - 1) / a.heads - r_first) + 1;
    if (a.weight)
        for (int c = lane; c < hd; c += 256) w_s[c] = a.weight[c];
    if (a.rope)
        for (int e = lane; e < n_r * a.rope_dims; e += 256) rope_s[e] = a.rope[r_first * a.rope_dims + e];
    __syncthreads();
    if (lane < here) {
        // head_inv_rms over the lane's own pair, sixteen LDS reads in flight per round; the
        // multiplications and additions are the same, in the same order
        const float *row = rows_lds + lane * stride;
        float inv = 1.0f;
        if (a.weight) {
#pragma clang fp contract(off)
            float sum = 0.0f;
            int c = 0;
            for (; c + 16 <= hd; c += 16) {
                float v[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) v[j] = row[c + j];
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const float sq = v[j] * v[j];
                    sum = sum + sq;
                }
            }
            for (; c < hd; ++c) {
                const float sq = row[c] * row[c];
                sum = sum + sq;
            }
            const float mean_square = sum / (float)hd;
            inv = 1.0f / sqrtf(mean_square + a.eps);
        }
        inv_s[lane] = inv;
    }
    __syncthreads();
    for (int p = sub; p < here; p += ppi) {
        const int pair = (int)pair0 + p;
        const int r = pair / a.heads;
        const float *rope_row = a.rope ? rope_s + (r - r_first) * a.rope_dims : nullptr;
        const float inv = inv_s[p];
        for (int c = c0; c < hd; c += tpp)
            a.out[(long)pair * hd + c] = norm_rope_elem(rows_lds + p * stride, c, inv, a.weight ? w_s : nullptr,
                                                  rope_row, a.rope_dims, a.rope_style);
    }
}

hipError_t launch_norm_rope(const NormRopeArgs &a, hipStream_t s) {
    if (a.heads <= 0 || a.head_dim <= 0 || a.head_dim > 512) return hipErrorInvalidValue;
    const int rows = a.n_rows > 0 ? a.n_rows : 1;
    if (rows > 65535) return hipErrorInvalidValue;
    if (rows >= 4) {
        const int pairs = a.head_dim <= 128 ? 16 : 8;
        const int rows_per_wg = std::min(rows, (pairs + a.heads - 1) / a.heads + 1);
        const size_t lds = (size_t)(pairs * (a.head_dim + 1) + pairs + a.head_dim +
                                    (a.rope ? (size_t)rows_per_wg * a.rope_dims : 0)) * sizeof(float);
        const long n_pairs = (long)rows * a.heads;
        NormRopeArgs b = a;
        b.n_rows = rows;
        const dim3 grid((unsigned)((n_pairs + pairs - 1) / pairs));
        if (pairs == 16)
            hipLaunchKernelGGL(norm_rope_rows_kernel<16>, grid, dim3(256), lds, s, b);
        else
            hipLaunchKernelGGL(norm_rope_rows_kernel<8>, grid, dim3(256), lds, s, b);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(norm_rope_kernel, dim3((unsigned)a.heads, (unsigned)rows), dim3(256), 0, s, a);
    return hipGetLastError();
}

// out = ctx * sigmoid(gate) (attn_gate_f32, src/decode_resident/kernels.rs:949-959); the
// gate may sit interleaved with q in the gated q projection (gate_head_stride = 2 * head_dim).
__global__ __launch_bounds__(256) void gate_kernel(GateArgs a) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= a.heads * a.head_dim) return;
    const int h = i / a.head_dim, c = i - h * a.head_dim;
    a.out[i] = a.ctx[i] * sigmoid_gate(a.gate[(long)h * a.gate_head_stride + c]);
}

hipError_t launch_gate(const GateArgs &a, hipStream_t s) {
    const int n = a.heads * a.head_dim;
    if (n <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gate_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a);
    return hipGetLastError();
}

} // namespace skv
