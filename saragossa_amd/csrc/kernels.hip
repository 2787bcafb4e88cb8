// gfx950 kernels of the KV hot path: append into paged bf16 tiles, gather back to
// rows, split-K GQA decode attention on the matrix cores, its merge, and the plain
// three-phase attention kernel kept behind the RETI_RUST_FLASH_SDPA kill-switch.
#include "skv_internal.h"

namespace skv {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;

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
// store into the K tile, eight 2-byte stores into the transposed V tile.
// Stands in for copy_at_f32_to_bf16 (src/decode_resident/kernels.rs:1036-1044).
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void append_kernel(AppendArgs a) {
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
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (e < nd) a.v_pool[tile + v_index(g.P, r, d0 + e)] = bf16_bits(vs[e]);
    }
}

hipError_t launch_append(const AppendArgs &a, hipStream_t s) {
    const int groups = (a.g.head_dim + 7) >> 3;
    const long total = (long)a.g.kv_heads * groups * a.n_rows;
    if (total <= 0) return hipSuccess;
    long blocks = (total + 255) / 256;
    if (blocks > 65535 * 4) blocks = 65535 * 4;
    hipLaunchKernelGGL(append_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
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
// Decode attention, split-K over the context, one workgroup per (split, kv head).
//
// The GQA group's queries are staged once in LDS as bf16 hi + lo halves (q = hi + lo
// to 2^-17), already multiplied by log2(e)/sqrt(head_dim). Each of the four wavefronts
// walks its share of the pages: a 16-key K tile is eight 1 KiB loads feeding
// S^T = K . Q^T on the matrix cores (16 keys x 16 query slots), an online softmax in
// base 2 runs on the accumulator registers (lane l holds keys 4*(l/16)..+3 of query
// slot l%16, so only two cross-lane exchanges are needed for the row maximum), and
// the probabilities go straight back in as the B operand of O^T += V^T . P^T with the
// V tile stored transposed. Probabilities are also split hi + lo, so the result has
// fp32-level accuracy although the operands are bf16.
//
// The wavefronts' states are merged through LDS; with one split the workgroup writes
// the final context, otherwise a partial (o, m, l) per query head, and the last
// workgroup to arrive for a kv head merges that head's partials.
// ------------------------------------------------------------------------------------
constexpr int DEC_WAVES = 4;
constexpr int DEC_THREADS = DEC_WAVES * 64;
constexpr int DEC_MAX_SPLITS = 512;

int decode_max_splits() { return DEC_MAX_SPLITS; }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor_max(float v, int mask) {
    return fmaxf(v, __shfl_xor(v, mask, 64));
}

// Position held by slot `slot` of the cache when `len` rows have been written, or -1.
__device__ __forceinline__ long pos_of_slot(long slot, long len, int ring_rows) {
    if (ring_rows <= 0) return slot;
    if (slot >= len) return -1;
    return slot + (long)ring_rows * ((len - 1 - slot) / ring_rows);
}

template <int P>
__global__ __launch_bounds__(DEC_THREADS, 2) void decode_split_kernel(DecodeArgs a) {
    constexpr int KK = P / 32; // K-steps of the QK product, also column-tile pairs of V
    constexpr int NT = P / 16; // 16-column tiles of the output
    constexpr int OSTRIDE = P + 4;
    const Geom g = a.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int n = lane & 15; // key row inside the tile (A operand) / query slot (B, D)
    const int j = lane >> 4;
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    const int G = g.gqa;

    __shared__ __attribute__((aligned(16))) uint4 q_hi[KK * 64];
    __shared__ __attribute__((aligned(16))) uint4 q_lo[KK * 64];
    __shared__ __attribute__((aligned(16))) float xo[2][16 * OSTRIDE];
    __shared__ float xm[2][16];
    __shared__ float xl[2][16];
    __shared__ float wts[DEC_MAX_SPLITS];
    __shared__ int last_flag;

    const int pb0 = a.page_first + (int)(((long)split * a.n_pages) / a.splits);
    const int pb1 = a.page_first + (int)(((long)(split + 1) * a.n_pages) / a.splits);

    // ---- stage the queries of this kv head -------------------------------------------
    for (int idx = tid; idx < KK * 64; idx += DEC_THREADS) {
        const int kk = idx >> 6;
        const int jj = (idx >> 4) & 3;
        const int qn = idx & 15;
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            uint32_t h2 = 0, l2 = 0;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int d = kk * 32 + jj * 8 + e2 * 2 + h;
                float v = 0.0f;
                if (qn < G && d < g.head_dim)
                    v = a.q[(long)(kvh * G + qn) * g.head_dim + d] * a.qscale;
                const uint16_t hb = bf16_bits(v);
                const uint16_t lb = bf16_bits(v - bf16_to_f32(hb));
                h2 |= (uint32_t)hb << (16 * h);
                l2 |= (uint32_t)lb << (16 * h);
            }
            hi[e2] = h2;
            lo[e2] = l2;
        }
        q_hi[idx] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        q_lo[idx] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    }
    __syncthreads();

    float4_t o[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) o[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY; // running maximum of query slot n (same in the 4 lanes sharing n)
    float l_run = 0.0f;      // this lane's share of the running sum

    for (int pb = pb0 + wave; pb < pb1; pb += DEC_WAVES) {
        const int page = __builtin_amdgcn_readfirstlane(a.table[pb]);
        const long tile = (long)page * g.page_elems + (long)kvh * g.tile_elems;
        const uint4 *kp = reinterpret_cast<const uint4 *>(a.k_pool + tile) + lane;
        const uint4 *vp = reinterpret_cast<const uint4 *>(a.v_pool + tile) + lane;
        uint4 kreg[KK], vreg[KK];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) kreg[kk] = kp[kk * 64];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) vreg[kk] = vp[kk * 64];

        float4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const bf16x8_t kv = __builtin_bit_cast(bf16x8_t, kreg[kk]);
            const bf16x8_t qh = __builtin_bit_cast(bf16x8_t, q_hi[kk * 64 + lane]);
            const bf16x8_t ql = __builtin_bit_cast(bf16x8_t, q_lo[kk * 64 + lane]);
            s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv, qh, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv, ql, s, 0, 0, 0);
        }
        // mask keys outside [window_start, len)
        float sv[4];
        float m_blk = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const long slot = (long)pb * 16 + j * 4 + i;
            const long pos = pos_of_slot(slot, a.len, g.ring_rows);
            const bool ok = pos >= a.window_start && pos < a.len;
            sv[i] = ok ? s[i] : -INFINITY;
            m_blk = fmaxf(m_blk, sv[i]);
        }
        m_blk = xor_max(m_blk, 16);
        m_blk = xor_max(m_blk, 32);
        const float m_new = fmaxf(m_run, m_blk);
        const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        float p[4];
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            p[i] = fast_exp2(sv[i] - m_safe);
            psum += p[i];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
            for (int t = 0; t < NT; ++t) o[t] *= alpha;
        }
        short4_t ph, pl;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint16_t hb = bf16_bits(p[i]);
            const uint16_t lb = bf16_bits(p[i] - bf16_to_f32(hb));
            ph[i] = (short)hb;
            pl[i] = (short)lb;
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const short4_t v0 = __builtin_bit_cast(short4_t, make_uint2(vreg[kk].x, vreg[kk].y));
            const short4_t v1 = __builtin_bit_cast(short4_t, make_uint2(vreg[kk].z, vreg[kk].w));
            o[2 * kk] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v0, ph, o[2 * kk], 0, 0, 0);
            o[2 * kk] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v0, pl, o[2 * kk], 0, 0, 0);
            o[2 * kk + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v1, ph, o[2 * kk + 1], 0, 0, 0);
            o[2 * kk + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v1, pl, o[2 * kk + 1], 0, 0, 0);
        }
    }

    // this lane's share of the sum -> the query slot's sum
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);

    // ---- merge the four wavefronts: (1,3) -> (0,2), then 2 -> 0 -------------------------
#pragma unroll
    for (int round = 0; round < 2; ++round) {
        const int stride = round == 0 ? 1 : 2;
        const bool sender = round == 0 ? (wave & 1) : (wave == 2);
        const bool receiver = round == 0 ? !(wave & 1) : (wave == 0);
        const int slot = round == 0 ? (wave >> 1) : 0;
        if (sender) {
            if (n < G) {
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    *reinterpret_cast<float4_t *>(&xo[slot][n * OSTRIDE + t * 16 + j * 4]) = o[t];
                if (j == 0) {
                    xm[slot][n] = m_run;
                    xl[slot][n] = l_run;
                }
            }
        }
        __syncthreads();
        if (receiver && n < G) {
            const float m2 = xm[slot][n];
            const float l2 = xl[slot][n];
            const float m_new = fmaxf(m_run, m2);
            const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
            const float a1 = fast_exp2(m_run - m_safe);
            const float a2 = fast_exp2(m2 - m_safe);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float4_t o2 =
                    *reinterpret_cast<const float4_t *>(&xo[slot][n * OSTRIDE + t * 16 + j * 4]);
                o[t] = o[t] * a1 + o2 * a2;
            }
            l_run = l_run * a1 + l2 * a2;
            m_run = m_new;
        }
        __syncthreads();
        (void)stride;
    }

    // ---- wavefront 0 holds the workgroup's result ------------------------------------------
    if (a.splits == 1) {
        if (wave == 0 && n < G) {
            const float inv = 1.0f / l_run;
            float *dst = a.out + (long)(kvh * G + n) * g.head_dim;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = t * 16 + j * 4 + i;
                    if (d < g.head_dim) dst[d] = o[t][i] * inv;
                }
        }
        return;
    }
    if (wave == 0 && n < G) {
        const long pidx = ((long)kvh * a.splits + split) * G + n;
        float *dst = a.part_o + pidx * g.head_dim;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = t * 16 + j * 4 + i;
                if (d < g.head_dim) dst[d] = o[t][i];
            }
        if (j == 0) {
            a.part_m[pidx] = m_run;
            a.part_l[pidx] = l_run;
        }
    }
    // ---- the last workgroup of this kv head merges its partials ---------------------------
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned prev = atomicAdd(&a.counters[kvh], 1u);
        const int is_last = prev == (unsigned)(a.splits - 1);
        if (is_last) a.counters[kvh] = 0; // ready for the next launch
        last_flag = is_last;
    }
    __syncthreads();
    if (!last_flag) return;
    __threadfence();
    for (int gq = 0; gq < G; ++gq) {
        const long base = ((long)kvh * a.splits) * G + gq;
        float mx = -INFINITY;
        for (int sidx = tid; sidx < a.splits; sidx += DEC_THREADS)
            mx = fmaxf(mx, __builtin_nontemporal_load(&a.part_m[base + (long)sidx * G]));
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        __syncthreads(); // previous head's readers are done with wts / xm
        if (lane == 0) xm[0][wave] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(xm[0][0], xm[0][1]), fmaxf(xm[0][2], xm[0][3]));
        const float m_safe = mx == -INFINITY ? 0.0f : mx;
        float lsum = 0.0f;
        for (int sidx = tid; sidx < a.splits; sidx += DEC_THREADS) {
            const float w = fast_exp2(__builtin_nontemporal_load(&a.part_m[base + (long)sidx * G]) - m_safe);
            wts[sidx] = w;
            lsum += w * __builtin_nontemporal_load(&a.part_l[base + (long)sidx * G]);
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) lsum += __shfl_xor(lsum, off, 64);
        if (lane == 0) xl[0][wave] = lsum;
        __syncthreads();
        const float inv = 1.0f / (xl[0][0] + xl[0][1] + xl[0][2] + xl[0][3]);
        for (int d = tid; d < g.head_dim; d += DEC_THREADS) {
            float acc = 0.0f;
            const float *src = a.part_o + base * g.head_dim + d;
            for (int sidx = 0; sidx < a.splits; ++sidx)
                acc += wts[sidx] * __builtin_nontemporal_load(src + (long)sidx * G * g.head_dim);
            a.out[(long)(kvh * G + gq) * g.head_dim + d] = acc * inv;
        }
    }
}

hipError_t launch_decode(const DecodeArgs &a, hipStream_t s) {
    dim3 grid((unsigned)a.splits, (unsigned)a.g.kv_heads);
    switch (a.g.P) {
    case 32: hipLaunchKernelGGL(decode_split_kernel<32>, grid, dim3(DEC_THREADS), 0, s, a); break;
    case 64: hipLaunchKernelGGL(decode_split_kernel<64>, grid, dim3(DEC_THREADS), 0, s, a); break;
    case 128: hipLaunchKernelGGL(decode_split_kernel<128>, grid, dim3(DEC_THREADS), 0, s, a); break;
    case 256: hipLaunchKernelGGL(decode_split_kernel<256>, grid, dim3(DEC_THREADS), 0, s, a); break;
    default: return hipErrorInvalidValue;
    }
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
        float dot = 0.0f;
        for (int d = 0; d < g.head_dim; ++d)
            dot = __fadd_rn(dot, __fmul_rn(q[d], bf16_to_f32(kt[k_index(g.P, r, d)])));
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
            acc = __fadd_rn(acc, __fmul_rn(pr, bf16_to_f32(vt[v_index(g.P, r, d)])));
        }
        a.out[(long)h * g.head_dim + d] = acc;
    }
}

hipError_t launch_naive(const NaiveArgs &a, hipStream_t s) {
    hipLaunchKernelGGL(naive_kernel, dim3((unsigned)a.g.q_heads), dim3(256), 0, s, a);
    return hipGetLastError();
}

} // namespace skv
