// gfx950 kernels of the KV hot path, part 2: split-K GQA decode attention over the
// paged bf16 cache on the matrix cores, and the merge of its partials.
#include "skv_internal.h"

namespace skv {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

__device__ __forceinline__ uint16_t bf16_bits(float v) {
    uint32_t b = __float_as_uint(v);
    uint32_t lsb = (b >> 16) & 1u;
    return (uint16_t)((b + 0x7fffu + lsb) >> 16);
}
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int DEC_MAX_SPLITS = 512;
constexpr size_t LDS_BYTES = 160 * 1024; // of a gfx950 compute unit
int decode_max_splits() { return DEC_MAX_SPLITS; }


// ------------------------------------------------------------------------------------
// Decode attention, split-K over the context, one workgroup per (split, kv head).
//
// The GQA group's queries are staged once in LDS as bf16 hi + lo halves (q = hi + lo
// to 2^-17), already multiplied by log2(e)/sqrt(head_dim). Each wavefront walks its
// share of the pages. A 16-key K tile arrives as 1 KiB loads from consecutive addresses
// and feeds S^T = K . Q^T on the matrix cores (16 keys x 16 query slots). The online
// softmax, in base 2, runs on the accumulator registers: lane l holds keys
// 4*(l/16)..+3 of query slot l%16, so the row maximum needs two cross-lane exchanges
// and the row sum none until the end. The probabilities go straight back in as the B
// operand of O^T += V^T . P^T, the V tile being stored transposed. Probabilities are
// split hi + lo as well, so the result has fp32-level accuracy with bf16 operands.
//
// K registers are refilled right after the QK product that consumed them and V
// registers right after the PV product, so each wavefront keeps about one page in
// flight with a single K and a single V buffer; two wavefronts per SIMD hide the rest.
//
// At the end every wavefront writes its (o, m, l) to LDS and the whole workgroup
// reduces them column-parallel: with one split that is the final context, otherwise a
// partial per query slot for the merge kernel.
//
// The same kernel serves chunked prefill over the cache: with n_queries > 1 the query
// slots are (query row, head of the group) pairs, 16 per workgroup (grid z), and slot
// (i, g) attends positions up to len - n_queries + i, the causal limit of the i-th new
// row (the per-row loop of cached_attention_prefill_rows,
// src/decoder/attention_ops.rs:976-1017, as one launch).
// ------------------------------------------------------------------------------------
template <int KK>
__device__ __forceinline__ void load_k(uint4 (&k)[KK], const DecodeArgs &a, int page, int kvh,
                                       int lane) {
    const long tile = (long)page * a.g.page_elems + (long)kvh * a.g.tile_elems;
    const u32x4_t *kp = reinterpret_cast<const u32x4_t *>(a.k_pool + tile) + lane;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) k[kk] = __builtin_bit_cast(uint4, __builtin_nontemporal_load(kp + kk * 64));
}
template <int KK>
__device__ __forceinline__ void load_v(uint4 (&v)[KK], const DecodeArgs &a, int page, int kvh,
                                       int lane) {
    const long tile = (long)page * a.g.page_elems + (long)kvh * a.g.tile_elems;
    const u32x4_t *vp = reinterpret_cast<const u32x4_t *>(a.v_pool + tile) + lane;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) v[kk] = __builtin_bit_cast(uint4, __builtin_nontemporal_load(vp + kk * 64));
}

// MQ = false is the decode case (one query row, at most 16 heads per group): query slot ==
// head of the group, which spares the integer divisions of the general slot -> (row, head)
// mapping.
// PRE = true fuses the step before the cache (decode only): q and the appended k row arrive
// raw, and every workgroup applies the per-head RMSNorm and the rotation of the position to
// the rows it uses, in LDS, while its first page is in flight.
template <int P, int WAVES, bool MQ, bool PRE>
__device__ __forceinline__ void decode_split_body(const DecodeArgs &a, const int split, const int kvh,
                                                  const int tile_z) {
    constexpr int THREADS = WAVES * 64;
    constexpr int KK = P / 32; // K-steps of the QK product, also column-tile pairs of V
    constexpr int NT = P / 16; // 16-column tiles of the output
    constexpr int OSTRIDE = P + 4;
    const Geom g = a.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15; // key row inside the tile (A operand) / query slot (B, D)
    const int j = lane >> 4;
    const int tile = MQ ? tile_z : 0;
    const int q_stride = (!MQ && a.q_head_stride > 0) ? a.q_head_stride : g.head_dim;
    const int G = g.gqa;
    const int C = MQ ? a.n_queries : 1;
    const int n_slots = C * G;
    const int rows = min(16, n_slots - tile * 16); // query slots of this workgroup
    // this lane's query slot in the B and D operand layouts
    const int my_slot = min(tile * 16 + n, n_slots - 1);
    const int my_q = MQ ? my_slot / G : 0;
    const int my_pos = a.q_pos0 + my_q;                 // position of the slot's query row
    const int my_limit = min(my_pos, a.limit_cap);      // last position the slot attends
    const int my_ws = a.window > 0 ? max(a.window_start, my_pos + 1 - a.window) : a.window_start;
    // extremes over the workgroup's slots
    const int qrow_lo = MQ ? (tile * 16) / G : 0;
    const int qrow_hi = MQ ? (tile * 16 + rows - 1) / G : 0;
    const int lim_lo = min(a.q_pos0 + qrow_lo, a.limit_cap);
    const int lim_hi = min(a.q_pos0 + qrow_hi, a.limit_cap);
    const int ws_lo = a.window > 0 ? max(a.window_start, a.q_pos0 + qrow_lo + 1 - a.window) : a.window_start;
    const int ws_hi = a.window > 0 ? max(a.window_start, a.q_pos0 + qrow_hi + 1 - a.window) : a.window_start;

    extern __shared__ __attribute__((aligned(16))) uint4 smem[];
    uint4 *q_hi = smem;
    uint4 *q_lo = smem + KK * 64;
    uint16_t *new_k = reinterpret_cast<uint16_t *>(smem + 2 * KK * 64); // [P] appended row
    uint16_t *new_v = new_k + P;
    // PRE: raw and finished rows of the group's queries plus the new k row, weights, rotation
    constexpr int PS = P + 1;      // row stride: lanes walking different rows hit different banks
    constexpr int PRE_ROWS = 17;   // 16 query slots + the k row
    float *pre_raw = reinterpret_cast<float *>(new_v + P); // [PRE_ROWS][PS]
    float *pre_out = pre_raw + PRE_ROWS * PS;              // [PRE_ROWS][PS]
    float *pre_wq = pre_out + PRE_ROWS * PS;               // [P]
    float *pre_wk = pre_wq + P;                            // [P]
    float *pre_rope = pre_wk + P;                          // [P]: (cos, sin) pairs
    float *pre_inv = pre_rope + P;                         // [PRE_ROWS] (+5 keeps pre_sq 16-byte aligned)
    constexpr int SQS = P + 4;                             // 16-byte aligned rows, conflict-free
    float *pre_sq = pre_inv + PRE_ROWS + 5;                // [PRE_ROWS][SQS]: squares, zero padded

    // pages this workgroup's slots can see, divided among the splits
    const int page_lo = g.ring_rows > 0 ? 0 : ws_lo >> 4;
    const int page_hi = g.ring_rows > 0 ? a.n_pages : (lim_hi >> 4) + 1;
    // (32-bit arithmetic: pages * splits stays far below 2^31)
    const unsigned span = (unsigned)(page_hi - page_lo);
    const int pb0 = page_lo + (int)(((unsigned)split * span) / (unsigned)a.splits);
    const int pb1 = page_lo + (int)(((unsigned)(split + 1) * span) / (unsigned)a.splits);
    // this wavefront walks pages pb0 + wave + it * WAVES, it = 0 .. n_it-1
    const int n_it = pb1 - pb0 > wave ? (pb1 - pb0 - wave + WAVES - 1) / WAVES : 0;
    // Every other split, the last one among them, walks its pages starting from the middle of
    // its range (rot .. n_it-1, then 0 .. rot-1); any order gives the same sums up to rounding.
    // Two things are gained. The last split holds the newest page, the one the previous steps'
    // appends wrote into, and is the split with a page more than the others when the pages do
    // not divide: read at the end of that workgroup's chain, the newest page made it the
    // slowest of the launch (176 against 167 us per token at 32768 rows of config 2, as much
    // as the whole surplus page had been found to cost); read early, its latency is covered.
    // And with pages laid out in order (an identity block table) all workgroups otherwise ask
    // for addresses that share their middle bits at the same time (185 against 181 us). Only
    // where every wavefront has two pages or more: on short launches (config 1: four or five
    // pages per workgroup) it costs 2 %. The f32 kernel, tried the same way, lost 1.5 %.
    const bool turns = ((split ^ (a.splits - 1)) & 1) == 0;
    const int rot = (turns && pb1 - pb0 >= 2 * WAVES && n_it <= 64) ? (n_it >> 1) : 0;
    auto turned = [&](int it) __attribute__((always_inline)) {
        const int r = it + rot;
        return r >= n_it ? r - n_it : r;
    };

    // Fused append: the workgroup whose range holds the page of the new row rounds that
    // row to bf16, stores it into the pools for later steps and keeps it in LDS; the
    // wavefront that walks the page patches its registers from there, so nothing is read
    // back from memory in this launch. The row is fetched here, ahead of the pages.
    const int pb_new = a.new_slot >> 4;
    const int r_new = a.new_slot & 15;
    const bool appends = a.k_new != nullptr && C == 1 && pb_new >= pb0 && pb_new < pb1;
    // elements tid (and tid + THREADS where the head is wider than the workgroup) of the new
    // row of this kv head
    constexpr int NE = (P + THREADS - 1) / THREADS;
    float k_rows[NE], v_rows[NE];
#pragma unroll
    for (int u = 0; u < NE; ++u) {
        k_rows[u] = 0.0f;
        v_rows[u] = 0.0f;
        if (appends && tid + u * THREADS < g.head_dim) {
            k_rows[u] = a.k_new[kvh * g.head_dim + tid + u * THREADS];
            v_rows[u] = a.v_new[kvh * g.head_dim + tid + u * THREADS];
        }
    }
    // PRE: raw query rows of the group (and the raw k row, already in k_row)
    constexpr int PRE_U = PRE ? (16 * P + THREADS - 1) / THREADS : 1;
    float pre_q[PRE_U];
    float pre_w0[NE], pre_w1[NE], pre_r[NE];
    if (PRE) {
#pragma unroll
        for (int u = 0; u < PRE_U; ++u) {
            const int e = tid + u * THREADS;
            const int r = e / P, c = e % P;
            pre_q[u] = (r < rows && c < g.head_dim) ? a.q[(long)(kvh * G + r) * q_stride + c] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < NE; ++u) {
            const int d = tid + u * THREADS;
            pre_w0[u] = (a.q_norm_w && d < g.head_dim) ? a.q_norm_w[d] : 1.0f;
            pre_w1[u] = (a.k_norm_w && d < g.head_dim) ? a.k_norm_w[d] : 1.0f;
            pre_r[u] = (a.rope && d < a.rope_dims) ? a.rope[d] : 0.0f;
        }
    }

    // Block-table entries of the next 64 iterations, one per lane.
    int ids = 0;
    auto fetch_ids = [&](int chunk) __attribute__((always_inline)) {
        const int it = chunk * 64 + lane;
        ids = it < n_it ? a.table[pb0 + wave + it * WAVES] : 0;
    };
    auto page_id = [&](int it) __attribute__((always_inline)) {
        if (n_it <= 64) return __builtin_amdgcn_readlane(ids, turned(it)); // one register holds them all
        if ((it & 63) == 0 && it > 0) fetch_ids(it >> 6);
        return __builtin_amdgcn_readlane(ids, it & 63);
    };
    fetch_ids(0);

    // ---- queries of this kv head: load, start the first page, then stage to LDS ----------
    constexpr int QI = (KK * 64 + THREADS - 1) / THREADS;
    float qv[QI][8];
#pragma unroll
    for (int u = 0; u < (PRE ? 0 : QI); ++u) {
        const int idx = min(tid + u * THREADS, KK * 64 - 1);
        const int kk = idx >> 6;
        const int jj = (idx >> 4) & 3;
        const int qs = min(tile * 16 + (idx & 15), n_slots - 1);
        const float *qrow = MQ ? a.q + ((long)(qs / G) * g.q_heads + kvh * G + qs % G) * g.head_dim
                               : a.q + (long)(kvh * G + qs) * q_stride;
        if (a.q_vec) { // two 16-byte loads from a clamped address (dims past head_dim are zeroed below)
            const float4_t *qp = reinterpret_cast<const float4_t *>(qrow + min(kk * 32 + jj * 8, g.head_dim - 8));
            const float4_t x0 = qp[0], x1 = qp[1];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                qv[u][e] = x0[e];
                qv[u][4 + e] = x1[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) qv[u][e] = qrow[min(kk * 32 + jj * 8 + e, g.head_dim - 1)];
        }
    }
    // Unconditional (a wavefront without pages reads physical page 0 and ignores it): a
    // conditional load here makes the compiler wait for these pages before the queries.
    // The first page's table entry comes through the scalar unit (the address is the same in
    // every lane): that read is counted apart from the vector loads above, so the first K/V
    // request waits for it alone and not for the queries, nor, in the workgroup that
    // appends, for the new row, which no other workgroup has pulled into a cache.
    uint4 kr[KK], vr[KK];
    {
        typedef const __attribute__((address_space(4))) int32_t *const_i32_ptr;
        const int pg = reinterpret_cast<const_i32_ptr>(reinterpret_cast<uintptr_t>(a.table))[min(pb0 + wave + rot * WAVES, max(page_hi - 1, 0))];
        load_k<KK>(kr, a, pg, kvh, lane);
        load_v<KK>(vr, a, pg, kvh, lane);
    }
    if (PRE) {
        auto sq_of = [](float x) {
#pragma clang fp contract(off)
            return x * x;
        };
        // rows 0..rows-1: the group's queries; row `rows`: the new k row (appending workgroup)
#pragma unroll
        for (int u = 0; u < PRE_U; ++u) {
            const int e = tid + u * THREADS;
            const int r = e / P, c = e % P;
            if (r < rows) {
                pre_raw[r * PS + c] = pre_q[u];
                pre_sq[r * SQS + c] = sq_of(pre_q[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < NE; ++u) {
            const int d = tid + u * THREADS;
            if (d < P) {
                pre_raw[rows * PS + d] = k_rows[u];
                pre_sq[rows * SQS + d] = sq_of(k_rows[u]);
                pre_wq[d] = pre_w0[u];
                pre_wk[d] = pre_w1[u];
                pre_rope[d] = pre_r[u];
            }
        }
        __syncthreads();
        const int n_rows = rows + (appends ? 1 : 0);
        if (tid < n_rows) {
            const bool is_k = tid == rows;
            const bool has_norm = is_k ? a.k_norm_w != nullptr : a.q_norm_w != nullptr;
            pre_inv[tid] = has_norm ? head_inv_rms_sq(pre_sq + tid * SQS, P, g.head_dim, a.eps) : 1.0f;
        }
        __syncthreads();
        const float *rope = a.rope ? pre_rope : nullptr;
        for (int e = tid; e < n_rows * P; e += THREADS) {
            const int r = e / P, c = e % P;
            if (c < g.head_dim) {
                const bool is_k = r == rows;
                const float *w = is_k ? (a.k_norm_w ? pre_wk : nullptr) : (a.q_norm_w ? pre_wq : nullptr);
                pre_out[r * PS + c] = norm_rope_elem(pre_raw + r * PS, c, pre_inv[r], w, rope,
                                                     a.rope_dims, a.rope_style);
            }
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < NE; ++u)
            if (appends && tid + u * THREADS < g.head_dim) k_rows[u] = pre_out[rows * PS + tid + u * THREADS];
    }
    if (appends) {
        // the page's physical id comes with the arguments: a table lookup here would wait for
        // every load issued before it, the first K/V page included
        const long tile_at = (long)a.new_page * g.page_elems + (long)kvh * g.tile_elems;
#pragma unroll
        for (int u = 0; u < NE; ++u) {
            const int d = tid + u * THREADS;
            if (d < P) {
                uint16_t kb = 0, vb = 0;
                if (d < g.head_dim) {
                    kb = bf16_bits(k_rows[u]);
                    vb = bf16_bits(v_rows[u]);
                    const_cast<uint16_t *>(a.k_pool)[tile_at + k_index(P, r_new, d)] = kb;
                    const_cast<uint16_t *>(a.v_pool)[tile_at + v_index(P, r_new, d)] = vb;
                }
                new_k[d] = kb;
                new_v[d] = vb;
            }
        }
    }
    if (PRE) {
#pragma unroll
        for (int u = 0; u < QI; ++u) {
            const int idx = min(tid + u * THREADS, KK * 64 - 1);
            const int kk = idx >> 6;
            const int jj = (idx >> 4) & 3;
            const int qs = min(idx & 15, rows - 1);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                qv[u][e] = pre_out[qs * PS + min(kk * 32 + jj * 8 + e, g.head_dim - 1)];
        }
    }
#pragma unroll
    for (int u = 0; u < QI; ++u) {
        const int idx = tid + u * THREADS;
        if (idx < KK * 64) {
            const int kk = idx >> 6;
            const int jj = (idx >> 4) & 3;
            const bool row_ok = (idx & 15) < rows;
            uint32_t hi[4], lo[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                uint32_t h2 = 0, l2 = 0;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int d = kk * 32 + jj * 8 + e2 * 2 + h;
                    const float v = (row_ok && d < g.head_dim) ? qv[u][e2 * 2 + h] * a.qscale : 0.0f;
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
    }
    __syncthreads();

    float4_t o[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) o[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY; // running maximum of query slot n (same in the 4 lanes sharing n)
    float l_run = 0.0f;      // this lane's share of the running sum

    // S^T = K . Q^T for the page in kr: two independent accumulator chains (hi, lo halves)
    auto qk = [&]() __attribute__((always_inline)) {
        float4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const bf16x8_t kv = __builtin_bit_cast(bf16x8_t, kr[kk]);
            const bf16x8_t qh = __builtin_bit_cast(bf16x8_t, q_hi[kk * 64 + lane]);
            const bf16x8_t ql = __builtin_bit_cast(bf16x8_t, q_lo[kk * 64 + lane]);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv, qh, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv, ql, s1, 0, 0, 0);
        }
        return s0 + s1;
    };
    // online softmax step on the four scores of this lane; returns P^T as bf16 hi / lo
    auto softmax_step = [&](float4_t s, int pb, short4_t &ph, short4_t &pl)
                            __attribute__((always_inline)) {
        // Only pages that touch the window start, the end of the cache or (ring layers) any
        // page at all can hold keys outside [window_start, len).
        const int first_slot = pb * 16;
        const bool interior = g.ring_rows == 0 && first_slot >= ws_hi && first_slot + 16 <= lim_lo + 1;
        if (!interior) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int slot = first_slot + j * 4 + i;
                int pos = slot;
                if (g.ring_rows > 0)
                    pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
                const bool ok = pos >= my_ws && pos <= my_limit;
                s[i] = ok ? s[i] : -INFINITY;
            }
        }
        float m_blk = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
        m_blk = rows_max(m_blk);
        const float m_new = fmaxf(m_run, m_blk);
        const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float p = fast_exp2(s[i] - m_safe);
            psum += p;
            const uint16_t hb = bf16_bits(p);
            const uint16_t lb = bf16_bits(p - bf16_to_f32(hb));
            ph[i] = (short)hb;
            pl[i] = (short)lb;
        }
        l_run = l_run * alpha + psum;
        // A slot that has seen no key yet holds zeros: no rescale for it (the first page of
        // every wavefront would otherwise walk all its accumulator registers for nothing, which
        // on a launch of one page per wavefront is a visible part of the whole).
        const bool rescale = alpha != 1.0f && m_run != -INFINITY;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(rescale)) {
#pragma unroll
            for (int t = 0; t < NT; ++t) o[t] *= alpha;
        }
    };
    auto pv = [&](short4_t ph, short4_t pl) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const short4_t v0 = __builtin_bit_cast(short4_t, make_uint2(vr[kk].x, vr[kk].y));
            const short4_t v1 = __builtin_bit_cast(short4_t, make_uint2(vr[kk].z, vr[kk].w));
            o[2 * kk] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v0, ph, o[2 * kk], 0, 0, 0);
            o[2 * kk + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v1, ph, o[2 * kk + 1], 0, 0, 0);
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const short4_t v0 = __builtin_bit_cast(short4_t, make_uint2(vr[kk].x, vr[kk].y));
            const short4_t v1 = __builtin_bit_cast(short4_t, make_uint2(vr[kk].z, vr[kk].w));
            o[2 * kk] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v0, pl, o[2 * kk], 0, 0, 0);
            o[2 * kk + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v1, pl, o[2 * kk + 1], 0, 0, 0);
        }
    };

    // the page that receives the appended row takes it from LDS instead of memory
    auto patch_k = [&](int pb) __attribute__((always_inline)) {
        if (appends && pb == pb_new && n == r_new) {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk)
                kr[kk] = *reinterpret_cast<const uint4 *>(new_k + kk * 32 + j * 8);
        }
    };
    auto patch_v = [&](int pb) __attribute__((always_inline)) {
        if (appends && pb == pb_new && j == (r_new >> 2)) {
            const int i = r_new & 3;
            const uint32_t keep = (i & 1) ? 0x0000ffffu : 0xffff0000u;
            const int sh = (i & 1) * 16;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const uint32_t b0 = (uint32_t)new_v[kk * 32 + n] << sh;
                const uint32_t b1 = (uint32_t)new_v[kk * 32 + 16 + n] << sh;
                if (i < 2) {
                    vr[kk].x = (vr[kk].x & keep) | b0;
                    vr[kk].z = (vr[kk].z & keep) | b1;
                } else {
                    vr[kk].y = (vr[kk].y & keep) | b0;
                    vr[kk].w = (vr[kk].w & keep) | b1;
                }
            }
        }
    };

    // Keys that no query slot of the workgroup attends (rows at or past the cache's length
    // after a rollback, ring rows not yet or no longer valid, rows before the window) get zero
    // probability, but 0 x NaN and 0 x Inf are NaN: their V values are cleared in the
    // registers as well, so whatever bits such a row holds never reach a context (the
    // reference never reads those rows, src/decode_resident/kernels.rs:11-88). Only pages
    // at the edges of the attended range, and ring pages, take the branch.
    auto mask_v = [&](int pb) __attribute__((always_inline)) {
        const int first_slot = pb * 16;
        const bool inside = g.ring_rows == 0 && first_slot >= ws_lo && first_slot + 16 <= lim_hi + 1;
        if (!inside) {
            uint32_t keep[2] = {0u, 0u}; // keys 4j, 4j+1 | keys 4j+2, 4j+3: 16 bits each
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int slot = first_slot + j * 4 + i;
                int pos = slot;
                if (g.ring_rows > 0)
                    pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
                if (pos >= ws_lo && pos <= lim_hi) keep[i >> 1] |= 0xffffu << ((i & 1) * 16);
            }
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                vr[kk].x &= keep[0];
                vr[kk].z &= keep[0];
                vr[kk].y &= keep[1];
                vr[kk].w &= keep[1];
            }
        }
    };

    // Steady state is unconditional (the compiler can then wait for exactly the loads it
    // needs); the last page is peeled.
    for (int it = 0; it + 1 < n_it; ++it) {
        const int pb = pb0 + wave + turned(it) * WAVES;
        const int next = page_id(it + 1);
        patch_k(pb);
        const float4_t s = qk();
        load_k<KK>(kr, a, next, kvh, lane);
        short4_t ph, pl;
        softmax_step(s, pb, ph, pl);
        patch_v(pb);
        mask_v(pb);
        pv(ph, pl);
        load_v<KK>(vr, a, next, kvh, lane);
    }
    if (n_it > 0) {
        const int pb = pb0 + wave + turned(n_it - 1) * WAVES;
        patch_k(pb);
        const float4_t s = qk();
        short4_t ph, pl;
        softmax_step(s, pb, ph, pl);
        patch_v(pb);
        mask_v(pb);
        pv(ph, pl);
    }

    // this lane's share of the sum -> the query slot's sum
    l_run = rows_sum(l_run);

    // ---- all wavefronts publish (o, m, l); the workgroup reduces them, four columns per thread.
    // Where the LDS holds both, the exchange has an area of its own behind the staged queries,
    // so a wavefront writes its state as soon as it has finished, without waiting for the
    // others to stop reading the queries; otherwise the staging area is reused after a barrier.
    if (a.xchg_off == 0) __syncthreads();
    float *xo = reinterpret_cast<float *>(reinterpret_cast<char *>(smem) + a.xchg_off); // [WAVES][rows][OSTRIDE]
    float *xm = xo + WAVES * rows * OSTRIDE;            // [WAVES][rows]
    float *xl = xm + WAVES * rows;                      // [WAVES][rows]
    if (n < rows) {
        float *dst = xo + (wave * rows + n) * OSTRIDE + j * 4;
#pragma unroll
        for (int t = 0; t < NT; ++t) *reinterpret_cast<float4_t *>(dst + t * 16) = o[t];
        if (j == 0) {
            xm[wave * rows + n] = m_run;
            xl[wave * rows + n] = l_run;
        }
    }
    __syncthreads();
    constexpr int P4 = P / 4;
    const bool vec_ok = (g.head_dim & 3) == 0;
    for (int u = tid; u < rows * P4; u += THREADS) {
        const int row = u / P4;
        const int c4 = (u - row * P4) * 4;
        float mw[WAVES];
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            mw[w] = xm[w * rows + row];
            mx = fmaxf(mx, mw[w]);
        }
        const float m_safe = mx == -INFINITY ? 0.0f : mx;
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
        float lsum = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float wgt = fast_exp2(mw[w] - m_safe);
            acc += wgt * *reinterpret_cast<const float4_t *>(&xo[(w * rows + row) * OSTRIDE + c4]);
            lsum += wgt * xl[w * rows + row];
        }
        if (c4 >= g.head_dim) continue;
        const int slot = tile * 16 + row;
        float *dst;
        if (a.splits_total == 1) {
            acc *= 1.0f / lsum;
            if (!MQ && a.gate) {
                const float *gp = a.gate + (long)(kvh * G + slot) * q_stride + c4;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (c4 + i < g.head_dim) acc[i] *= sigmoid_gate(gp[i]);
            }
            dst = a.out + (MQ ? ((long)(slot / G) * g.q_heads + kvh * G + slot % G)
                              : (long)(kvh * G + slot)) * g.head_dim + c4;
        } else {
            const long pidx = ((long)kvh * a.splits_total + a.split_base + split) * n_slots + slot;
            dst = a.part_o + pidx * g.head_dim + c4;
            if (c4 == 0) {
                a.part_m[pidx] = mx;
                a.part_l[pidx] = lsum;
            }
        }
        if (vec_ok) {
            // partials are read once by another kernel: keep them out of the caches
            if (a.splits_total == 1) *reinterpret_cast<float4_t *>(dst) = acc;
            else __builtin_nontemporal_store(acc, reinterpret_cast<float4_t *>(dst));
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (c4 + i < g.head_dim) dst[i] = acc[i];
        }
    }
}

template <int P, int WAVES, bool MQ, bool PRE>
__global__ __launch_bounds__(WAVES * 64) void decode_split_kernel(DecodeArgs a) {
    decode_split_body<P, WAVES, MQ, PRE>(a, blockIdx.x, blockIdx.y, blockIdx.z);
}

// Several independent sequences of the same model layer in one launch: grid z is the
// sequence, grid x covers the largest split count and the others leave early.
template <int P, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void decode_split_batch_kernel(DecodeBatchArgs b) {
    const DecodeArgs &a = b.seq[blockIdx.z];
    if ((int)blockIdx.x >= a.splits) return;
    decode_split_body<P, WAVES, false, false>(a, blockIdx.x, blockIdx.y, 0);
}

// ------------------------------------------------------------------------------------
// Merge of the split-K partials: one workgroup per (query head, 16 columns). The 256
// threads are 16 columns x 16 split lanes. Every thread issues all its loads (o, m, l
// of its splits) at once, so the kernel costs one round trip to memory; the maximum
// and the two sums are then reduced across the split lanes through LDS.
// Stands in for attention_decode_2pass_2 (src/decode_resident/kernels.rs:801-917).
// ------------------------------------------------------------------------------------
constexpr int MERGE_PER_LANE_MAX = DEC_MAX_SPLITS / 16;

// MERGE_PER_LANE: splits each of the 16 split lanes covers, the smallest power of two that fits
template <int MERGE_PER_LANE>
__device__ __forceinline__ void decode_merge_body(const DecodeArgs &a) {
    const Geom g = a.g;
    const int n_slots = a.n_queries * g.gqa;
    const int kvh = blockIdx.x / n_slots;
    const int slot = blockIdx.x - kvh * n_slots;
    const long h = (long)(slot / g.gqa) * g.q_heads + kvh * g.gqa + slot % g.gqa; // output row
    const int tid = threadIdx.x;
    const int c = tid & 15;
    const int col = min((int)blockIdx.y * 16 + c, g.head_dim - 1);
    const int sl = tid >> 4;
    __shared__ float red_m[16];
    __shared__ float red_l[16];
    __shared__ float acc_x[16][17];
    const long base = ((long)kvh * a.splits_total) * n_slots + slot;
    const long ostride = (long)n_slots * g.head_dim;
    const float *po = a.part_o + base * g.head_dim + col;
    float ov[MERGE_PER_LANE], mv[MERGE_PER_LANE], lv[MERGE_PER_LANE];
#pragma unroll
    for (int i = 0; i < MERGE_PER_LANE; ++i) {
        const int s = sl + 16 * i;
        const bool ok = s < a.splits_total;
        const int sc = ok ? s : 0;
        mv[i] = a.part_m[base + (long)sc * n_slots];
        lv[i] = a.part_l[base + (long)sc * n_slots];
        ov[i] = po[(long)sc * ostride];
        if (!ok) {
            mv[i] = -INFINITY;
            lv[i] = 0.0f;
            ov[i] = 0.0f;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < MERGE_PER_LANE; ++i) mx = fmaxf(mx, mv[i]);
    if (c == 0) red_m[sl] = mx;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, red_m[i]);
    const float m_safe = mx == -INFINITY ? 0.0f : mx;
    float acc = 0.0f, lsum = 0.0f;
#pragma unroll
    for (int i = 0; i < MERGE_PER_LANE; ++i) {
        const float w = fast_exp2(mv[i] - m_safe);
        acc += w * ov[i];
        lsum += w * lv[i];
    }
    acc_x[sl][c] = acc;
    if (c == 0) red_l[sl] = lsum;
    __syncthreads();
    if (sl == 0 && (int)blockIdx.y * 16 + c < g.head_dim) {
        float t = 0.0f, l = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            t += acc_x[i][c];
            l += red_l[i];
        }
        float r = t / l;
        if (a.gate && a.n_queries == 1)
            r *= sigmoid_gate(a.gate[h * (a.q_head_stride > 0 ? a.q_head_stride : g.head_dim) + col]);
        a.out[h * g.head_dim + col] = r;
    }
}

template <int MERGE_PER_LANE>
__global__ __launch_bounds__(256) void decode_merge_kernel(DecodeArgs a) {
    decode_merge_body<MERGE_PER_LANE>(a);
}

// grid z is the sequence; a sequence with a single split already has its context
template <int MERGE_PER_LANE>
__global__ __launch_bounds__(256) void decode_merge_batch_kernel(DecodeBatchArgs b) {
    const DecodeArgs &a = b.seq[blockIdx.z];
    if (a.splits_total <= 1) return;
    decode_merge_body<MERGE_PER_LANE>(a);
}

// ------------------------------------------------------------------------------------
// The same merge with one wavefront per (query head, 16 columns) and nothing shared between
// wavefronts: the 64 lanes are 4 column lanes (four columns each, one 16-byte load per
// split) x 16 split lanes. Every lane asks for o, m and l of its splits at once; the
// maximum and the sums go across the split lanes with row rotations and row swaps in the
// vector unit, so that no lane waits at a barrier or for LDS. Row offsets are 32-bit: the
// launcher checks that one kv head's partials stay below 4 GiB and that head_dim is a
// multiple of four.
// ------------------------------------------------------------------------------------
struct MergeArgs {
    const float *part_o;
    const float *part_m;
    const float *part_l;
    float *out;
    const float *gate;
    int splits_total, n_queries, gqa, q_heads, head_dim, q_head_stride;
    int waves; // wavefronts (column groups) per workgroup
};

template <int CTRL>
__device__ __forceinline__ float row_rotated(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// the value that lane K of each group of four lanes holds
__device__ __forceinline__ float quad_lane(float v, int k) {
    const int x = __float_as_int(v);
    switch (k) { // k is a constant wherever this is used: one instruction
    case 0: return __int_as_float(__builtin_amdgcn_update_dpp(0, x, 0x00, 0xf, 0xf, false));
    case 1: return __int_as_float(__builtin_amdgcn_update_dpp(0, x, 0x55, 0xf, 0xf, false));
    case 2: return __int_as_float(__builtin_amdgcn_update_dpp(0, x, 0xaa, 0xf, 0xf, false));
    default: return __int_as_float(__builtin_amdgcn_update_dpp(0, x, 0xff, 0xf, 0xf, false));
    }
}
// over the 16 split lanes (lane bits 2..5) of one column lane, every lane receiving the result
__device__ __forceinline__ float split_lanes_max(float v) {
    v = fmaxf(v, row_rotated<0x124>(v)); // row_ror:4
    v = fmaxf(v, row_rotated<0x128>(v)); // row_ror:8
    return rows_max(v);
}
__device__ __forceinline__ float split_lanes_sum(float v) {
    v += row_rotated<0x124>(v);
    v += row_rotated<0x128>(v);
    return rows_sum(v);
}

template <int PER>
__device__ __forceinline__ void merge_wave_body(const MergeArgs &a, int kvh, int slot, int cg) {
    const int lane = threadIdx.x & 63;
    const int c4 = lane & 3, g = lane >> 2;
    const int n_slots = a.n_queries * a.gqa;
    const int col = cg * 16 + c4 * 4;
    const bool col_ok = col < a.head_dim;
    const long base = ((long)kvh * a.splits_total) * n_slots + slot;
    const char *pm = reinterpret_cast<const char *>(a.part_m + base);
    const char *pl = reinterpret_cast<const char *>(a.part_l + base);
    const char *po = reinterpret_cast<const char *>(a.part_o + base * a.head_dim);
    const uint32_t ml_stride = (uint32_t)n_slots * 4u;
    const uint32_t o_stride = ml_stride * (uint32_t)a.head_dim;
    const uint32_t g0 = g < a.splits_total ? (uint32_t)g : 0u;
    const uint32_t ml0 = g0 * ml_stride;
    const uint32_t o0 = g0 * o_stride + (col_ok ? (uint32_t)col * 4u : 0u);
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    f32x4_t ov[PER];
    // m and l of a split are the same for the four column lanes: each of them asks for a
    // quarter of the splits' pairs and hands them to the other three below
    constexpr int NML = (PER + 3) / 4;
    float mq[NML], lq[NML];
#pragma unroll
    for (int j = 0; j < NML; ++j) {
        const int i = c4 + 4 * j;
        const bool ok = i < PER && g + 16 * i < a.splits_total;
        const uint32_t mo = ok ? ml0 + (uint32_t)(16 * i) * ml_stride : ml0;
        mq[j] = *reinterpret_cast<const float *>(pm + mo);
        lq[j] = *reinterpret_cast<const float *>(pl + mo);
        if (!ok) {
            mq[j] = -INFINITY;
            lq[j] = 0.0f;
        }
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const bool ok = g + 16 * i < a.splits_total;
        const uint32_t oo = ok ? o0 + (uint32_t)(16 * i) * o_stride : o0;
        ov[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(po + oo)); // read once
    }
    float mv[PER], lv[PER];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        mv[i] = quad_lane(mq[i >> 2], i & 3);
        lv[i] = quad_lane(lq[i >> 2], i & 3);
        mx = fmaxf(mx, mv[i]);
    }
    mx = split_lanes_max(mx);
    const float m_safe = mx == -INFINITY ? 0.0f : mx;
    f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    float lsum = 0.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const float w = fast_exp2(mv[i] - m_safe); // 0 for the splits beyond the last
        acc += w * ov[i];
        lsum += w * lv[i];
    }
    acc.x = split_lanes_sum(acc.x);
    acc.y = split_lanes_sum(acc.y);
    acc.z = split_lanes_sum(acc.z);
    acc.w = split_lanes_sum(acc.w);
    lsum = split_lanes_sum(lsum);
    if (g == 0 && col_ok) {
        const int qi = a.n_queries == 1 ? 0 : slot / a.gqa;
        const long h = (long)qi * a.q_heads + kvh * a.gqa + (slot - qi * a.gqa); // output row
        f32x4_t r = {acc.x / lsum, acc.y / lsum, acc.z / lsum, acc.w / lsum};
        if (a.gate && a.n_queries == 1) {
            const float *gp = a.gate + h * (a.q_head_stride > 0 ? a.q_head_stride : a.head_dim) + col;
            r.x *= sigmoid_gate(gp[0]);
            r.y *= sigmoid_gate(gp[1]);
            r.z *= sigmoid_gate(gp[2]);
            r.w *= sigmoid_gate(gp[3]);
        }
        *reinterpret_cast<f32x4_t *>(a.out + h * a.head_dim + col) = r;
    }
}

// grid (column groups / wavefronts per workgroup, query slots, kv heads)
template <int PER>
__global__ __launch_bounds__(256) void decode_merge_wave_kernel(MergeArgs a) {
    // a wavefront beyond the last column group goes through the motions on column 0 and
    // stores nothing: no early exit, so that every kernel argument is asked for at once
    const int cg = (int)blockIdx.x * a.waves + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    merge_wave_body<PER>(a, blockIdx.z, blockIdx.y, cg);
}

// Several sequences of one geometry, one query row each: grid (pairs of column groups, query
// heads, sequences); a sequence with a single split already has its context.
template <int PER>
__global__ __launch_bounds__(128) void decode_merge_wave_batch_kernel(DecodeBatchArgs b) {
    const DecodeArgs &d = b.seq[blockIdx.z];
    if (d.splits_total <= 1) return;
    MergeArgs a;
    a.part_o = d.part_o;
    a.part_m = d.part_m;
    a.part_l = d.part_l;
    a.out = d.out;
    a.gate = d.gate;
    a.splits_total = d.splits_total;
    a.n_queries = 1;
    a.gqa = d.g.gqa;
    a.q_heads = d.g.q_heads;
    a.head_dim = d.g.head_dim;
    a.q_head_stride = d.q_head_stride;
    a.waves = 2;
    const int kvh = (int)blockIdx.y / d.g.gqa;
    const int cg = (int)blockIdx.x * 2 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    merge_wave_body<PER>(a, kvh, (int)blockIdx.y - kvh * d.g.gqa, cg);
}

template <int P, int WAVES, bool MQ, bool PRE>
static hipError_t launch_split_mq(const DecodeArgs &a, hipStream_t s) {
    constexpr int KK = P / 32;
    size_t stage = (size_t)2 * KK * 64 * sizeof(uint4) + 2 * P * sizeof(uint16_t);
    if (PRE) stage += ((size_t)2 * 17 * (P + 1) + 3 * P + 22 + 17 * (P + 4)) * sizeof(float);
    const int n_slots = a.n_queries * a.g.gqa;
    const int rows = n_slots < 16 ? n_slots : 16;
    const size_t xchg = ((size_t)WAVES * rows * (P + 4) + 2 * WAVES * rows) * sizeof(float);
    const size_t stage16 = (stage + 15) & ~(size_t)15;
    const bool apart = stage16 + xchg <= LDS_BYTES;
    const size_t lds = apart ? stage16 + xchg : (stage > xchg ? stage : xchg);
    static std::atomic<uint64_t> lds_ok{0}; // per instantiation
    {
        hipError_t e = allow_full_lds(reinterpret_cast<const void *>(&decode_split_kernel<P, WAVES, MQ, PRE>), lds_ok);
        if (e != hipSuccess) return e;
    }
    DecodeArgs b = a;
    b.xchg_off = apart ? (int)stage16 : 0;
    dim3 grid((unsigned)a.splits, (unsigned)a.g.kv_heads, (unsigned)((n_slots + 15) / 16));
    hipLaunchKernelGGL((decode_split_kernel<P, WAVES, MQ, PRE>), grid, dim3(WAVES * 64), lds, s, b);
    return hipGetLastError();
}

template <int P, int WAVES>
static hipError_t launch_split(const DecodeArgs &a, hipStream_t s) {
    // the decode specialisation assumes a single tile of query slots
    if (a.n_queries > 1 || a.g.gqa > 16) {
        if (a.pre) return hipErrorInvalidValue; // the caller keeps the fused step to single-tile decode
        return launch_split_mq<P, WAVES, true, false>(a, s);
    }
    return a.pre ? launch_split_mq<P, WAVES, false, true>(a, s) : launch_split_mq<P, WAVES, false, false>(a, s);
}

// head_dim 257..512 (global layers of Gemma-4-style models, src/config/accessors.rs:118-123):
// the accumulators and one K and one V page alone are 256 registers, so the workgroup has
// four wavefronts, one per SIMD with 512 registers each (two row elements per thread in the
// fused pre-KV step and the fused append).
static hipError_t launch_split_wide(const DecodeArgs &a, hipStream_t s) {
    if (a.n_queries > 1 || a.g.gqa > 16) {
        if (a.pre) return hipErrorInvalidValue;
        return launch_split_mq<512, 4, true, false>(a, s);
    }
    return a.pre ? launch_split_mq<512, 4, false, true>(a, s) : launch_split_mq<512, 4, false, false>(a, s);
}

hipError_t launch_decode(const DecodeArgs &a, hipStream_t s) {
    hipError_t e = hipErrorInvalidValue;
    const bool w8 = a.waves == 8;
    switch (a.g.P) {
    case 512: e = launch_split_wide(a, s); break;
    case 32: e = w8 ? launch_split<32, 8>(a, s) : launch_split<32, 4>(a, s); break;
    case 64: e = w8 ? launch_split<64, 8>(a, s) : launch_split<64, 4>(a, s); break;
    case 128: e = w8 ? launch_split<128, 8>(a, s) : launch_split<128, 4>(a, s); break;
    case 256: e = w8 ? launch_split<256, 8>(a, s) : launch_split<256, 4>(a, s); break;
    default: break;
    }
    if (e != hipSuccess || a.splits_total == 1) return e;
    return launch_merge(a, s);
}

// Whether the wavefront merge serves these partials: 16-byte column loads, 32-bit offsets
// within a kv head, and a grid that fits.
static bool merge_wave_fits(const DecodeArgs &a) {
    const uint64_t n_slots = (uint64_t)a.n_queries * a.g.gqa;
    return a.g.head_dim % 4 == 0 && (uint64_t)a.splits_total * n_slots * a.g.head_dim * 4 < (1ull << 32) &&
           n_slots <= 65535 && a.g.kv_heads <= 65535 && a.splits_total <= 16 * MERGE_PER_LANE_MAX &&
           ((uintptr_t)a.part_o & 15) == 0 && ((uintptr_t)a.out & 15) == 0;
}

static hipError_t launch_merge_wave(const DecodeArgs &a, hipStream_t s) {
    MergeArgs m;
    m.part_o = a.part_o;
    m.part_m = a.part_m;
    m.part_l = a.part_l;
    m.out = a.out;
    m.gate = a.gate;
    m.splits_total = a.splits_total;
    m.n_queries = a.n_queries;
    m.gqa = a.g.gqa;
    m.q_heads = a.g.q_heads;
    m.head_dim = a.g.head_dim;
    m.q_head_stride = a.q_head_stride;
    const int n_slots = a.n_queries * a.g.gqa;
    const int n_cg = (a.g.head_dim + 15) / 16;
    // Two wavefronts per workgroup, i.e. two neighbouring column groups on one compute unit,
    // so that the 128-byte lines of the partials are fetched once and not once per half
    // (FETCH_SIZE of the merge: 2235 KiB against 4277 KiB with one wavefront per workgroup, same
    // time); four where the grid is large anyway (four on the decode step: 0.3 us slower).
    const int waves = (long)n_cg * n_slots * a.g.kv_heads <= 1024 ? 2 : 4;
    m.waves = waves;
    dim3 grid((unsigned)((n_cg + waves - 1) / waves), (unsigned)n_slots, (unsigned)a.g.kv_heads);
    const dim3 block((unsigned)(64 * waves));
    const int per = (a.splits_total + 15) / 16;
    if (per <= 1) hipLaunchKernelGGL(decode_merge_wave_kernel<1>, grid, block, 0, s, m);
    else if (per <= 2) hipLaunchKernelGGL(decode_merge_wave_kernel<2>, grid, block, 0, s, m);
    else if (per <= 4) hipLaunchKernelGGL(decode_merge_wave_kernel<4>, grid, block, 0, s, m);
    else if (per <= 8) hipLaunchKernelGGL(decode_merge_wave_kernel<8>, grid, block, 0, s, m);
    else hipLaunchKernelGGL(decode_merge_wave_kernel<16>, grid, block, 0, s, m);
    return hipGetLastError();
}

hipError_t launch_merge(const DecodeArgs &a, hipStream_t s) {
    if (merge_wave_fits(a)) return launch_merge_wave(a, s);
    dim3 mgrid((unsigned)(a.g.kv_heads * a.n_queries * a.g.gqa), (unsigned)((a.g.head_dim + 15) / 16));
    const int per_lane = (a.splits_total + 15) / 16;
    if (per_lane <= 1) hipLaunchKernelGGL(decode_merge_kernel<1>, mgrid, dim3(256), 0, s, a);
    else if (per_lane <= 2) hipLaunchKernelGGL(decode_merge_kernel<2>, mgrid, dim3(256), 0, s, a);
    else if (per_lane <= 4) hipLaunchKernelGGL(decode_merge_kernel<4>, mgrid, dim3(256), 0, s, a);
    else if (per_lane <= 8) hipLaunchKernelGGL(decode_merge_kernel<8>, mgrid, dim3(256), 0, s, a);
    else if (per_lane <= 16) hipLaunchKernelGGL(decode_merge_kernel<16>, mgrid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL(decode_merge_kernel<MERGE_PER_LANE_MAX>, mgrid, dim3(256), 0, s, a);
    return hipGetLastError();
}

template <int P, int WAVES>
static hipError_t launch_split_batch(const DecodeBatchArgs &b, int n_seq, int max_splits, hipStream_t s) {
    constexpr int KK = P / 32;
    const Geom &g = b.seq[0].g;
    const size_t stage = (size_t)2 * KK * 64 * sizeof(uint4) + 2 * P * sizeof(uint16_t);
    const int rows = g.gqa < 16 ? g.gqa : 16;
    const size_t xchg = ((size_t)WAVES * rows * (P + 4) + 2 * WAVES * rows) * sizeof(float);
    const size_t stage16 = (stage + 15) & ~(size_t)15;
    const bool apart = stage16 + xchg <= LDS_BYTES;
    const size_t lds = apart ? stage16 + xchg : (stage > xchg ? stage : xchg);
    static std::atomic<uint64_t> lds_ok{0}; // per instantiation
    {
        hipError_t e = allow_full_lds(reinterpret_cast<const void *>(&decode_split_batch_kernel<P, WAVES>), lds_ok);
        if (e != hipSuccess) return e;
    }
    DecodeBatchArgs bb = b;
    for (int i = 0; i < n_seq; ++i) bb.seq[i].xchg_off = apart ? (int)stage16 : 0;
    dim3 grid((unsigned)max_splits, (unsigned)g.kv_heads, (unsigned)n_seq);
    hipLaunchKernelGGL((decode_split_batch_kernel<P, WAVES>), grid, dim3(WAVES * 64), lds, s, bb);
    return hipGetLastError();
}

// All sequences share one geometry and one wavefront count, and each has n_queries == 1
// and gqa <= 16 (checked by the caller).
hipError_t launch_decode_batch(const DecodeBatchArgs &b, int n_seq, hipStream_t s) {
    if (n_seq < 1 || n_seq > SKV_MAX_BATCH) return hipErrorInvalidValue;
    const DecodeArgs &a0 = b.seq[0];
    int max_splits = 1;
    for (int i = 0; i < n_seq; ++i) max_splits = b.seq[i].splits > max_splits ? b.seq[i].splits : max_splits; // == splits_total here
    hipError_t e = hipErrorInvalidValue;
    const bool w8 = a0.waves == 8;
    if (a0.g.f32) e = launch_f32_split_batch(b, n_seq, max_splits, s);
    else switch (a0.g.P) {
    case 512: e = launch_split_batch<512, 4>(b, n_seq, max_splits, s); break;
    case 32: e = w8 ? launch_split_batch<32, 8>(b, n_seq, max_splits, s) : launch_split_batch<32, 4>(b, n_seq, max_splits, s); break;
    case 64: e = w8 ? launch_split_batch<64, 8>(b, n_seq, max_splits, s) : launch_split_batch<64, 4>(b, n_seq, max_splits, s); break;
    case 128: e = w8 ? launch_split_batch<128, 8>(b, n_seq, max_splits, s) : launch_split_batch<128, 4>(b, n_seq, max_splits, s); break;
    case 256: e = w8 ? launch_split_batch<256, 8>(b, n_seq, max_splits, s) : launch_split_batch<256, 4>(b, n_seq, max_splits, s); break;
    default: break;
    }
    if (e != hipSuccess || max_splits == 1) return e;
    const int per_lane = (max_splits + 15) / 16;
    bool wave_merge = a0.g.kv_heads * a0.g.gqa <= 65535;
    for (int i = 0; i < n_seq; ++i) wave_merge = wave_merge && b.seq[i].n_queries == 1 && merge_wave_fits(b.seq[i]);
    if (wave_merge) {
        dim3 grid((unsigned)(((a0.g.head_dim + 15) / 16 + 1) / 2), (unsigned)(a0.g.kv_heads * a0.g.gqa), (unsigned)n_seq);
        if (per_lane <= 1) hipLaunchKernelGGL(decode_merge_wave_batch_kernel<1>, grid, dim3(128), 0, s, b);
        else if (per_lane <= 2) hipLaunchKernelGGL(decode_merge_wave_batch_kernel<2>, grid, dim3(128), 0, s, b);
        else if (per_lane <= 4) hipLaunchKernelGGL(decode_merge_wave_batch_kernel<4>, grid, dim3(128), 0, s, b);
        else if (per_lane <= 8) hipLaunchKernelGGL(decode_merge_wave_batch_kernel<8>, grid, dim3(128), 0, s, b);
        else hipLaunchKernelGGL(decode_merge_wave_batch_kernel<16>, grid, dim3(128), 0, s, b);
        return hipGetLastError();
    }
    dim3 mgrid((unsigned)(a0.g.kv_heads * a0.g.gqa), (unsigned)((a0.g.head_dim + 15) / 16), (unsigned)n_seq);
    if (per_lane <= 1) hipLaunchKernelGGL(decode_merge_batch_kernel<1>, mgrid, dim3(256), 0, s, b);
    else if (per_lane <= 2) hipLaunchKernelGGL(decode_merge_batch_kernel<2>, mgrid, dim3(256), 0, s, b);
    else if (per_lane <= 4) hipLaunchKernelGGL(decode_merge_batch_kernel<4>, mgrid, dim3(256), 0, s, b);
    else if (per_lane <= 8) hipLaunchKernelGGL(decode_merge_batch_kernel<8>, mgrid, dim3(256), 0, s, b);
    else if (per_lane <= 16) hipLaunchKernelGGL(decode_merge_batch_kernel<16>, mgrid, dim3(256), 0, s, b);
    else hipLaunchKernelGGL(decode_merge_batch_kernel<MERGE_PER_LANE_MAX>, mgrid, dim3(256), 0, s, b);
    return hipGetLastError();
}

} // namespace skv
