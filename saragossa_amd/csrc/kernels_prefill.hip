// gfx950 kernels of the KV hot path, part 3: chunked prefill over the paged cache, the one
// matrix-core-bound kernel of the path.
#include "skv_internal.h"

namespace skv {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;

namespace {

__device__ __forceinline__ uint16_t bf16_bits(float v) {
    uint32_t b = __float_as_uint(v);
    uint32_t lsb = (b >> 16) & 1u;
    return (uint16_t)((b + 0x7fffu + lsb) >> 16);
}
__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

} // namespace

// ------------------------------------------------------------------------------------
// Many query rows over the cache (cached_attention_prefill_rows,
// src/decoder/attention_ops.rs:976-1017, as one launch): query slot (i, g) = new row i,
// head g of the kv head's group, attends positions up to len - n_queries + i through the
// layer's window.
//
// One workgroup = 8 wavefronts = 8 * TILES tiles of 16 query slots of one kv head, and a
// range of the context's pages (split). The workgroup walks its pages once: all threads
// copy PG pages' K and V tiles (already in matrix-operand order) from memory to LDS, double
// buffered, and every wavefront multiplies them with its own query tiles, which it holds in
// registers as bf16 hi + lo halves (pre-scaled by log2(e)/sqrt(head_dim)). So a K/V byte is
// fetched from memory once per 128 * TILES query slots instead of once per 16. Pages are
// consumed in pairs: S^T = K . Q^T per page (16 keys x 16 slots, 16x16x32 over the head
// dims), one online-softmax step in base 2 over the pair's 32 keys on the accumulator
// registers, then O^T += V^T . P^T as 16x16x32 products over those 32 keys with P split
// hi + lo. There is no merge inside the workgroup (every wavefront owns its slots); with
// several splits the (o, m, l) partials go to merge_rows_kernel.
// ------------------------------------------------------------------------------------
// Copies of PG pages (K tile then V tile each) of one kv head: memory -> registers -> LDS.
template <int P, int PG, int THREADS>
__device__ __forceinline__ void fetch_step(uint4 (&stage)[PG][(2 * (P / 32) * 64 + THREADS - 1) / THREADS], const DecodeArgs &a,
                                           int pb0, int step, int n_it, int kvh, int tid) {
    constexpr int TILE_U4 = (P / 32) * 64;
    constexpr int LOAD_U = (2 * TILE_U4 + THREADS - 1) / THREADS;
#pragma unroll
    for (int pg = 0; pg < PG; ++pg) {
        // past the end: a page again, unused; always a page the layer holds
        const int it = max(min(step * PG + pg, n_it - 1), 0);
        const int page = a.table[min(pb0 + it, a.page_first + a.n_pages - 1)]; // uniform: a scalar load
        const long tile = (long)page * a.g.page_elems + (long)kvh * a.g.tile_elems;
        const uint4 *kp = reinterpret_cast<const uint4 *>(a.k_pool + tile);
        const uint4 *vp = reinterpret_cast<const uint4 *>(a.v_pool + tile);
#pragma unroll
        for (int u = 0; u < LOAD_U; ++u) {
            // unconditional (a thread past the end re-reads the last unit and drops it)
            const int i = min(tid + u * THREADS, 2 * TILE_U4 - 1);
            const uint4 *src = i < TILE_U4 ? kp + i : vp + (i - TILE_U4);
            stage[pg][u] = *src;
        }
    }
}
// LDS order of a step: [PG/2 pairs][K tile of page A | K tile of page B | V tiles of both].
// The K tiles are copied verbatim. The two V tiles of a pair are interleaved in 8-byte
// halves, unit (kk, h, lane) = {page A's four keys, page B's four keys} of dim tile h, so
// that one 16-byte read is the 32-key operand of the PV product as it stands.
//
// Keys that no query slot of the workgroup attends (rows at or past the cache's length after a
// rollback, ring rows not valid, rows before every slot's window, the stand-in page past the
// end of a split) get zero probability, but 0 x NaN is NaN: on the pages at the edges of the
// attended range [ws_lo, lim_hi] (and on ring pages) their V values are cleared on the way
// into LDS, so the bits of such a row never reach a context (the reference never reads those
// rows, src/decode_resident/kernels.rs:11-88).
template <int P, int PG, int THREADS>
__device__ __forceinline__ void store_step(const uint4 (&stage)[PG][(2 * (P / 32) * 64 + THREADS - 1) / THREADS], uint4 *buf,
                                           int tid, const DecodeArgs &a, int pb0, int step, int n_it, int ws_lo,
                                           int lim_hi) {
    constexpr int TILE_U4 = (P / 32) * 64;
    constexpr int LOAD_U = (2 * TILE_U4 + THREADS - 1) / THREADS;
    static_assert(PG % 2 == 0, "pages are consumed in pairs");
#pragma unroll
    for (int pg = 0; pg < PG; ++pg) {
        uint4 *pair = buf + (pg >> 1) * 4 * TILE_U4;
        const int it = step * PG + pg;
        const int slot_a = (pb0 + it) * 16; // first cache slot of the page
        const bool inside = it < n_it && a.g.ring_rows == 0 && slot_a >= ws_lo && slot_a + 15 <= lim_hi;
#pragma unroll
        for (int u = 0; u < LOAD_U; ++u) {
            const int i = tid + u * THREADS;
            if (2 * TILE_U4 < THREADS && i >= 2 * TILE_U4) continue;
            uint4 x = stage[pg][u];
            if (i < TILE_U4) {
                pair[(pg & 1) * TILE_U4 + i] = x;
            } else {
                const int iv = i - TILE_U4;
                if (!inside) {
                    // the unit holds keys 4rq .. 4rq+3 of two dim tiles: (x, y) and (z, w), two keys a word
                    const int rq = (iv >> 4) & 3;
                    uint32_t keep[2] = {0u, 0u};
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int slot = slot_a + rq * 4 + r;
                        int pos = slot;
                        if (a.g.ring_rows > 0)
                            pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - a.g.ring_rows + slot;
                        if (it < n_it && pos >= ws_lo && pos <= lim_hi) keep[r >> 1] |= 0xffffu << ((r & 1) * 16);
                    }
                    x.x &= keep[0];
                    x.z &= keep[0];
                    x.y &= keep[1];
                    x.w &= keep[1];
                }
                uint2 *dst = reinterpret_cast<uint2 *>(pair + 2 * TILE_U4 + (iv >> 6) * 128 + (iv & 63)) + (pg & 1);
                dst[0] = make_uint2(x.x, x.y);
                dst[128] = make_uint2(x.z, x.w); // dim tile 1: 64 units of 16 bytes further
            }
        }
    }
}

// PG: pages copied and consumed per barrier step (the copies of step i+1 are in flight while
// step i is multiplied, so a step must hold about a memory latency's worth of work).
template <int P, int TILES, int PG, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void prefill_tile_kernel(DecodeArgs a) {
    constexpr int THREADS = WAVES * 64;
    constexpr int KK = P / 32;
    constexpr int NT = P / 16;
    constexpr int TILE_U4 = KK * 64;                       // 16-byte units of one K (or V) tile
    constexpr int LOAD_U = (2 * TILE_U4 + THREADS - 1) / THREADS;
    extern __shared__ __attribute__((aligned(16))) uint4 kv_lds[]; // [2 buffers][PG][K tile | V tile]
    constexpr int BUF_U4 = PG * 2 * TILE_U4;

    const Geom g = a.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int j = lane >> 4;
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    const int G = g.gqa;
    const int C = a.n_queries;
    const int n_slots = C * G;
    const int wg_slot0 = blockIdx.z * (WAVES * TILES * 16);
    const int wg_slot1 = min(n_slots, wg_slot0 + WAVES * TILES * 16) - 1; // last slot of the workgroup

    // query slot -> position of its row, last position it attends, first position it attends
    auto pos_of = [&](int slot) { return a.q_pos0 + slot / G; };
    auto limit_of = [&](int slot) { return min(pos_of(slot), a.limit_cap); };
    auto ws_of = [&](int slot) { return a.window > 0 ? max(a.window_start, pos_of(slot) + 1 - a.window) : a.window_start; };

    // pages any slot of the workgroup can see, divided among the splits
    const int wg_ws_lo = ws_of(wg_slot0);
    const int wg_lim_hi = limit_of(wg_slot1);
    const int page_lo = g.ring_rows > 0 ? 0 : wg_ws_lo >> 4;
    const int page_hi = g.ring_rows > 0 ? a.n_pages : (wg_lim_hi >> 4) + 1;
    const unsigned span = (unsigned)(page_hi - page_lo);
    const int pb0 = page_lo + (int)(((unsigned)split * span) / (unsigned)a.splits);
    const int pb1 = page_lo + (int)(((unsigned)(split + 1) * span) / (unsigned)a.splits);
    const int n_it = pb1 - pb0;

    // ---- this wavefront's query tiles ------------------------------------------------
    int my_limit[TILES], my_ws[TILES];
    int t_ws_hi[TILES], t_lim_lo[TILES], t_ws_lo[TILES], t_lim_hi[TILES]; // per tile extremes
    bool t_on[TILES];
    bf16x8_t qh[TILES][KK], ql[TILES][KK];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const int s0 = wg_slot0 + (wave * TILES + t) * 16;
        t_on[t] = s0 < n_slots;
        const int s_last = min(s0 + 15, n_slots - 1);
        const int my_slot = min(s0 + n, n_slots - 1);
        my_limit[t] = limit_of(my_slot);
        my_ws[t] = ws_of(my_slot);
        t_lim_lo[t] = limit_of(min(s0, n_slots - 1));
        t_lim_hi[t] = limit_of(s_last);
        t_ws_lo[t] = ws_of(min(s0, n_slots - 1));
        t_ws_hi[t] = ws_of(s_last);
        const float *qrow = a.q + ((long)(my_slot / G) * g.q_heads + kvh * G + my_slot % G) * g.head_dim;
        // eight consecutive dims of the slot's row per k-step: all loads first (two 16-byte
        // loads per step when the row allows), unconditional from clamped addresses, so that
        // they are one round trip; dims past head_dim are zeroed afterwards
        float qv[KK][8];
        if (a.q_vec) {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const int d0 = kk * 32 + j * 8;
                const float4_t *qp = reinterpret_cast<const float4_t *>(qrow + min(d0, g.head_dim - 8));
                const float4_t x0 = qp[0], x1 = qp[1];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    qv[kk][e] = x0[e];
                    qv[kk][4 + e] = x1[e];
                }
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
                for (int e = 0; e < 8; ++e) qv[kk][e] = qrow[min(kk * 32 + j * 8 + e, g.head_dim - 1)];
            }
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const int d0 = kk * 32 + j * 8;
            uint32_t hi[4], lo[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                uint32_t h2 = 0, l2 = 0;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float v = d0 + e2 * 2 + h < g.head_dim ? qv[kk][e2 * 2 + h] * a.qscale : 0.0f;
                    const uint16_t hb = bf16_bits(v);
                    const uint16_t lb = bf16_bits(v - bf16_to_f32(hb));
                    h2 |= (uint32_t)hb << (16 * h);
                    l2 |= (uint32_t)lb << (16 * h);
                }
                hi[e2] = h2;
                lo[e2] = l2;
            }
            qh[t][kk] = __builtin_bit_cast(bf16x8_t, make_uint4(hi[0], hi[1], hi[2], hi[3]));
            ql[t][kk] = __builtin_bit_cast(bf16x8_t, make_uint4(lo[0], lo[1], lo[2], lo[3]));
        }
    }

    float4_t o[TILES][NT];
    float m_run[TILES], l_run[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
#pragma unroll
        for (int c = 0; c < NT; ++c) o[t][c] = float4_t{0.f, 0.f, 0.f, 0.f};
        m_run[t] = -INFINITY;
        l_run[t] = 0.0f;
    }

    // ---- page copies: memory -> registers -> LDS -------------------------------------
    const int n_steps = (n_it + PG - 1) / PG;
    constexpr int FETCH_PAIR = PG / 2 - 1; // in front of the step's last pair
    uint4 stage[PG][LOAD_U];
    // (a split without pages still reads one valid page, and writes empty partials below)
    fetch_step<P, PG, THREADS>(stage, a, pb0, 0, n_it, kvh, tid);
    store_step<P, PG, THREADS>(stage, kv_lds, tid, a, pb0, 0, n_it, wg_ws_lo, wg_lim_hi);
    __syncthreads();

    for (int step = 0; step < n_steps; ++step) {
      // The next step's pages are asked for in front of the last pair of this step, not at its
      // top: the copies still land before store_step needs them, and the staging registers are
      // live for less of the step (a stream of calls, same box each: config 2 shape 450 against
      // 466 us and 470.6 against 480.3; config 1 shape, four pairs per step, 56.8 in front of the
      // last pair, 57.4 and 57.9 in front of the third and second, 57.75 at the top; inside the
      // last pair, after its scores or its softmax, 481-483 against 475 at config 2 shape).
      // Unconditional: after the last step this re-reads its pages into the idle buffer.
      // Pages are consumed in pairs (A, B): the PV product then contracts over 32 keys with
      // the k index of lane group j, element e meaning key 4j+e of page A (e < 4) or key
      // 4j+e-4 of page B, which is exactly how the two S^T tiles and the two V tiles already
      // sit in the lanes.
#pragma unroll
      for (int pp = 0; pp < PG / 2; ++pp) {
        if (pp == FETCH_PAIR) fetch_step<P, PG, THREADS>(stage, a, pb0, min(step + 1, n_steps - 1), n_it, kvh, tid);
        const int it_a = step * PG + 2 * pp;
        if (it_a >= n_it) continue;
        const bool has_b = it_a + 1 < n_it;
        const uint4 *kt_a = kv_lds + (step & 1) * BUF_U4 + pp * 4 * TILE_U4;
        const uint4 *kt_b = kt_a + TILE_U4;
        const uint4 *vt = kt_a + 2 * TILE_U4; // both pages' V tiles, interleaved (store_step)
        const int slot_a = (pb0 + it_a) * 16; // first cache slot of page A; page B follows it

        // which of the wavefront's tiles see the pair at all
        bool use[TILES];
        bool any = false;
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            use[t] = t_on[t] && (g.ring_rows > 0 || (slot_a <= t_lim_hi[t] && slot_a + 31 >= t_ws_lo[t]));
            any = any || use[t];
        }
        if (!any) continue;
        // S^T = K . Q^T for both pages, the K registers shared by the tiles
        float4_t sa0[TILES], sa1[TILES], sb0[TILES], sb1[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            sa0[t] = float4_t{0.f, 0.f, 0.f, 0.f};
            sa1[t] = float4_t{0.f, 0.f, 0.f, 0.f};
            sb0[t] = float4_t{0.f, 0.f, 0.f, 0.f};
            sb1[t] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
        // The operands of a K-step are asked for DEPTH K-steps before its products are issued,
        // and the order is pinned: left to itself the compiler keeps one read ahead, issues the
        // product that needs the newest operand first, and every other product then waits for
        // LDS (the two wavefronts of a SIMD cannot cover a latency each of them hits at once).
        constexpr int DEPTH = (KK < 2 || P > 256) ? 1 : 2;
        uint4 ra[KK], rb[KK];
#pragma unroll
        for (int kk = 0; kk < DEPTH; ++kk) {
            ra[kk] = kt_a[kk * 64 + lane];
            rb[kk] = kt_b[kk * 64 + lane];
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            if (kk + DEPTH < KK) {
                ra[kk + DEPTH] = kt_a[(kk + DEPTH) * 64 + lane];
                rb[kk + DEPTH] = kt_b[(kk + DEPTH) * 64 + lane];
            }
            __builtin_amdgcn_sched_barrier(0);
            const bf16x8_t ka = __builtin_bit_cast(bf16x8_t, ra[kk]);
            const bf16x8_t kb = __builtin_bit_cast(bf16x8_t, rb[kk]);
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                sa0[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qh[t][kk], sa0[t], 0, 0, 0);
                sb0[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, qh[t][kk], sb0[t], 0, 0, 0);
                sa1[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, ql[t][kk], sa1[t], 0, 0, 0);
                sb1[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, ql[t][kk], sb1[t], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // the first V operands of the pair travel while the softmax runs
        uint4 rv0[KK], rv1[KK];
#pragma unroll
        for (int kk = 0; kk < DEPTH; ++kk) {
            rv0[kk] = vt[kk * 128 + lane];
            rv1[kk] = vt[kk * 128 + 64 + lane];
        }
        __builtin_amdgcn_sched_barrier(0);
        bf16x8_t ph[TILES], pl[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            float sv[8];
            {
                const float4_t xa = sa0[t] + sa1[t], xb = sb0[t] + sb1[t];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sv[i] = xa[i];
                    sv[4 + i] = xb[i];
                }
            }
            const bool interior = has_b && g.ring_rows == 0 && slot_a >= t_ws_hi[t] && slot_a + 31 <= t_lim_lo[t];
            if (!interior || !use[t]) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int slot = slot_a + (e >> 2) * 16 + j * 4 + (e & 3);
                    int pos = slot;
                    if (g.ring_rows > 0)
                        pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
                    const bool ok = use[t] && (e < 4 || has_b) && pos >= my_ws[t] && pos <= my_limit[t];
                    sv[e] = ok ? sv[e] : -INFINITY;
                }
            }
            float m_blk = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])),
                                fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
            m_blk = rows_max(m_blk);
            const float m_new = fmaxf(m_run[t], m_blk);
            const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = fast_exp2(m_run[t] - m_safe);
            // p = hi + lo with hi the upper 16 bits of p (truncated) and lo the upper 16 bits of
            // the exact remainder: 2^-16 relative, two byte permutes per pair of values
            float psum = 0.0f;
            uint32_t pb_[8], rb_[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pv = fast_exp2(sv[e] - m_safe);
                psum += pv;
                pb_[e] = __float_as_uint(pv);
                rb_[e] = __float_as_uint(pv - __uint_as_float(pb_[e] & 0xffff0000u));
            }
            ph[t] = __builtin_bit_cast(bf16x8_t, make_uint4(__builtin_amdgcn_perm(pb_[1], pb_[0], 0x07060302u),
                                                            __builtin_amdgcn_perm(pb_[3], pb_[2], 0x07060302u),
                                                            __builtin_amdgcn_perm(pb_[5], pb_[4], 0x07060302u),
                                                            __builtin_amdgcn_perm(pb_[7], pb_[6], 0x07060302u)));
            pl[t] = __builtin_bit_cast(bf16x8_t, make_uint4(__builtin_amdgcn_perm(rb_[1], rb_[0], 0x07060302u),
                                                            __builtin_amdgcn_perm(rb_[3], rb_[2], 0x07060302u),
                                                            __builtin_amdgcn_perm(rb_[5], rb_[4], 0x07060302u),
                                                            __builtin_amdgcn_perm(rb_[7], rb_[6], 0x07060302u)));
            l_run[t] = l_run[t] * alpha + psum;
            m_run[t] = m_new;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
                for (int c = 0; c < NT; ++c) o[t][c] *= alpha;
            }
        }
        // O^T += V^T . P^T over the 32 keys of the pair, the V registers shared by the tiles.
        // Without a page B its probabilities are zero and its place holds a page the layer
        // owns (fetch_step clamps), so the products vanish.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            if (kk + DEPTH < KK) {
                rv0[kk + DEPTH] = vt[(kk + DEPTH) * 128 + lane];
                rv1[kk + DEPTH] = vt[(kk + DEPTH) * 128 + 64 + lane];
            }
            __builtin_amdgcn_sched_barrier(0);
            const bf16x8_t v0 = __builtin_bit_cast(bf16x8_t, rv0[kk]);
            const bf16x8_t v1 = __builtin_bit_cast(bf16x8_t, rv1[kk]);
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                o[t][2 * kk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v0, ph[t], o[t][2 * kk], 0, 0, 0);
                o[t][2 * kk + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v1, ph[t], o[t][2 * kk + 1], 0, 0, 0);
                o[t][2 * kk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v0, pl[t], o[t][2 * kk], 0, 0, 0);
                o[t][2 * kk + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v1, pl[t], o[t][2 * kk + 1], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
      }
      store_step<P, PG, THREADS>(stage, kv_lds + ((step + 1) & 1) * BUF_U4, tid, a, pb0, min(step + 1, n_steps - 1),
                                 n_it, wg_ws_lo, wg_lim_hi);
      __syncthreads();
    }

    // ---- every wavefront writes its own slots -------------------------------------------
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        float l = l_run[t];
        l = rows_sum(l);
        const int slot = wg_slot0 + (wave * TILES + t) * 16 + n;
        if (!t_on[t] || slot >= n_slots) continue;
        float *dst;
        float scale = 1.0f;
        if (a.splits_total == 1) {
            scale = 1.0f / l;
            dst = a.out + ((long)(slot / G) * g.q_heads + kvh * G + slot % G) * g.head_dim;
        } else {
            const long pidx = ((long)kvh * a.splits_total + a.split_base + split) * n_slots + slot;
            dst = a.part_o + pidx * g.head_dim;
            if (j == 0) {
                a.part_m[pidx] = m_run[t];
                a.part_l[pidx] = l;
            }
        }
        const bool vec_ok = (g.head_dim & 3) == 0;
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            const int col = c * 16 + j * 4;
            const float4_t v = o[t][c] * scale;
            if (vec_ok) {
                if (col < g.head_dim) *reinterpret_cast<float4_t *>(dst + col) = v;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (col + i < g.head_dim) dst[col + i] = v[i];
            }
        }
    }
}

// Merge of the split partials of many query slots: one thread per (kv head, slot, four
// columns) walks the few splits. (The decode merge spends a workgroup per 16 columns of a
// head, which is right for a handful of heads and many splits, not for thousands of slots.)
__global__ __launch_bounds__(256) void merge_rows_kernel(DecodeArgs a) {
    const Geom g = a.g;
    const int n_slots = a.n_queries * g.gqa;
    const int c4n = (g.head_dim + 3) >> 2;
    const long total = (long)g.kv_heads * n_slots * c4n;
    const long id = (long)blockIdx.x * 256 + threadIdx.x;
    if (id >= total) return;
    const int c4 = (int)(id % c4n) * 4;
    const long ks = id / c4n;             // kvh * n_slots + slot
    const int kvh = (int)(ks / n_slots);
    const int slot = (int)(ks - (long)kvh * n_slots);
    const long base = ((long)kvh * a.splits_total) * n_slots + slot;
    // Up to four splits (the usual case: a chunk's tiles fill the device with few splits) are
    // one round trip: the maximum comes from the m values that the round below loads anyway.
    // More splits take a pass over m first.
    const bool one_round = a.splits_total <= 4;
    float mx = -INFINITY;
    if (!one_round)
        for (int sp = 0; sp < a.splits_total; ++sp) mx = fmaxf(mx, a.part_m[base + (long)sp * n_slots]);
    float m_safe = mx == -INFINITY ? 0.0f : mx;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float lsum = 0.0f;
    const bool vec_ok = (g.head_dim & 3) == 0;
    // four splits per round: their loads are all issued before the first is consumed (the
    // partials are read once: non-temporal)
    for (int sp0 = 0; sp0 < a.splits_total; sp0 += 4) {
        float w[4], lp[4];
        float4_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int sp = min(sp0 + u, a.splits_total - 1); // a repeat of the last one weighs zero below
            const long pidx = base + (long)sp * n_slots;
            w[u] = a.part_m[pidx];
            lp[u] = a.part_l[pidx];
            const float *po = a.part_o + pidx * g.head_dim + c4;
            if (vec_ok) {
                v[u] = __builtin_nontemporal_load(reinterpret_cast<const float4_t *>(po));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) v[u][i] = c4 + i < g.head_dim ? po[i] : 0.0f;
            }
        }
        if (one_round) {
            mx = fmaxf(fmaxf(w[0], w[1]), fmaxf(w[2], w[3])); // repeats of the last split do not move it
            m_safe = mx == -INFINITY ? 0.0f : mx;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float wu = sp0 + u < a.splits_total ? fast_exp2(w[u] - m_safe) : 0.0f;
            lsum += wu * lp[u];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += wu * v[u][i];
        }
    }
    float *dst = a.out + ((long)(slot / g.gqa) * g.q_heads + kvh * g.gqa + slot % g.gqa) * g.head_dim + c4;
    const float inv = 1.0f / lsum;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (c4 + i < g.head_dim) dst[i] = acc[i] * inv;
}

hipError_t launch_merge_rows(const DecodeArgs &a, hipStream_t s) {
    const long total = (long)a.g.kv_heads * a.n_queries * a.g.gqa * ((a.g.head_dim + 3) >> 2);
    hipLaunchKernelGGL(merge_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a);
    return hipGetLastError();
}

// Query slots one workgroup of the kernel covers for a padded head_dim.
int prefill_tile_slots(int P, bool two_tiles) {
    if (P > 256) return 64; // four wavefronts, one per SIMD (the accumulators and query halves are 256 registers)
    return two_tiles && prefill_two_tiles_possible(P) ? 256 : 128;
}
// Two query tiles per wavefront need twice the accumulator and query registers: up to
// head_dim 128.
bool prefill_two_tiles_possible(int P) { return P <= 128; }

template <int P, int TILES, int PG, int WAVES = 8>
static hipError_t launch_tiles(const DecodeArgs &a, dim3 grid, hipStream_t s) {
    constexpr size_t lds = (size_t)2 * PG * 2 * (P / 32) * 64 * sizeof(uint4);
    static std::atomic<uint64_t> lds_ok{0}; // per instantiation
    {
        hipError_t e = allow_full_lds(reinterpret_cast<const void *>(&prefill_tile_kernel<P, TILES, PG, WAVES>), lds_ok);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((prefill_tile_kernel<P, TILES, PG, WAVES>), grid, dim3(WAVES * 64), lds, s, a);
    return hipGetLastError();
}

hipError_t launch_prefill_tiles(const DecodeArgs &a, hipStream_t s) {
    const int n_slots = a.n_queries * a.g.gqa;
    const bool two = a.tiles2 && prefill_two_tiles_possible(a.g.P);
    const int per_wg = prefill_tile_slots(a.g.P, two);
    dim3 grid((unsigned)a.splits, (unsigned)a.g.kv_heads, (unsigned)((n_slots + per_wg - 1) / per_wg));
    switch (a.g.P) {
    case 32: return two ? launch_tiles<32, 2, 8>(a, grid, s) : launch_tiles<32, 1, 8>(a, grid, s);
    case 64: return two ? launch_tiles<64, 2, 8>(a, grid, s) : launch_tiles<64, 1, 8>(a, grid, s);
    case 128: return two ? launch_tiles<128, 2, 8>(a, grid, s) : launch_tiles<128, 1, 8>(a, grid, s);
    case 256: return launch_tiles<256, 1, 4>(a, grid, s);
    case 512: return launch_tiles<512, 1, 2, 4>(a, grid, s);
    default: return hipErrorInvalidValue;
    }
}

} // namespace skv
