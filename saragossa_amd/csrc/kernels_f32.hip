// gfx950 kernels of the KV hot path, part 4: the f32 storage mode of the cache
// (KvElement::F32, src/decode_resident/attention.rs:26-45; the reference's default for greedy
// decoding, src/decode_resident/utils.rs:202-210). Same pages, block table, ring and split
// partials as the bf16 mode; the tiles hold f32 and the products run on the f32 matrix
// instruction (v_mfma_f32_16x16x4_f32), which has the operand layout of the bf16 kernels'
// 16x16 tiles with a contraction of 4 per instruction.
//
// Tile layouts (one tile = 16 rows x P dims of one kv head, P * 16 floats), chosen so that a
// wavefront's operand fetch is one contiguous KiB and a lane's 16-byte load is four
// consecutive contraction steps:
//   K: float4 unit (m, j, r) = dims 16m + 4j .. +3 of row r, at unit index m * 64 + j * 16 + r
//   V: float4 unit (c, jj, dd) = rows 4jj .. 4jj+3 of dim 16c + dd, at unit index c * 64 + jj * 16 + dd
#include <type_traits>

#include "skv_internal.h"

namespace skv {

typedef __attribute__((ext_vector_type(4))) float float4_t;

namespace {
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
} // namespace

bool f32_decode_kernel_serves(const DecodeArgs &a);

// ------------------------------------------------------------------------------------
// append: rows [n_rows, kv_dim] f32 -> tiles, verbatim. One thread per (row, kv head, four
// dims): a 16-byte K store and four 4-byte V stores.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void append_f32_kernel(AppendArgs a) {
    const Geom g = a.g;
    const int groups = (g.head_dim + 3) >> 2;
    const long per_row = (long)g.kv_heads * groups;
    const long total = per_row * a.n_rows;
    const int kv_dim = g.kv_heads * g.head_dim;
    float *k_pool = reinterpret_cast<float *>(a.k_pool);
    float *v_pool = reinterpret_cast<float *>(a.v_pool);
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const int row = (int)(t / per_row);
        const int rem = (int)(t - (long)row * per_row);
        const int kvh = rem / groups;
        const int d0 = (rem - kvh * groups) * 4;
        const long slot = slot_of(a.first_pos + row, g.ring_rows);
        const int page = a.table[slot >> 4];
        const int r = (int)(slot & 15);
        // tile_elems and page_elems count 16-bit units: two per float
        const long tile = ((long)page * g.page_elems + (long)kvh * g.tile_elems) >> 1;
        const float *ks = a.k_src + (long)row * kv_dim + kvh * g.head_dim + d0;
        const float *vs = a.v_src + (long)row * kv_dim + kvh * g.head_dim + d0;
        float4_t kq;
#pragma unroll
        for (int e = 0; e < 4; ++e) kq[e] = d0 + e < g.head_dim ? ks[e] : 0.0f;
        *reinterpret_cast<float4_t *>(k_pool + tile + k_index_f32(r, d0)) = kq;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (d0 + e < g.head_dim) v_pool[tile + v_index_f32(r, d0 + e)] = vs[e];
    }
}

hipError_t launch_append_f32(const AppendArgs &a, hipStream_t s) {
    const long total = (long)a.g.kv_heads * ((a.g.head_dim + 3) >> 2) * a.n_rows;
    long blocks = (total + 255) / 256;
    if (blocks > 65535 * 4) blocks = 65535 * 4;
    hipLaunchKernelGGL(append_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    return hipGetLastError();
}

// gather: tiles -> row-major f32 rows [n_rows, kv_dim], through the block table.
__global__ __launch_bounds__(256) void gather_f32_kernel(GatherArgs a) {
    const Geom g = a.g;
    const int kv_dim = g.kv_heads * g.head_dim;
    const long total = (long)kv_dim * a.n_rows;
    const float *k_pool = reinterpret_cast<const float *>(a.k_pool);
    const float *v_pool = reinterpret_cast<const float *>(a.v_pool);
    float *k_dst = reinterpret_cast<float *>(a.k_dst);
    float *v_dst = reinterpret_cast<float *>(a.v_dst);
    for (long t = (long)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const int row = (int)(t / kv_dim);
        const int col = (int)(t - (long)row * kv_dim);
        const int kvh = col / g.head_dim;
        const int d = col - kvh * g.head_dim;
        const long slot = slot_of(a.first_pos + row, g.ring_rows);
        const int page = a.table[slot >> 4];
        const int r = (int)(slot & 15);
        const long tile = ((long)page * g.page_elems + (long)kvh * g.tile_elems) >> 1;
        if (k_dst) k_dst[t] = k_pool[tile + k_index_f32(r, d)];
        if (v_dst) v_dst[t] = v_pool[tile + v_index_f32(r, d)];
    }
}

hipError_t launch_gather_f32(const GatherArgs &a, hipStream_t s) {
    const long total = (long)a.g.kv_heads * a.g.head_dim * a.n_rows;
    long blocks = (total + 255) / 256;
    if (blocks > 65535 * 4) blocks = 65535 * 4;
    hipLaunchKernelGGL(gather_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------
// Attention over the f32 cache, decode and chunked prefill alike (cached_attention_one and
// cached_attention_prefill_rows, src/decoder/attention_ops.rs:976-1046): query slot
// (i, g) = query row i, head g of the kv head's group, attends positions up to
// min(q_pos0 + i, limit_cap) through the layer's window.
//
// grid (splits, kv heads, tiles of 16 query slots); a workgroup is four wavefronts that take
// the pages of its split in turn. A wavefront holds the 16 slots' queries (pre-scaled by
// log2(e)/sqrt(head_dim)) and its own (o, m, l) in registers and streams K and V tiles straight
// from memory into the matrix operands: S^T = K . Q^T (16 keys x 16 slots), one online-softmax
// step in base 2 per page, O^T += V^T . P^T with the probabilities taken from the very
// registers the scores arrived in (contraction step k of lane group jj is key 4jj + k, which
// is where the score tile keeps it). The four wavefronts' states meet in LDS at the end; the
// workgroup writes the context (one split) or its (o, m, l) partial in the layout of the
// bf16 kernels, for the same merge kernels.
// ------------------------------------------------------------------------------------
template <int P>
__global__ __launch_bounds__(256) void f32_split_kernel(DecodeArgs a) {
    constexpr int NT = P / 16;
    extern __shared__ __attribute__((aligned(16))) float4_t xch[]; // [4 wavefronts][NT][64] o | [4][16] m | [4][16] l
    const Geom g = a.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15; // slot column of the tiles; key row of the K operand; dim of the V operand
    const int j = lane >> 4; // lane group
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    const int G = g.gqa;
    const int n_slots = a.n_queries * G;
    const int slot0 = blockIdx.z * 16;
    const int s_last = min(slot0 + 15, n_slots - 1);
    const int my_slot = min(slot0 + n, n_slots - 1);

    auto pos_of = [&](int slot) { return a.q_pos0 + slot / G; };
    auto limit_of = [&](int slot) { return min(pos_of(slot), a.limit_cap); };
    auto ws_of = [&](int slot) { return a.window > 0 ? max(a.window_start, pos_of(slot) + 1 - a.window) : a.window_start; };
    const int my_limit = limit_of(my_slot), my_ws = ws_of(my_slot);
    const int t_ws_lo = ws_of(slot0), t_ws_hi = ws_of(s_last);
    const int t_lim_lo = limit_of(slot0), t_lim_hi = limit_of(s_last);

    // pages any slot of the tile can see, divided among the splits, then among the wavefronts
    const int page_lo = g.ring_rows > 0 ? 0 : t_ws_lo >> 4;
    const int page_hi = g.ring_rows > 0 ? a.n_pages : (t_lim_hi >> 4) + 1;
    const unsigned span = (unsigned)max(page_hi - page_lo, 0);
    const int pb0 = page_lo + (int)(((unsigned)split * span) / (unsigned)a.splits);
    const int pb1 = page_lo + (int)(((unsigned)(split + 1) * span) / (unsigned)a.splits);

    const float *k_pool = reinterpret_cast<const float *>(a.k_pool);
    const float *v_pool = reinterpret_cast<const float *>(a.v_pool);
    const int last_page = a.page_first + a.n_pages - 1;
    // Block-table entries of this wavefront's next 64 pages, one per lane, read back with
    // v_readlane: a page's requests then depend on no load of their own (a table read in
    // front of every page stalls the wavefront for a round trip before it can ask).
    int ids = 0;
    auto fetch_ids = [&](int first_pb) __attribute__((always_inline)) {
        ids = a.table[min(first_pb + 4 * lane, last_page)];
    };
    int ids_base = pb0 + wave; // the page lane 0's entry belongs to
    fetch_ids(ids_base);
    // (every page of [page_lo, page_hi) is visible to some slot of the tile)
    auto fetch_tile = [&](int pb, const float *pool, float4_t (&dst)[NT]) __attribute__((always_inline)) {
        if (pb >= ids_base + 256) { // uniform: the wavefront has walked 64 pages
            ids_base += 256;
            fetch_ids(ids_base);
        }
        const int page = __builtin_amdgcn_readlane(ids, (pb - ids_base) >> 2);
        const long tile = ((long)page * g.page_elems + (long)kvh * g.tile_elems) >> 1;
        const float4_t *t = reinterpret_cast<const float4_t *>(pool + tile);
        // (plain loads: this kernel serves chunks, whose query tiles share every page through
        // the L2 of their XCD; the decode kernel below reads its pages once and says so)
#pragma unroll
        for (int m = 0; m < NT; ++m) dst[m] = t[m * 64 + lane];
    };
    // the page whose table entry lane `idx` of `ids` holds, K then V (no conditional reload)
    auto fetch = [&](int idx, float4_t (&kq)[NT], float4_t (&vq)[NT]) __attribute__((always_inline)) {
        const int page = __builtin_amdgcn_readlane(ids, idx);
        const long tile = ((long)page * g.page_elems + (long)kvh * g.tile_elems) >> 1;
        const float4_t *kt = reinterpret_cast<const float4_t *>(k_pool + tile) + lane;
        const float4_t *vt = reinterpret_cast<const float4_t *>(v_pool + tile) + lane;
#pragma unroll
        for (int m = 0; m < NT; ++m) kq[m] = kt[m * 64];
#pragma unroll
        for (int m = 0; m < NT; ++m) vq[m] = vt[m * 64];
    };
    // Up to head_dim 256 a wavefront holds two pages (K and V each); above, one tile at a
    // time (K, then V in the same registers).
    constexpr bool TWO_PAGES = P <= 256;
    constexpr int NB = TWO_PAGES ? NT : 1;
    float4_t k_a[NT], v_a[NB], k_b[NB], v_b[NB];
    int pb = pb0 + wave;

    // queries: lane (slot n, group j) holds dims 16m + 4j .. +3 of every block m
    float4_t qv[NT];
    {
        const float *qrow = a.q + ((long)(my_slot / G) * g.q_heads + kvh * G + my_slot % G) * g.head_dim;
        // all loads first, unconditional from clamped addresses (one round trip); dims past
        // head_dim are zeroed afterwards
        if (a.q_vec) {
#pragma unroll
            for (int m = 0; m < NT; ++m)
                qv[m] = *reinterpret_cast<const float4_t *>(qrow + min(m * 16 + j * 4, g.head_dim - 4));
        } else {
#pragma unroll
            for (int m = 0; m < NT; ++m) {
#pragma unroll
                for (int e = 0; e < 4; ++e) qv[m][e] = qrow[min(m * 16 + j * 4 + e, g.head_dim - 1)];
            }
        }
        // The first page is requested right behind the queries (loads return in order: in
        // front of them it would hold them back for the whole page) and without a condition: a
        // wavefront without pages reads a page it ignores, and the wait for the queries
        // below counts exactly the page's loads.
        if constexpr (TWO_PAGES) fetch(0, k_a, v_a);
        else fetch_tile(min(pb, last_page), k_pool, k_a);
#pragma unroll
        for (int m = 0; m < NT; ++m) {
#pragma unroll
            for (int e = 0; e < 4; ++e) qv[m][e] = m * 16 + j * 4 + e < g.head_dim ? qv[m][e] * a.qscale : 0.0f;
        }
    }
    float4_t o[NT];
#pragma unroll
    for (int c = 0; c < NT; ++c) o[c] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.0f;

    // scores and probabilities of one page (pv), running state updated
    auto attend = [&](int pb, const float4_t (&kq)[NT], float (&pv)[4]) {
        const int slot_a = pb * 16; // first cache slot of the page
        // S^T = K . Q^T: two accumulators so that consecutive products do not wait for each other
        float4_t s0 = float4_t{0.f, 0.f, 0.f, 0.f}, s1 = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < NT; ++m) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][0], qv[m][0], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][1], qv[m][1], s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][2], qv[m][2], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][3], qv[m][3], s1, 0, 0, 0);
        }
        float sv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) sv[e] = s0[e] + s1[e];
        const bool interior = g.ring_rows == 0 && slot_a >= t_ws_hi && slot_a + 15 <= t_lim_lo;
        if (!interior) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int slot = slot_a + j * 4 + e; // this lane's key e
                int pos = slot;
                if (g.ring_rows > 0) pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
                sv[e] = (pos >= my_ws && pos <= my_limit) ? sv[e] : -INFINITY;
            }
        }
        float m_blk = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
        m_blk = rows_max(m_blk);
        const float m_new = fmaxf(m_run, m_blk);
        const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        float psum = 0.0f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pv[e] = fast_exp2(sv[e] - m_safe);
            psum += pv[e];
        }
        l_run = l_run * alpha + psum;
        const bool rescale = alpha != 1.0f && m_run != -INFINITY; // a slot without a key so far holds zeros
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(rescale)) {
#pragma unroll
            for (int c = 0; c < NT; ++c) o[c] *= alpha;
        }
    };
    // Keys that no slot of the tile attends (rows at or past the length after a rollback, ring
    // rows not valid, rows before the window) have zero probability, but 0 x NaN is NaN: on the
    // pages at the edges of the attended range (and ring pages) their V values are replaced by
    // zero in the registers, so the bits of such a row never reach a context (the reference
    // never reads them, src/decode_resident/kernels.rs:11-88).
    auto mask_v = [&](int pb, float4_t (&vq)[NT]) {
        const int slot_a = pb * 16;
        const bool inside = g.ring_rows == 0 && slot_a >= t_ws_lo && slot_a + 15 <= t_lim_hi;
        if (inside) return;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int slot = slot_a + j * 4 + k; // this lane's key k
            int pos = slot;
            if (g.ring_rows > 0) pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
            const bool live = pos >= t_ws_lo && pos <= t_lim_hi;
#pragma unroll
            for (int c = 0; c < NT; ++c) vq[c][k] = live ? vq[c][k] : 0.0f;
        }
    };
    // O^T += V^T . P^T, contraction step outermost: consecutive products use different accumulators
    auto accumulate = [&](const float4_t (&vq)[NT], const float (&pv)[4]) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int c = 0; c < NT; ++c) o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vq[c][k], pv[k], o[c], 0, 0, 0);
        }
    };
    if constexpr (TWO_PAGES) {
        // The page after the one being multiplied is on its way into a second set of registers:
        // its K tile is asked for in front of this page's QK products, its V tile in front of
        // the PV products, each tile's loads back to back (spread out among the products, one
        // load per four, they arrive more slowly: 353.7 against 345.9 us per token at 32768
        // rows of kv2/hd256).
        const int n_it = pb < pb1 ? (pb1 - pb + 3) / 4 : 0;
        auto next_tile = [&](int at, const float *pool) __attribute__((always_inline)) {
            const int page = __builtin_amdgcn_readlane(ids, (at - ids_base) >> 2);
            return reinterpret_cast<const float4_t *>(pool + (((long)page * g.page_elems + (long)kvh * g.tile_elems) >> 1)) + lane;
        };
        // page `at` from (kq, vq); PREFETCH: page at + 4 into (kn, vn) meanwhile
        auto step = [&](int at, const float4_t (&kq)[NT], float4_t (&vq)[NT], float4_t (&kn)[NT], float4_t (&vn)[NT],
                        auto prefetch) __attribute__((always_inline)) {
            constexpr bool PREFETCH = decltype(prefetch)::value;
            float pv[4];
            {
                const float4_t *kt = PREFETCH ? next_tile(at + 4, k_pool) : nullptr;
                const int slot_a = at * 16;
                float4_t s0 = float4_t{0.f, 0.f, 0.f, 0.f}, s1 = float4_t{0.f, 0.f, 0.f, 0.f};
                if constexpr (PREFETCH) {
#pragma unroll
                    for (int m = 0; m < NT; ++m) kn[m] = kt[m * 64];
                }
#pragma unroll
                for (int m = 0; m < NT; ++m) {
                    s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][0], qv[m][0], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][1], qv[m][1], s1, 0, 0, 0);
                    s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][2], qv[m][2], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][3], qv[m][3], s1, 0, 0, 0);
                }
                float sv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) sv[e] = s0[e] + s1[e];
                const bool interior = g.ring_rows == 0 && slot_a >= t_ws_hi && slot_a + 15 <= t_lim_lo;
                if (!interior) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int slot = slot_a + j * 4 + e; // this lane's key e
                        int pos = slot;
                        if (g.ring_rows > 0) pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
                        sv[e] = (pos >= my_ws && pos <= my_limit) ? sv[e] : -INFINITY;
                    }
                }
                float m_blk = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
                m_blk = rows_max(m_blk);
                const float m_new = fmaxf(m_run, m_blk);
                const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
                const float alpha = fast_exp2(m_run - m_safe);
                float psum = 0.0f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pv[e] = fast_exp2(sv[e] - m_safe);
                    psum += pv[e];
                }
                l_run = l_run * alpha + psum;
                const bool rescale = alpha != 1.0f && m_run != -INFINITY; // a slot without a key so far holds zeros
                m_run = m_new;
                if (__builtin_amdgcn_ballot_w64(rescale)) {
#pragma unroll
                    for (int c = 0; c < NT; ++c) o[c] *= alpha;
                }
            }
            mask_v(at, vq);
            {
                const float4_t *vt = PREFETCH ? next_tile(at + 4, v_pool) : nullptr;
                // contraction step outermost: consecutive products use different accumulators
                if constexpr (PREFETCH) {
#pragma unroll
                    for (int m = 0; m < NT; ++m) vn[m] = vt[m * 64];
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
#pragma unroll
                    for (int c = 0; c < NT; ++c) o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vq[c][k], pv[k], o[c], 0, 0, 0);
                }
            }
        };
        const std::true_type with_prefetch{};
        const std::false_type last_page_of_run{};
        // The wavefront's pages in runs of up to 64, the block-table entries one register holds:
        // inside a run no load is conditional (a conditional load makes the compiler wait for
        // everything in flight where it joins), between runs the pipeline drains once.
        for (int done = 0; done < n_it;) {
            const int run = min(n_it - done, 64);
            const int at0 = pb + 4 * done; // first page of the run, already in (k_a, v_a)
            int it = 0;
            for (; it + 2 < run; it += 2) {
                step(at0 + 4 * it, k_a, v_a, k_b, v_b, with_prefetch);
                step(at0 + 4 * it + 4, k_b, v_b, k_a, v_a, with_prefetch);
            }
            if (run - it == 2) {
                step(at0 + 4 * it, k_a, v_a, k_b, v_b, with_prefetch);
                step(at0 + 4 * it + 4, k_b, v_b, k_a, v_a, last_page_of_run);
            } else {
                step(at0 + 4 * it, k_a, v_a, k_b, v_b, last_page_of_run);
            }
            done += run;
            if (done < n_it) {
                ids_base = pb + 4 * done;
                fetch_ids(ids_base);
                fetch(0, k_a, v_a);
            }
        }
    } else {
        // head_dim 257..512: the queries and the accumulators are 256 registers by themselves;
        // K, then V of the page, then K of the next one pass through the same 128
        for (; pb < pb1; pb += 4) {
            float pv[4];
            attend(pb, k_a, pv);
            fetch_tile(pb, v_pool, k_a);
            mask_v(pb, k_a);
            accumulate(k_a, pv);
            if (pb + 4 < pb1) fetch_tile(pb + 4, k_pool, k_a);
        }
    }

    // ---- the four wavefronts' states meet in LDS ------------------------------------------
    float *xm = reinterpret_cast<float *>(xch + 4 * NT * 64);
    float *xl = xm + 64;
    const float l_mine = rows_sum(l_run);
#pragma unroll
    for (int c = 0; c < NT; ++c) xch[(wave * NT + c) * 64 + lane] = o[c];
    if (j == 0) {
        xm[wave * 16 + n] = m_run;
        xl[wave * 16 + n] = l_mine;
    }
    __syncthreads();
    float mw[4], lw[4];
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        mw[w] = xm[w * 16 + n];
        lw[w] = xl[w * 16 + n];
        mx = fmaxf(mx, mw[w]);
    }
    const float m_safe = mx == -INFINITY ? 0.0f : mx;
    float l = 0.0f;
    float sc[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        sc[w] = fast_exp2(mw[w] - m_safe);
        l += sc[w] * lw[w];
    }
    const int slot = slot0 + n;
    if (slot >= n_slots) return;
    float *dst;
    float scale = 1.0f;
    if (a.splits_total == 1) {
        scale = 1.0f / l;
        dst = a.out + ((long)(slot / G) * g.q_heads + kvh * G + slot % G) * g.head_dim;
    } else {
        const long pidx = ((long)kvh * a.splits_total + a.split_base + split) * n_slots + slot;
        dst = a.part_o + pidx * g.head_dim;
        if (j == 0 && wave == 0) {
            a.part_m[pidx] = mx;
            a.part_l[pidx] = l;
        }
    }
    // wavefront w finishes the dim tiles c = w, w + 4, ...
    for (int c = wave; c < NT; c += 4) {
        float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < 4; ++w) acc += xch[(w * NT + c) * 64 + lane] * sc[w];
        acc *= scale;
        const int col = c * 16 + j * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (col + i < g.head_dim) dst[col + i] = acc[i];
    }
}

// ------------------------------------------------------------------------------------
// The same split launch for one query row (decode) up to head_dim 256, in the shape of the
// bf16 decode kernel: eight wavefronts, two per SIMD (four where eight would leave most
// compute units without a workgroup), each with ONE page in its registers (K and V tile, 128
// registers at head_dim 256) and the queries in LDS instead of registers. A wavefront that
// waits for its page, or for the compute unit to accept its next requests, leaves the SIMD's
// matrix pipe to the other one; with one wavefront per SIMD and two pages each (the kernel
// above) the products and the waiting take turns. K registers are refilled right after the
// QK products that read them, V registers right after the PV products.
// Fused append (k_new non-null): the workgroup whose range holds the new row's page stores
// the row into the pools for later steps and keeps it in LDS; the wavefront that walks the
// page patches its registers from there, so nothing is read back in this launch.
// ------------------------------------------------------------------------------------
template <int P, int WAVES, bool PRE>
__device__ __forceinline__ void f32_decode_body(const DecodeArgs &a, const int split, const int kvh) {
    constexpr int NT = P / 16;
    constexpr int THREADS = WAVES * 64;
    extern __shared__ __attribute__((aligned(16))) float4_t lds8[];
    float4_t *q_lds = lds8;                  // [NT][64]: lane (slot n, group j) of block m holds dims 16m + 4j .. +3
    float4_t *xch = lds8 + NT * 64;          // [wavefronts][NT][64] o
    float *xm = reinterpret_cast<float *>(xch + WAVES * NT * 64); // [wavefronts][16] m | l
    float *xl = xm + WAVES * 16;
    float *new_k = xl + WAVES * 16;          // [P] the appended row
    float *new_v = new_k + P;
    const Geom g = a.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int j = lane >> 4;
    const int G = g.gqa;
    const int n_slots = G; // one query row
    const int q_stride = a.q_head_stride > 0 ? a.q_head_stride : g.head_dim;
    constexpr int slot0 = 0; // at most 16 heads per group: one tile of query slots
    const int my_limit = min(a.q_pos0, a.limit_cap);
    const int my_ws = a.window > 0 ? max(a.window_start, a.q_pos0 + 1 - a.window) : a.window_start;

    const int page_lo = g.ring_rows > 0 ? 0 : my_ws >> 4;
    const int page_hi = g.ring_rows > 0 ? a.n_pages : (my_limit >> 4) + 1;
    const unsigned span = (unsigned)max(page_hi - page_lo, 0);
    const int pb0 = page_lo + (int)(((unsigned)split * span) / (unsigned)a.splits);
    const int pb1 = page_lo + (int)(((unsigned)(split + 1) * span) / (unsigned)a.splits);
    const int pb = pb0 + wave;
    const int n_it = pb < pb1 ? (pb1 - pb + WAVES - 1) / WAVES : 0;

    const float *k_pool = reinterpret_cast<const float *>(a.k_pool);
    const float *v_pool = reinterpret_cast<const float *>(a.v_pool);
    const int last_page = a.page_first + a.n_pages - 1;
    // block-table entries of this wavefront's next 64 pages, one per lane
    int ids = 0;
    auto fetch_ids = [&](int first_pb) __attribute__((always_inline)) {
        ids = a.table[min(first_pb + WAVES * lane, last_page)];
    };
    fetch_ids(pb);

    // ---- fused append: the new row goes to the pools and to LDS
    const int pb_new = a.new_slot >> 4;
    const int r_new = a.new_slot & 15;
    const bool appends = a.k_new != nullptr && pb_new >= pb0 && pb_new < pb1;

    // ---- PRE: q and the new k row arrive raw; the per-head RMSNorm and the rotation of the
    // position are applied here, in LDS (the area the wavefronts' states use at the end), with
    // the arithmetic and the order of rms_norm_rope_heads_at (src/decoder/attention_ops.rs:682-777),
    // so that the finished rows, and the k row this launch stores, equal the CPU path's.
    constexpr int PS = P + 1;      // row stride: lanes walking different rows hit different banks
    constexpr int SQS = P + 4;     // squares: 16-byte aligned rows
    constexpr int PRE_ROWS = 17;   // 16 query slots + the k row
    float *pre_raw = reinterpret_cast<float *>(xch);   // [PRE_ROWS][PS]
    float *pre_out = pre_raw + PRE_ROWS * PS;          // [PRE_ROWS][PS]
    float *pre_wq = pre_out + PRE_ROWS * PS;           // [P]
    float *pre_wk = pre_wq + P;                        // [P]
    float *pre_rope = pre_wk + P;                      // [P]: (cos, sin) pairs
    float *pre_inv = pre_rope + P;                     // [PRE_ROWS] (+5 keeps pre_sq 16-byte aligned)
    float *pre_sq = pre_inv + PRE_ROWS + 5;            // [PRE_ROWS][SQS]
    static_assert(!PRE || ((size_t)(2 * PRE_ROWS * PS + 3 * P + PRE_ROWS + 5 + PRE_ROWS * SQS) * sizeof(float) <=
                           (size_t)WAVES * NT * 64 * sizeof(float4_t)),
                  "the pre-KV scratch fits the exchange area it borrows");
    const int rows = min(16, n_slots - slot0);
    if constexpr (PRE) {
        auto sq_of = [](float x) {
#pragma clang fp contract(off)
            return x * x;
        };
        for (int e = tid; e < rows * P; e += THREADS) {
            const int r = e / P, c = e % P;
            const float x = c < g.head_dim ? a.q[(long)(kvh * G + slot0 + r) * q_stride + c] : 0.0f;
            pre_raw[r * PS + c] = x;
            pre_sq[r * SQS + c] = sq_of(x);
        }
        for (int c = tid; c < P; c += THREADS) {
            const float x = (appends && c < g.head_dim) ? a.k_new[kvh * g.head_dim + c] : 0.0f;
            pre_raw[rows * PS + c] = x;
            pre_sq[rows * SQS + c] = sq_of(x);
            pre_wq[c] = (a.q_norm_w && c < g.head_dim) ? a.q_norm_w[c] : 1.0f;
            pre_wk[c] = (a.k_norm_w && c < g.head_dim) ? a.k_norm_w[c] : 1.0f;
            pre_rope[c] = (a.rope && c < a.rope_dims) ? a.rope[c] : 0.0f;
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
                pre_out[r * PS + c] = norm_rope_elem(pre_raw + r * PS, c, pre_inv[r], w, rope, a.rope_dims, a.rope_style);
            }
        }
        __syncthreads();
    }
    if (appends) {
        const long tile_at = ((long)a.new_page * g.page_elems + (long)kvh * g.tile_elems) >> 1;
        for (int d = tid; d < P; d += THREADS) {
            float kf = 0.0f, vf = 0.0f;
            if (d < g.head_dim) {
                kf = PRE ? pre_out[rows * PS + d] : a.k_new[kvh * g.head_dim + d];
                vf = a.v_new[kvh * g.head_dim + d];
                const_cast<float *>(k_pool)[tile_at + k_index_f32(r_new, d)] = kf;
                const_cast<float *>(v_pool)[tile_at + v_index_f32(r_new, d)] = vf;
            }
            new_k[d] = kf;
            new_v[d] = vf;
        }
    }

    // ---- queries of the group to LDS, scaled; dims past head_dim are zero
    {
        constexpr int QU = (NT * 64 + THREADS - 1) / THREADS;
        float4_t qv[QU];
#pragma unroll
        for (int u = 0; u < QU; ++u) {
            const int idx = min(tid + u * THREADS, NT * 64 - 1);
            const int m = idx >> 6, nn = idx & 15, jj = (idx >> 4) & 3;
            const int slot = min(slot0 + nn, n_slots - 1);
            if constexpr (PRE) {
                const float *qrow = pre_out + (slot - slot0) * PS;
#pragma unroll
                for (int e = 0; e < 4; ++e) qv[u][e] = qrow[min(m * 16 + jj * 4 + e, g.head_dim - 1)];
            } else {
                const float *qrow = a.q + (long)(kvh * G + slot) * q_stride;
                if (a.q_vec) {
                    qv[u] = *reinterpret_cast<const float4_t *>(qrow + min(m * 16 + jj * 4, g.head_dim - 4));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) qv[u][e] = qrow[min(m * 16 + jj * 4 + e, g.head_dim - 1)];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < QU; ++u) {
            const int idx = tid + u * THREADS;
            if (idx < NT * 64) {
                const int m = idx >> 6, jj = (idx >> 4) & 3;
                float4_t v = qv[u];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = m * 16 + jj * 4 + e < g.head_dim ? v[e] * a.qscale : 0.0f;
                q_lds[idx] = v;
            }
        }
    }
    float4_t kq[NT], vq[NT];
    auto tile_of = [&](int idx, const float *pool) __attribute__((always_inline)) {
        const int page = __builtin_amdgcn_readlane(ids, idx);
        return reinterpret_cast<const float4_t *>(pool + (((long)page * g.page_elems + (long)kvh * g.tile_elems) >> 1)) + lane;
    };
    auto load_tile = [&](const float4_t *t, float4_t (&dst)[NT]) __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < NT; ++m) dst[m] = __builtin_nontemporal_load(t + m * 64);
    };
    // The queries are staged before the first page is asked for: a compute unit accepts
    // requests only as fast as memory answers them, and a barrier behind a page's loads would
    // hold every wavefront until the last one's were accepted. The first page comes without a
    // condition (a wavefront without pages reads a page it ignores).
    __syncthreads();
    load_tile(tile_of(0, k_pool), kq);
    load_tile(tile_of(0, v_pool), vq);

    float4_t o[NT];
#pragma unroll
    for (int c = 0; c < NT; ++c) o[c] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.0f;

    auto attend = [&](int at, float (&pv)[4]) __attribute__((always_inline)) {
        const int slot_a = at * 16;
        // the queries come from LDS for every page, through an offset the compiler cannot see
        // through: hoisted out of the page loop they would take 64 registers that do not exist
        int q_at = lane;
        asm volatile("" : "+v"(q_at));
        float4_t s0 = float4_t{0.f, 0.f, 0.f, 0.f}, s1 = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < NT; ++m) {
            const float4_t qv = q_lds[m * 64 + q_at];
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][0], qv[0], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][1], qv[1], s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][2], qv[2], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kq[m][3], qv[3], s1, 0, 0, 0);
        }
        float sv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) sv[e] = s0[e] + s1[e];
        const bool interior = g.ring_rows == 0 && slot_a >= my_ws && slot_a + 15 <= my_limit;
        if (!interior) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int slot = slot_a + j * 4 + e;
                int pos = slot;
                if (g.ring_rows > 0) pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
                sv[e] = (pos >= my_ws && pos <= my_limit) ? sv[e] : -INFINITY;
            }
        }
        float m_blk = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
        m_blk = rows_max(m_blk);
        const float m_new = fmaxf(m_run, m_blk);
        const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        float psum = 0.0f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pv[e] = fast_exp2(sv[e] - m_safe);
            psum += pv[e];
        }
        l_run = l_run * alpha + psum;
        const bool rescale = alpha != 1.0f && m_run != -INFINITY; // a slot without a key so far holds zeros
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(rescale)) {
#pragma unroll
            for (int c = 0; c < NT; ++c) o[c] *= alpha;
        }
    };
    // V of keys that are not attended is replaced by zero on the pages at the edges of the
    // range (and ring pages): 0 x NaN would be NaN, and the reference never reads those rows
    // (src/decode_resident/kernels.rs:11-88)
    auto mask_v = [&](int at) __attribute__((always_inline)) {
        const int slot_a = at * 16;
        const bool inside = g.ring_rows == 0 && slot_a >= my_ws && slot_a + 15 <= my_limit;
        if (inside) return;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int slot = slot_a + j * 4 + k;
            int pos = slot;
            if (g.ring_rows > 0) pos = slot <= a.ring_t ? a.ring_base + slot : a.ring_base - g.ring_rows + slot;
            const bool live = pos >= my_ws && pos <= my_limit;
#pragma unroll
            for (int c = 0; c < NT; ++c) vq[c][k] = live ? vq[c][k] : 0.0f;
        }
    };
    // the page that receives the appended row takes it from LDS instead of memory
    auto patch_k = [&](int at) __attribute__((always_inline)) {
        if (appends && at == pb_new && n == r_new) {
#pragma unroll
            for (int m = 0; m < NT; ++m) kq[m] = *reinterpret_cast<const float4_t *>(new_k + m * 16 + j * 4);
        }
    };
    auto patch_v = [&](int at) __attribute__((always_inline)) {
        if (appends && at == pb_new && j == (r_new >> 2)) {
            const int e = r_new & 3;
#pragma unroll
            for (int c = 0; c < NT; ++c) {
                const float x = new_v[c * 16 + n];
                vq[c][0] = e == 0 ? x : vq[c][0];
                vq[c][1] = e == 1 ? x : vq[c][1];
                vq[c][2] = e == 2 ? x : vq[c][2];
                vq[c][3] = e == 3 ? x : vq[c][3];
            }
        }
    };
    auto accumulate = [&](const float (&pv)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int c = 0; c < NT; ++c) o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vq[c][k], pv[k], o[c], 0, 0, 0);
        }
    };
    // the wavefront's pages in runs of up to 64 (the table entries one register holds); inside
    // a run the steady state is unconditional and the last page is peeled, so the waits count
    // exactly the loads in flight
    for (int done = 0; done < n_it;) {
        const int run = min(n_it - done, 64);
        const int at0 = pb + WAVES * done;
        for (int it = 0; it + 1 < run; ++it) {
            const int at = at0 + WAVES * it;
            float pv[4];
            patch_k(at);
            attend(at, pv);
            load_tile(tile_of(it + 1, k_pool), kq);
            patch_v(at);
            mask_v(at);
            accumulate(pv);
            load_tile(tile_of(it + 1, v_pool), vq);
        }
        {
            const int at = at0 + WAVES * (run - 1);
            float pv[4];
            patch_k(at);
            attend(at, pv);
            patch_v(at);
            mask_v(at);
            accumulate(pv);
        }
        done += run;
        if (done < n_it) {
            fetch_ids(pb + WAVES * done);
            load_tile(tile_of(0, k_pool), kq);
            load_tile(tile_of(0, v_pool), vq);
        }
    }

    // ---- the wavefronts' states meet in LDS (an area of their own: a wavefront that
    // has finished does not wait for the others to stop reading the queries)
    const float l_mine = rows_sum(l_run);
#pragma unroll
    for (int c = 0; c < NT; ++c) xch[(wave * NT + c) * 64 + lane] = o[c];
    if (j == 0) {
        xm[wave * 16 + n] = m_run;
        xl[wave * 16 + n] = l_mine;
    }
    __syncthreads();
    float mx = -INFINITY;
    float mw[WAVES];
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        mw[w] = xm[w * 16 + n];
        mx = fmaxf(mx, mw[w]);
    }
    const float m_safe = mx == -INFINITY ? 0.0f : mx;
    float l = 0.0f;
    float sc[WAVES];
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        sc[w] = fast_exp2(mw[w] - m_safe);
        l += sc[w] * xl[w * 16 + n];
    }
    const int slot = slot0 + n;
    if (slot >= n_slots) return;
    float *dst;
    float scale = 1.0f;
    const float *gp = nullptr;
    if (a.splits_total == 1) {
        scale = 1.0f / l;
        dst = a.out + (long)(kvh * G + slot) * g.head_dim;
        if (a.gate) gp = a.gate + (long)(kvh * G + slot) * q_stride;
    } else {
        const long pidx = ((long)kvh * a.splits_total + a.split_base + split) * n_slots + slot;
        dst = a.part_o + pidx * g.head_dim;
        if (j == 0 && wave == 0) {
            a.part_m[pidx] = mx;
            a.part_l[pidx] = l;
        }
    }
    // wavefront w finishes the dim tiles c = w, w + 8, ...
    for (int c = wave; c < NT; c += WAVES) {
        float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < WAVES; ++w) acc += xch[(w * NT + c) * 64 + lane] * sc[w];
        acc *= scale;
        const int col = c * 16 + j * 4;
        if (gp) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (col + i < g.head_dim) acc[i] *= sigmoid_gate(gp[col + i]);
        }
        if (a.splits_total > 1 && (g.head_dim & 3) == 0) {
            if (col < g.head_dim) __builtin_nontemporal_store(acc, reinterpret_cast<float4_t *>(dst + col));
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (col + i < g.head_dim) dst[col + i] = acc[i];
        }
    }
}

template <int P, int WAVES, bool PRE>
__global__ __launch_bounds__(WAVES * 64) void f32_decode_kernel(DecodeArgs a) {
    f32_decode_body<P, WAVES, PRE>(a, blockIdx.x, blockIdx.y);
}

// Several independent sequences of the same model layer in one launch: grid z is the
// sequence, grid x covers the largest split count and the others leave early.
template <int P, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void f32_decode_batch_kernel(DecodeBatchArgs b) {
    const DecodeArgs &a = b.seq[blockIdx.z];
    if ((int)blockIdx.x >= a.splits) return;
    f32_decode_body<P, WAVES, false>(a, blockIdx.x, blockIdx.y);
}

template <int P, int WAVES>
constexpr size_t f32_decode_lds() {
    return (size_t)((P / 16) * 64 + WAVES * (P / 16) * 64) * sizeof(float4_t) + (2 * WAVES * 16 + 2 * P) * sizeof(float);
}

template <int P, int WAVES, bool PRE>
static hipError_t launch_f32_decode_pre(const DecodeArgs &a, dim3 grid, hipStream_t s) {
    constexpr size_t lds = f32_decode_lds<P, WAVES>();
    static_assert(lds <= 160 * 1024, "queries and the wavefronts' states share the LDS of a compute unit");
    static std::atomic<uint64_t> lds_ok{0}; // per instantiation
    {
        hipError_t e = allow_full_lds(reinterpret_cast<const void *>(&f32_decode_kernel<P, WAVES, PRE>), lds_ok);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((f32_decode_kernel<P, WAVES, PRE>), grid, dim3(WAVES * 64), lds, s, a);
    return hipGetLastError();
}
template <int P, int WAVES>
static hipError_t launch_f32_decode(const DecodeArgs &a, dim3 grid, hipStream_t s) {
    return a.pre ? launch_f32_decode_pre<P, WAVES, true>(a, grid, s) : launch_f32_decode_pre<P, WAVES, false>(a, grid, s);
}

template <int P>
static hipError_t launch_f32(const DecodeArgs &a, dim3 grid, hipStream_t s) {
    constexpr size_t lds = (size_t)4 * (P / 16) * 64 * sizeof(float4_t) + 2 * 64 * sizeof(float);
    static std::atomic<uint64_t> lds_ok{0}; // per instantiation
    {
        hipError_t e = allow_full_lds(reinterpret_cast<const void *>(&f32_split_kernel<P>), lds_ok);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((f32_split_kernel<P>), grid, dim3(256), lds, s, a);
    return hipGetLastError();
}

// The split launch of an f32 layer; the caller merges (launch_merge for one query row,
// launch_merge_rows for a chunk) when splits_total > 1.
hipError_t launch_f32_split(const DecodeArgs &a, hipStream_t s) {
    const int n_slots = a.n_queries * a.g.gqa;
    dim3 grid((unsigned)a.splits, (unsigned)a.g.kv_heads, (unsigned)((n_slots + 15) / 16));
    if (f32_decode_kernel_serves(a)) {
        const bool w8 = a.waves == 8;
        switch (a.g.P) {
        case 32: return w8 ? launch_f32_decode<32, 8>(a, grid, s) : launch_f32_decode<32, 4>(a, grid, s);
        case 64: return w8 ? launch_f32_decode<64, 8>(a, grid, s) : launch_f32_decode<64, 4>(a, grid, s);
        case 128: return w8 ? launch_f32_decode<128, 8>(a, grid, s) : launch_f32_decode<128, 4>(a, grid, s);
        case 256: return w8 ? launch_f32_decode<256, 8>(a, grid, s) : launch_f32_decode<256, 4>(a, grid, s);
        default: break;
        }
    }
    if (a.k_new || a.pre) return hipErrorInvalidValue; // the chunk kernel has no fused append or pre-KV step
    switch (a.g.P) {
    case 32: return launch_f32<32>(a, grid, s);
    case 64: return launch_f32<64>(a, grid, s);
    case 128: return launch_f32<128>(a, grid, s);
    case 256: return launch_f32<256>(a, grid, s);
    case 512: return launch_f32<512>(a, grid, s);
    default: return hipErrorInvalidValue;
    }
}

template <int P, int WAVES>
static hipError_t launch_f32_batch(const DecodeBatchArgs &b, int n_seq, int max_splits, hipStream_t s) {
    constexpr size_t lds = f32_decode_lds<P, WAVES>();
    static std::atomic<uint64_t> lds_ok{0}; // per instantiation
    {
        hipError_t e = allow_full_lds(reinterpret_cast<const void *>(&f32_decode_batch_kernel<P, WAVES>), lds_ok);
        if (e != hipSuccess) return e;
    }
    dim3 grid((unsigned)max_splits, (unsigned)b.seq[0].g.kv_heads, (unsigned)n_seq);
    hipLaunchKernelGGL((f32_decode_batch_kernel<P, WAVES>), grid, dim3(WAVES * 64), lds, s, b);
    return hipGetLastError();
}

// The split launch of a batch of f32 sequences (one query row each, every sequence a shape
// f32_decode_kernel_serves accepts, one geometry; the wavefront count of the first sequence
// serves all, as in the bf16 batch launch); the caller merges.
hipError_t launch_f32_split_batch(const DecodeBatchArgs &b, int n_seq, int max_splits, hipStream_t s) {
    const DecodeArgs &a0 = b.seq[0];
    for (int i = 0; i < n_seq; ++i)
        if (!f32_decode_kernel_serves(b.seq[i]) || b.seq[i].pre) return hipErrorInvalidValue;
    const bool w8 = a0.waves == 8;
    switch (a0.g.P) {
    case 32: return w8 ? launch_f32_batch<32, 8>(b, n_seq, max_splits, s) : launch_f32_batch<32, 4>(b, n_seq, max_splits, s);
    case 64: return w8 ? launch_f32_batch<64, 8>(b, n_seq, max_splits, s) : launch_f32_batch<64, 4>(b, n_seq, max_splits, s);
    case 128: return w8 ? launch_f32_batch<128, 8>(b, n_seq, max_splits, s) : launch_f32_batch<128, 4>(b, n_seq, max_splits, s);
    case 256: return w8 ? launch_f32_batch<256, 8>(b, n_seq, max_splits, s) : launch_f32_batch<256, 4>(b, n_seq, max_splits, s);
    default: return hipErrorInvalidValue;
    }
}

// One query row of up to 16 heads per group, head_dim up to 256: the decode kernel (which
// also appends); chunks and wider heads take f32_split_kernel.
bool f32_decode_kernel_serves(const DecodeArgs &a) {
    return a.n_queries == 1 && a.g.gqa <= 16 && a.g.P <= 256 && (a.waves == 4 || a.waves == 8);
}

} // namespace skv
