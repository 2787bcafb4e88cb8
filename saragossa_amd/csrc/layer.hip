// Host side of one layer's paged KV cache: the stand-in for FullAttentionMetalState
// (src/decode_resident/attention.rs:457-1038). All bookkeeping (len, block table)
// lives on the host and advances at call time, before the GPU has run the work,
// exactly like the reference's encode-time `len += 1` (attention.rs:993).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <new>
#include <string>
#include <vector>

#include "layer.h"

namespace skv {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }
int32_t fail(int32_t code, const std::string &msg) {
    g_last_error = msg;
    return code;
}
int32_t fail_hip(hipError_t e, const char *what) {
    g_last_error = std::string("HIP: ") + hipGetErrorString(e) + " (" + what + ")";
    return SKV_ERR_DEVICE;
}

hipError_t arena_get(skv_ctx *ctx, size_t bytes, void **ptr, size_t *got) {
    *ptr = nullptr;
    *got = 0;
    if (bytes == 0) bytes = 256;
    {
        std::lock_guard<std::mutex> lk(ctx->arena_mu);
        auto it = ctx->arena_free.lower_bound(bytes);
        if (it != ctx->arena_free.end() && it->first <= bytes + bytes / 4) {
            *ptr = it->second;
            *got = it->first;
            ctx->arena_bytes -= it->first;
            ctx->arena_free.erase(it);
            return hipSuccess;
        }
    }
    const hipError_t e = hipMalloc(ptr, bytes);
    if (e == hipSuccess) *got = bytes;
    return e;
}

void arena_put(skv_ctx *ctx, void *ptr, size_t bytes) {
    if (!ptr) return;
    {
        std::lock_guard<std::mutex> lk(ctx->arena_mu);
        if (!ctx->closed && ctx->arena_bytes + bytes <= ctx->arena_cap) {
            ctx->arena_free.emplace(bytes, ptr);
            ctx->arena_bytes += bytes;
            return;
        }
    }
    (void)hipFree(ptr);
}

// Frees what the context holds on the device; the caller has synchronised the device.
static void ctx_drain(skv_ctx *ctx) {
    std::lock_guard<std::mutex> lk(ctx->arena_mu);
    for (auto &kv : ctx->mq_scratch)
        if (kv.second.ptr) (void)hipFree(kv.second.ptr);
    ctx->mq_scratch.clear();
    for (auto &kv : ctx->arena_free) (void)hipFree(kv.second);
    ctx->arena_free.clear();
    ctx->arena_bytes = 0;
}

void ctx_release(skv_ctx *ctx) {
    if (ctx->refs.fetch_sub(1, std::memory_order_acq_rel) != 1) return;
    // a layer that outlived skv_ctx_destroy may have grown the multi-query scratch again
    if (!ctx->mq_scratch.empty()) {
        (void)hipSetDevice(ctx->device);
        (void)hipDeviceSynchronize();
        ctx_drain(ctx);
    }
    delete ctx;
}

} // namespace skv

using namespace skv;

// Split-K partials of skv_decode_step_static_device, for callers that cannot allocate. Every
// GPU the library runs on holds its own copy of the array until the process ends. In host
// code the array's name is only a stand-in: its device address comes from
// hipGetSymbolAddress, once per device (static_scratch_ptr), and only that pointer is ever
// handed to a kernel.
static __device__ __align__(256) unsigned char scratch[SKV_STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[MAX_DEVICES] = {};

// The device address of `scratch` on `device`, which must be the current device.
hipError_t static_scratch_ptr(int device, void **ptr) {
    *ptr = nullptr;
    if (device < 0 || device >= MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[device] = p;
    }
    *ptr = g_scratch_ptr[device];
    return hipSuccess;
}

int padded_head_dim(size_t hd) {
    for (int p : {32, 64, 128, 256, 512})
        if ((size_t)p >= hd) return p;
    return 0;
}

size_t env_usize(const char *name, size_t dflt) {
    const char *raw = std::getenv(name);
    if (!raw || !*raw) return dflt;
    char *end = nullptr;
    unsigned long long v = std::strtoull(raw, &end, 10);
    if (end == raw) return dflt;
    return (size_t)v;
}

// Launch-shaping knobs from the environment, read once per flag generation
// (skv_flags_reload starts a new one), not once per launch.
struct Tuning {
    size_t split_min_len;   // rows below which the context is not split
    size_t target_wgs;      // workgroups a decode launch aims for
    size_t min_pages;       // pages per split at least (0 = one per wavefront)
    size_t forced_waves;    // 4 or 8, 0 = by shape
    bool q_vec, fused_append, prefill_tiles;
    size_t prefill_wgs, prefill_max_splits;
    long prefill_tiles2_min_pages; // -1 = by head_dim
};

const Tuning &tuning() {
    thread_local Tuning t{};
    thread_local uint64_t seen = 0;
    const uint64_t epoch = skv_internal_flags_epoch();
    if (epoch != seen) {
        t.split_min_len = skv_effective_split_min_len();
        t.target_wgs = std::max<size_t>(env_usize("SKV_DECODE_WGS", 256), 1);
        t.min_pages = env_usize("SKV_DECODE_MIN_PAGES", 0);
        t.forced_waves = env_usize("SKV_DECODE_WAVES", 0);
        t.q_vec = env_usize("SKV_Q_VEC", 1) != 0;
        t.fused_append = env_usize("SKV_FUSED_APPEND", 1) != 0;
        t.prefill_tiles = env_usize("SKV_PREFILL_TILES", 1) != 0;
        t.prefill_wgs = std::max<size_t>(env_usize("SKV_PREFILL_WGS", 256), 1);
        t.prefill_max_splits = std::max<size_t>(env_usize("SKV_PREFILL_MAX_SPLITS", 512), 1);
        t.prefill_tiles2_min_pages = std::getenv("SKV_PREFILL_TILES2_MIN_PAGES")
                                         ? (long)env_usize("SKV_PREFILL_TILES2_MIN_PAGES", 0) : -1;
        seen = epoch;
    }
    return t;
}

// Wavefronts per workgroup of the split kernel. Eight halve the number of partials for the
// same number of wavefronts in flight; four are better when eight would leave three
// quarters of the compute units without a workgroup (short contexts, ring layers).
int choose_waves(const skv_layer *L, int n_pages_scan) {
    if (L->g.P > 256) return 4; // one wavefront per SIMD: 512 registers each
    const size_t forced = tuning().forced_waves;
    if (forced == 4 || forced == 8) return (int)forced;
    const size_t kvh = (size_t)L->g.kv_heads;
    const size_t wgs8 = kvh * std::max<size_t>(std::min<size_t>(256 / std::max<size_t>(kvh, 1), (size_t)n_pages_scan / 8), 1);
    return wgs8 <= 64 && n_pages_scan >= 8 ? 4 : 8;
}

size_t decode_target_wgs() { return tuning().target_wgs; }

// Two 16-slot query tiles per wavefront in the prefill tile kernel halve the LDS reads and
// barriers per product but also the number of workgroups. Measured with 512-row chunks: at
// head_dim 128 they win from about 256 pages of context on (+15 % at 16k-32k rows, -4..-20 %
// under 2k rows), at head_dim 64 from about 512 pages (+10 % at 32k rows, -10..-20 % under 4k);
// at 256 the registers do not allow them.
bool prefill_two_tiles(const Geom &g, int n_pages_scan) {
    if (!prefill_two_tiles_possible(g.P)) return false;
    const long knob = tuning().prefill_tiles2_min_pages;
    const long min_pages = knob >= 0 ? knob : (g.P <= 64 ? 512 : 256);
    return (long)n_pages_scan >= min_pages;
}

int choose_splits(const skv_layer *L, int n_pages_scan, size_t rows, int waves, size_t target_wgs) {
    const Tuning &t = tuning();
    if (!skv_flag_sdpa_2pass_enabled() || rows < t.split_min_len) return 1;
    const size_t min_pages = std::max<size_t>(t.min_pages ? t.min_pages : (size_t)waves, 1);
    size_t s = std::max<size_t>(target_wgs / (size_t)L->g.kv_heads, 1);
    // Short contexts: as many splits as leave no split more than min_pages pages (rounded up,
    // not down: with one page per wavefront no wavefront then walks a second page, which
    // would be a whole memory latency more for the launch).
    s = std::min<size_t>(s, ((size_t)n_pages_scan + min_pages - 1) / min_pages);
    s = std::min<size_t>(s, (size_t)L->max_splits);
    return (int)std::max<size_t>(s, 1);
}

hipStream_t as_stream(skv_stream s) { return reinterpret_cast<hipStream_t>(s); }

int32_t check_window(const skv_layer *L, size_t window_start) {
    if (L->len == 0) return fail(SKV_ERR_DIMENSION, "attention_decode sur KV vide");
    if (window_start >= L->len)
        return fail(SKV_ERR_DIMENSION, "attention_decode fenêtre vide: début=" +
                                           std::to_string(window_start) +
                                           ", len=" + std::to_string(L->len));
    if (L->g.ring_rows > 0 && window_start < L->floor_pos)
        return fail(SKV_ERR_DIMENSION,
                    "attention_decode: fenêtre début=" + std::to_string(window_start) +
                        " avant la plus ancienne ligne conservée " + std::to_string(L->floor_pos));
    return SKV_OK;
}

bool uses_flash(const skv_layer *L) { return skv_flag_flash_sdpa_enabled() && L->g.P <= 512; }
// The attention launch of a decode step can append the row itself: always on bf16 layers,
// on f32 layers where the f32 decode kernel serves the shape (head_dim up to 256, at most 16
// heads per group).
bool fused_append_built(const skv_layer *L) { return !L->g.f32 || (L->g.P <= 256 && L->g.gqa <= 16); }
// The fused pre-KV step is built for bf16 layers up to head_dim 512 and for f32 layers up to
// head_dim 256; wide f32 heads take the separate norm/rotation launches.
bool wide_f32_heads(const skv_layer *L) { return L->g.f32 && L->g.P > 256; }

// Arguments of the matrix-core attention kernel for the layer's current length.
void fill_decode_args(const skv_layer *L, const float *q_dev, float *out_dev, size_t window_start,
                      const float *k_new, const float *v_new, size_t n_queries, size_t target_wgs,
                      DecodeArgs &a) {
    const Geom &g = L->g;
    a.q = q_dev;
    a.out = out_dev;
    a.k_pool = L->k_pool;
    a.v_pool = L->v_pool;
    a.table = L->table_dev;
    a.part_o = L->part_o;
    a.part_m = L->part_m;
    a.part_l = L->part_l;
    a.len = (int)L->len;
    a.n_queries = (int)n_queries;
    a.q_pos0 = (int)(L->len - n_queries); // the queries are the last n_queries rows
    a.limit_cap = INT32_MAX;
    a.split_base = 0;
    a.window = n_queries > 1 ? (int)L->window : 0; // decode callers pass window_start themselves
    a.window_start = (int)window_start;
    if (g.ring_rows > 0) {
        a.page_first = 0;
        a.n_pages = (int)std::min<size_t>((L->len + 15) / 16, (size_t)L->n_pages);
        a.ring_t = (int)((L->len - 1) % (size_t)g.ring_rows);
        a.ring_base = (int)(L->len - 1) - a.ring_t;
    } else {
        a.page_first = (int)(window_start / 16);
        a.n_pages = (int)((L->len + 15) / 16) - a.page_first;
    }
    a.waves = choose_waves(L, a.n_pages);
    a.splits = choose_splits(L, a.n_pages, L->len - window_start, a.waves, target_wgs);
    a.splits_total = a.splits;
    // scores are multiplied by 1/sqrt(head_dim) (src/decode_resident/kernels.rs:36, 198, 395,
    // 575); log2(e) moves the softmax to base 2.
    a.qscale = (1.0f / std::sqrt((float)g.head_dim)) * 1.4426950408889634f;
    a.k_new = k_new;
    a.v_new = v_new;
    a.new_slot = (int)slot_of((long)L->len - 1, g.ring_rows);
    a.new_page = L->table[(size_t)(a.new_slot >> 4)];
    a.q_vec = (tuning().q_vec && (reinterpret_cast<uintptr_t>(q_dev) & 15) == 0 && (g.head_dim & 7) == 0) ? 1 : 0;
    a.g = g;
}

// Split partials of a multi-query launch live in the context's scratch, grown on demand:
// [kv_heads][n_sets][n_queries * gqa] of (o[head_dim], m, l).
int32_t multi_query_partials(skv_layer *L, hipStream_t s, size_t n_sets, size_t n_queries, DecodeArgs &a) {
    const Geom &g = L->g;
    const size_t n_part = (size_t)g.kv_heads * n_sets * n_queries * g.gqa;
    const size_t need = n_part * ((size_t)g.head_dim + 2) * sizeof(float);
    skv_ctx *c = L->ctx;
    void *buf = nullptr;
    void *old = nullptr;     // this stream's buffer, too small: freed once the stream has drained
    void *evicted = nullptr; // another stream's buffer, pushed out of the bounded map
    {
        std::lock_guard<std::mutex> lk(c->arena_mu);
        auto it = c->mq_scratch.find(s);
        if (it != c->mq_scratch.end() && it->second.bytes >= need) {
            it->second.used = ++c->mq_clock;
            buf = it->second.ptr;
        } else if (it != c->mq_scratch.end()) {
            old = it->second.ptr;
            c->mq_scratch.erase(it); // nobody else uses this stream's entry (one thread per stream)
        } else if (c->mq_scratch.size() >= skv_ctx::MQ_SCRATCH_STREAMS) {
            auto lru = c->mq_scratch.begin();
            for (auto j = c->mq_scratch.begin(); j != c->mq_scratch.end(); ++j)
                if (j->second.used < lru->second.used) lru = j;
            evicted = lru->second.ptr;
            c->mq_scratch.erase(lru);
        }
    }
    if (!buf) {
        // waits, frees and the allocation outside the lock: other threads' arena_get / arena_put
        // and launches on other streams go on meanwhile
        if (old) {
            SKV_HIP(hipStreamSynchronize(s)); // work queued on the stream may still read it
            SKV_HIP(hipFree(old));
        }
        if (evicted) {
            SKV_HIP(hipDeviceSynchronize()); // its stream may be gone: wait for everything
            SKV_HIP(hipFree(evicted));
        }
        void *p = nullptr;
        SKV_HIP(hipMalloc(&p, need));
        std::lock_guard<std::mutex> lk(c->arena_mu);
        skv_ctx::MqScratch &slot = c->mq_scratch[s];
        slot.ptr = p;
        slot.bytes = need;
        slot.used = ++c->mq_clock;
        buf = p;
    }
    a.part_o = reinterpret_cast<float *>(buf);
    a.part_m = a.part_o + n_part * g.head_dim;
    a.part_l = a.part_m + n_part;
    return SKV_OK;
}

// k_new / v_new non-null: the row at position len-1 has not been written yet and the
// attention kernel appends it itself (the host bookkeeping has already advanced).
// n_queries > 1: chunked prefill over the cache; the last n_queries rows are the new ones
// and query i attends positions up to len - n_queries + i, each through the layer's
// sliding window. The matrix-core kernel only.
// attn_scalar > 0 replaces head_dim under the square root of the score scale
// (encode_query_attention_scale, src/decode_resident/layers.rs:7-33); pre non-null asks the
// kernel to norm and rotate q and the new k row itself.
struct PreKv {
    const float *rope;
    const float *q_norm_w;
    const float *k_norm_w;
    float eps;
    int rope_dims;
    int rope_style;
    const float *gate;  // multiplied into the context through a sigmoid (null = none)
    int q_head_stride;  // elements between the heads of q and of gate (0 = head_dim)
};

// Points the launch's split partials at `buf` instead of the layer's own buffers
// (decode, one query row): [kv_heads][splits][gqa] of (o[head_dim], m, l).
int32_t partials_in(void *buf, size_t buf_bytes, DecodeArgs &a) {
    const Geom &g = a.g;
    const size_t n_part = (size_t)g.kv_heads * (size_t)a.splits_total * (size_t)g.gqa * (size_t)a.n_queries;
    const size_t need = n_part * ((size_t)g.head_dim + 2) * sizeof(float);
    if (need > buf_bytes)
        return fail(SKV_ERR_DIMENSION, "decode_step_static: partiels split-K de " + std::to_string(need) +
                                           " o > tampon statique de " + std::to_string(buf_bytes) + " o");
    a.part_o = reinterpret_cast<float *>(buf);
    a.part_m = a.part_o + n_part * g.head_dim;
    a.part_l = a.part_m + n_part;
    return SKV_OK;
}

int32_t encode_attention(skv_layer *L, hipStream_t s, const float *q_dev, float *out_dev,
                         size_t window_start, const float *k_new = nullptr,
                         const float *v_new = nullptr, size_t n_queries = 1,
                         float attn_scalar = 0.0f, const PreKv *pre = nullptr,
                         void *static_partials = nullptr) {
    int32_t rc = check_window(L, window_start);
    if (rc) return rc;
    const Geom &g = L->g;
    if (static_partials && (n_queries != 1 || !uses_flash(L)))
        return fail(SKV_ERR_CONFIG, "decode_step_static: une ligne de requête, noyau matriciel seulement");
    if (g.f32 && (uses_flash(L) || n_queries > 1)) {
        // the f32 element's matrix kernels: 16 query slots per workgroup, the context split while
        // that leaves compute units idle; one query row of narrow heads takes the kernel that
        // can append the row (and norm and rotate q and k) itself
        DecodeArgs a{};
        fill_decode_args(L, q_dev, out_dev, window_start, k_new, v_new, n_queries, decode_target_wgs(), a);
        if ((k_new || v_new || pre) && !f32_decode_kernel_serves(a))
            return fail(SKV_ERR_CONFIG, "KV f32: étape fusionnée non construite pour cette forme");
        if (pre) {
            a.pre = 1;
            a.rope = pre->rope;
            a.q_norm_w = pre->q_norm_w;
            a.k_norm_w = pre->k_norm_w;
            a.eps = pre->eps;
            a.rope_dims = pre->rope ? pre->rope_dims : 0;
            a.rope_style = pre->rope_style;
            a.gate = pre->gate;
            a.q_head_stride = pre->q_head_stride;
        }
        if (attn_scalar > 0.0f) a.qscale = (1.0f / std::sqrt(attn_scalar)) * 1.4426950408889634f;
        if (n_queries > 1) {
            const size_t tiles = (n_queries * (size_t)g.gqa + 15) / 16 * (size_t)g.kv_heads;
            const size_t want = std::max<size_t>(2 * decode_target_wgs() / tiles, 1);
            a.splits = (int)std::min<size_t>((size_t)a.splits, want);
            a.splits_total = a.splits;
            if (a.splits > 1) {
                int32_t rc2 = multi_query_partials(L, s, (size_t)a.splits, n_queries, a);
                if (rc2) return rc2;
            }
        }
        if (static_partials && a.splits > 1) {
            int32_t rc2 = partials_in(static_partials, SKV_STATIC_SCRATCH_BYTES, a);
            if (rc2) return rc2;
        }
        SKV_HIP(launch_f32_split(a, s));
        if (a.splits > 1) SKV_HIP(n_queries > 1 ? launch_merge_rows(a, s) : launch_merge(a, s));
        return SKV_OK;
    }
    const bool use_flash = uses_flash(L) || n_queries > 1;
    if (!use_flash) {
        const size_t need = (size_t)g.q_heads * L->capacity;
        if (L->scores_cap < need) {
            if (L->scores) {
                SKV_HIP(hipDeviceSynchronize());
                SKV_HIP(hipFree(L->scores));
                L->scores = nullptr;
                L->scores_cap = 0;
            }
            SKV_HIP(hipMalloc(&L->scores, need * sizeof(float)));
            L->scores_cap = need;
        }
        NaiveArgs a{};
        a.q = q_dev;
        a.out = out_dev;
        a.k_pool = L->k_pool;
        a.v_pool = L->v_pool;
        a.table = L->table_dev;
        a.scores = L->scores;
        a.len = (long)L->len;
        a.window_start = (long)window_start;
        a.inv_scale = 1.0f / std::sqrt(attn_scalar > 0.0f ? attn_scalar : (float)g.head_dim);
        a.g = g;
        SKV_HIP(launch_naive(a, s));
        return SKV_OK;
    }
    DecodeArgs a{};
    fill_decode_args(L, q_dev, out_dev, window_start, k_new, v_new, n_queries, decode_target_wgs(), a);
    if (attn_scalar > 0.0f) a.qscale = (1.0f / std::sqrt(attn_scalar)) * 1.4426950408889634f;
    if (pre) {
        a.pre = 1;
        a.rope = pre->rope;
        a.q_norm_w = pre->q_norm_w;
        a.k_norm_w = pre->k_norm_w;
        a.eps = pre->eps;
        a.rope_dims = pre->rope ? pre->rope_dims : 0;
        a.rope_style = pre->rope_style;
        a.gate = pre->gate;
        a.q_head_stride = pre->q_head_stride;
    }
    // Chunks of at least 64 query slots take the kernel that shares each K/V page among 128
    // or 256 slots through LDS; shorter ones (speculative verify rows) the decode kernel's
    // multi-query mode, one workgroup per 16 slots.
    const bool use_tiles = tuning().prefill_tiles && n_queries > 1 && n_queries * (size_t)g.gqa >= 64;
    if (n_queries > 1) {
        // split the context only while the query tiles alone leave compute units idle, and
        // keep the partials in the context's scratch
        a.tiles2 = use_tiles && prefill_two_tiles(g, a.n_pages) ? 1 : 0;
        const size_t per_wg = use_tiles ? (size_t)prefill_tile_slots(g.P, a.tiles2 != 0) : 16;
        const size_t tiles = (n_queries * (size_t)g.gqa + per_wg - 1) / per_wg * (size_t)g.kv_heads;
        size_t want = std::max<size_t>((use_tiles ? tuning().prefill_wgs : 256) / tiles, 1);
        if (use_tiles) {
            want = std::min<size_t>(want, std::max<size_t>((size_t)a.n_pages / 16, 1));
            want = std::min<size_t>(want, tuning().prefill_max_splits);
        }
        a.splits = (int)std::min<size_t>((size_t)a.splits, want);
        a.splits_total = a.splits;
        if (a.splits > 1) {
            int32_t rc2 = multi_query_partials(L, s, (size_t)a.splits, n_queries, a);
            if (rc2) return rc2;
        }
    }
    if (static_partials && a.splits_total > 1) {
        int32_t rc2 = partials_in(static_partials, SKV_STATIC_SCRATCH_BYTES, a);
        if (rc2) return rc2;
    }
    if (use_tiles) {
        SKV_HIP(launch_prefill_tiles(a, s));
        if (a.splits > 1) SKV_HIP(launch_merge_rows(a, s));
        return SKV_OK;
    }
    SKV_HIP(launch_decode(a, s));
    return SKV_OK;
}

int32_t encode_append(skv_layer *L, hipStream_t s, const float *k_dev, const float *v_dev,
                      size_t n_rows) {
    if (n_rows == 0) return SKV_OK;
    if (L->len + n_rows > L->capacity)
        return fail(SKV_ERR_DIMENSION, "append KV résident: capacité " +
                                           std::to_string(L->capacity) + " atteinte (overflow)");
    AppendArgs a{};
    a.k_src = k_dev;
    a.v_src = v_dev;
    a.k_pool = L->k_pool;
    a.v_pool = L->v_pool;
    a.table = L->table_dev;
    a.first_pos = (long)L->len;
    a.n_rows = (int)n_rows;
    a.g = L->g;
    if (L->g.ring_rows > 0 && n_rows > (size_t)L->g.ring_rows) {
        // only the last ring_rows rows survive; skip the ones that would be overwritten
        const size_t skip = n_rows - (size_t)L->g.ring_rows;
        const size_t kv_dim = (size_t)L->g.kv_heads * L->g.head_dim;
        a.k_src += skip * kv_dim;
        a.v_src += skip * kv_dim;
        a.first_pos += (long)skip;
        a.n_rows = L->g.ring_rows;
    }
    if (L->g.f32) {
        SKV_HIP(launch_append_f32(a, s));
        L->len += n_rows;
        if (L->g.ring_rows > 0 && L->len > (size_t)L->g.ring_rows)
            L->floor_pos = std::max(L->floor_pos, L->len - (size_t)L->g.ring_rows);
        return SKV_OK;
    }
    // whole groups of four rows at positions that are multiples of 4 write V in 16-byte units
    if (a.n_rows >= 8) {
        a.by_page = 1;
        const long lead = (4 - (a.first_pos & 3)) & 3;
        a.v_grp_first = (int)lead;
        a.v_grp_rows = (int)((a.n_rows - lead) & ~3L);
    }
    SKV_HIP(launch_append(a, s));
    L->len += n_rows;
    if (L->g.ring_rows > 0 && L->len > (size_t)L->g.ring_rows)
        L->floor_pos = std::max(L->floor_pos, L->len - (size_t)L->g.ring_rows);
    return SKV_OK;
}

} // namespace

extern "C" {

const char *skv_last_error(void) { return g_last_error.c_str(); }
int32_t skv_abi_version(void) { return 1; }

int32_t skv_ctx_create(int32_t device, skv_ctx **out) try {
    if (!out) return fail(SKV_ERR_DEVICE, "skv_ctx_create: out nul");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(SKV_ERR_DEVICE, "aucun GPU HIP disponible (le chemin KV gfx950 exige un MI355X)");
    if (device < 0 || device >= count)
        return fail(SKV_ERR_CONFIG, "device " + std::to_string(device) + " hors plage");
    SKV_HIP(hipSetDevice(device));
    // The synchronous host entry points run on the legacy default stream, which
    // orders itself against every blocking stream of the process (a framework's
    // default stream included), so a host call that follows device-side calls on
    // such a stream sees their effect without an explicit wait.
    // the library's set-up call on this device: the address of the static scratch array here
    void *static_scratch = nullptr;
    SKV_HIP(static_scratch_ptr(device, &static_scratch));
    skv_ctx *c = new skv_ctx();
    c->device = device;
    c->stream = nullptr;
    c->static_scratch = static_scratch;
    c->arena_cap = env_usize("SKV_ARENA_MAX_MB", 4096) << 20;
    *out = c;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

void skv_ctx_destroy(skv_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipDeviceSynchronize();
    {
        std::lock_guard<std::mutex> lk(ctx->arena_mu);
        ctx->closed = true;
    }
    ctx_drain(ctx);
    ctx_release(ctx);
}

int32_t skv_ctx_synchronize(skv_ctx *ctx) try {
    if (!ctx) return fail(SKV_ERR_DEVICE, "ctx nul");
    SKV_HIP(hipSetDevice(ctx->device));
    SKV_HIP(hipDeviceSynchronize());
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

void skv_layer_destroy(skv_layer *L) {
    if (!L) return;
    (void)hipSetDevice(L->ctx->device);
    (void)hipDeviceSynchronize();
    for (auto &b : L->leased) arena_put(L->ctx, b.first, b.second);
    if (L->scores) (void)hipFree(L->scores);
    delete L;
}

// Shape checks of full_attention_with_element (src/decode_resident/attention.rs:56-108) and
// the geometry, page count and buffer sizes that follow from them; shared by the factory and
// by skv_layer_bytes so that the budget figure is the factory's own arithmetic.
struct LayerPlan {
    Geom g{};
    int n_pages = 0;
    int max_splits = 1;
    size_t pool_bytes = 0, table_bytes = 0, part_o_bytes = 0, part_ml_bytes = 0, q_bytes = 0, kv_stage_bytes = 0;
    size_t total() const {
        // every buffer is its own allocation, rounded up by the allocator to 256 bytes at least
        auto r = [](size_t b) { return (std::max<size_t>(b, 256) + 255) / 256 * 256; };
        return 2 * r(pool_bytes) + r(table_bytes) + r(part_o_bytes) + 2 * r(part_ml_bytes) + 2 * r(q_bytes) +
               r(kv_stage_bytes);
    }
};

// rollback_rows: rows a ring layer keeps behind its window (SIZE_MAX = the default: the
// environment's SKV_RING_SLACK_ROWS, else 32)
static int32_t plan_layer(size_t capacity, size_t q_heads, size_t kv_heads, size_t head_dim, int32_t dtype,
                          size_t window, size_t rollback_rows, LayerPlan &p) {
    if (capacity == 0 || q_heads == 0 || kv_heads == 0 || head_dim == 0)
        return fail(SKV_ERR_CONFIG, "FullAttentionMetalState: dimension nulle");
    if (q_heads % kv_heads != 0)
        return fail(SKV_ERR_CONFIG, "GQA invalide: q_heads=" + std::to_string(q_heads) +
                                        " non multiple de kv_heads=" + std::to_string(kv_heads));
    if (dtype != SKV_DTYPE_BF16 && dtype != SKV_DTYPE_F32)
        return fail(SKV_ERR_CONFIG, "élément KV inconnu: " + std::to_string(dtype));
    const bool f32 = dtype == SKV_DTYPE_F32;
    const int P = padded_head_dim(head_dim);
    if (P == 0) return fail(SKV_ERR_CONFIG, "head_dim > 512 non supporté");
    if (capacity > (size_t)1 << 30 || q_heads > 4096 || kv_heads > 4096 || window > (size_t)1 << 30 ||
        (rollback_rows != SIZE_MAX && rollback_rows > (size_t)1 << 30))
        return fail(SKV_ERR_CONFIG, "capacité KV déborde");
    Geom &g = p.g;
    g.q_heads = (int)q_heads;
    g.kv_heads = (int)kv_heads;
    g.head_dim = (int)head_dim;
    g.P = P;
    g.gqa = (int)(q_heads / kv_heads);
    g.f32 = f32 ? 1 : 0;
    g.tile_elems = P * 16 * (f32 ? 2 : 1);
    g.page_elems = (int)kv_heads * g.tile_elems;
    size_t rows = capacity;
    if (window > 0) {
        // The ring keeps the window plus some rows behind it, so that the rows a speculative
        // verify appended can be rolled back (truncate) without the ring having overwritten
        // what the next query attends: the reference keeps the whole cache and rolls back
        // freely (src/decoder/attention_cache.rs:72-100). A ring never needs more rows than
        // the capacity.
        const size_t slack = rollback_rows != SIZE_MAX ? rollback_rows : env_usize("SKV_RING_SLACK_ROWS", 32);
        size_t ring = (window + slack + 15) / 16 * 16;
        ring = std::min(ring, (capacity + 15) / 16 * 16);
        g.ring_rows = (int)ring;
        rows = ring;
    }
    p.n_pages = (int)((rows + 15) / 16);
    p.pool_bytes = (size_t)p.n_pages * g.page_elems * sizeof(uint16_t);
    p.max_splits = std::min(decode_max_splits(), std::max(1, p.n_pages));
    const size_t n_part = (size_t)kv_heads * p.max_splits * g.gqa;
    p.table_bytes = (size_t)p.n_pages * sizeof(int32_t);
    p.part_o_bytes = n_part * head_dim * sizeof(float);
    p.part_ml_bytes = n_part * sizeof(float);
    p.q_bytes = q_heads * head_dim * sizeof(float);
    p.kv_stage_bytes = 2 * kv_heads * head_dim * sizeof(float);
    return SKV_OK;
}

int32_t skv_layer_bytes(size_t capacity, size_t q_heads, size_t kv_heads, size_t head_dim, int32_t dtype,
                        size_t window, uint64_t *bytes) try {
    if (!bytes) return fail(SKV_ERR_DEVICE, "skv_layer_bytes: pointeur nul");
    LayerPlan p;
    int32_t rc = plan_layer(capacity, q_heads, kv_heads, head_dim, dtype, window, SIZE_MAX, p);
    if (rc) return rc;
    *bytes = (uint64_t)p.total();
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_check_allocation(skv_ctx *ctx, uint64_t requested, uint64_t static_cap, uint64_t headroom,
                             uint64_t *available, uint64_t *projected) try {
    if (!ctx) return fail(SKV_ERR_DEVICE, "skv_check_allocation: ctx nul");
    SKV_HIP(hipSetDevice(ctx->device));
    size_t free_b = 0, total_b = 0;
    SKV_HIP(hipMemGetInfo(&free_b, &total_b));
    // effective_limit: the smallest of the caps that are set (src/memory_guard.rs:109-127); the
    // device's memory minus the headroom stands where the host's memory stands there
    uint64_t limit = (uint64_t)total_b > headroom ? (uint64_t)total_b - headroom : 0;
    if (static_cap) limit = std::min(limit, static_cap);
    // what the context's arena holds is free for the next layers of the same context
    uint64_t held = 0;
    {
        std::lock_guard<std::mutex> lk(ctx->arena_mu);
        held = ctx->arena_bytes;
    }
    const uint64_t used = (uint64_t)(total_b - free_b);
    const uint64_t current = used > held ? used - held : 0;
    uint64_t proj = 0, avail = 0;
    const int32_t over = skv_memory_projection(current, 0, requested, limit, &proj, &avail);
    if (available) *available = avail;
    if (projected) *projected = proj;
    if (over)
        return fail(SKV_ERR_MEMORY, "garde mémoire: demande " + std::to_string(requested) + " o, projection " +
                                        std::to_string(proj) + " o > plafond " + std::to_string(limit) +
                                        " o (disponible " + std::to_string(avail) + " o)");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_layer_create(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads,
                         size_t head_dim, int32_t dtype, size_t window, skv_layer **out) {
    return skv_layer_create_ring(ctx, capacity, q_heads, kv_heads, head_dim, dtype, window, SIZE_MAX, out);
}

int32_t skv_layer_bytes_ring(size_t capacity, size_t q_heads, size_t kv_heads, size_t head_dim, int32_t dtype,
                             size_t window, size_t rollback_rows, uint64_t *bytes) try {
    if (!bytes) return fail(SKV_ERR_DEVICE, "skv_layer_bytes: pointeur nul");
    LayerPlan p;
    int32_t rc = plan_layer(capacity, q_heads, kv_heads, head_dim, dtype, window, rollback_rows, p);
    if (rc) return rc;
    *bytes = (uint64_t)p.total();
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_layer_create_ring(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads, size_t head_dim,
                              int32_t dtype, size_t window, size_t rollback_rows, skv_layer **out) try {
    if (!ctx || !out) return fail(SKV_ERR_DEVICE, "skv_layer_create: pointeur nul");
    *out = nullptr;
    LayerPlan plan;
    {
        int32_t rc = plan_layer(capacity, q_heads, kv_heads, head_dim, dtype, window, rollback_rows, plan);
        if (rc) return rc;
    }
    SKV_HIP(hipSetDevice(ctx->device));

    skv_layer *L = new skv_layer();
    L->ctx = ctx;
    L->capacity = capacity;
    L->window = window;
    L->g = plan.g;
    const Geom &g = L->g;
    L->n_pages = plan.n_pages;
    const size_t pool_bytes = plan.pool_bytes;
    const size_t q_dim = q_heads * head_dim;
    const size_t kv_dim = kv_heads * head_dim;
    L->max_splits = plan.max_splits;
    const size_t n_part = (size_t)kv_heads * L->max_splits * g.gqa;

    hipError_t e = hipSuccess;
    auto alloc = [&](void **p, size_t bytes) {
        if (e != hipSuccess) return;
        size_t got = 0;
        e = arena_get(ctx, bytes, p, &got);
        if (e == hipSuccess) L->leased.emplace_back(*p, got);
    };
    alloc((void **)&L->k_pool, pool_bytes);
    alloc((void **)&L->v_pool, pool_bytes);
    alloc((void **)&L->table_dev, (size_t)L->n_pages * sizeof(int32_t));
    alloc((void **)&L->part_o, n_part * head_dim * sizeof(float));
    alloc((void **)&L->part_m, n_part * sizeof(float));
    alloc((void **)&L->part_l, n_part * sizeof(float));
    alloc((void **)&L->q_stage, q_dim * sizeof(float));
    alloc((void **)&L->out_stage, q_dim * sizeof(float));
    alloc((void **)&L->kv_stage, 2 * kv_dim * sizeof(float));
    // Padding dims and rows past `len` are multiplied by zero probabilities and zero
    // query padding; they must hold finite values, so the pools start at zero.
    if (e == hipSuccess) e = hipMemsetAsync(L->k_pool, 0, pool_bytes, ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(L->v_pool, 0, pool_bytes, ctx->stream);
    L->table.resize(L->n_pages);
    for (int i = 0; i < L->n_pages; ++i) L->table[i] = i;
    if (e == hipSuccess) e = launch_iota(L->table_dev, L->n_pages, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        skv_layer_destroy(L);
        return fail_hip(e, "allocation du cache KV");
    }
    *out = L;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_layer_create_for(skv_ctx *ctx, size_t capacity, size_t q_heads, size_t kv_heads,
                             size_t head_dim, int32_t sampled, skv_layer **out) try {
    const int32_t dtype = skv_flag_kv_bf16_for(sampled) ? SKV_DTYPE_BF16 : SKV_DTYPE_F32;
    return skv_layer_create(ctx, capacity, q_heads, kv_heads, head_dim, dtype, 0, out);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_layer_set_block_table(skv_layer *L, const int32_t *table, size_t n) try {
    if (!L || !table) return fail(SKV_ERR_DEVICE, "set_block_table: pointeur nul");
    if (L->len != 0) return fail(SKV_ERR_DIMENSION, "set_block_table: cache non vide");
    if (n != (size_t)L->n_pages)
        return fail(SKV_ERR_DIMENSION, "set_block_table: attendu " + std::to_string(L->n_pages) +
                                           " entrées, reçu " + std::to_string(n));
    std::vector<char> seen(n, 0);
    for (size_t i = 0; i < n; ++i) {
        if (table[i] < 0 || (size_t)table[i] >= n || seen[table[i]])
            return fail(SKV_ERR_DIMENSION, "set_block_table: pas une permutation");
        seen[table[i]] = 1;
    }
    SKV_HIP(hipSetDevice(L->ctx->device));
    L->table.assign(table, table + n);
    SKV_HIP(hipMemcpyAsync(L->table_dev, L->table.data(), n * sizeof(int32_t), hipMemcpyHostToDevice,
                           L->ctx->stream));
    SKV_HIP(hipStreamSynchronize(L->ctx->stream));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

size_t skv_layer_pages(const skv_layer *L) { return L ? (size_t)L->n_pages : 0; }
size_t skv_kv_dim(const skv_layer *L) { return L ? (size_t)L->g.kv_heads * L->g.head_dim : 0; }
size_t skv_len(const skv_layer *L) { return L ? L->len : 0; }
size_t skv_capacity(const skv_layer *L) { return L ? L->capacity : 0; }
size_t skv_q_heads(const skv_layer *L) { return L ? (size_t)L->g.q_heads : 0; }
size_t skv_kv_heads(const skv_layer *L) { return L ? (size_t)L->g.kv_heads : 0; }
size_t skv_head_dim(const skv_layer *L) { return L ? (size_t)L->g.head_dim : 0; }
size_t skv_window(const skv_layer *L) { return L ? L->window : 0; }
size_t skv_logical_byte_len(const skv_layer *L) {
    return L ? L->capacity * (size_t)L->g.kv_heads * L->g.head_dim * (L->g.f32 ? 4 : 2) : 0;
}

int32_t skv_truncate(skv_layer *L, size_t len) try {
    if (!L) return fail(SKV_ERR_DEVICE, "truncate: pointeur nul");
    if (len > L->capacity)
        return fail(SKV_ERR_DIMENSION, "truncate KV " + std::to_string(len) + " > capacité " +
                                           std::to_string(L->capacity));
    L->len = len;
    if (len == 0) L->floor_pos = 0;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_seed(skv_layer *L, const float *keys, const float *values, size_t n_elems,
                 size_t n_rows) try {
    if (!L) return fail(SKV_ERR_DEVICE, "seed: pointeur nul");
    if (n_rows > L->capacity)
        return fail(SKV_ERR_DIMENSION, "seed KV " + std::to_string(n_rows) + " > capacité " +
                                           std::to_string(L->capacity));
    const size_t kv_dim = skv_kv_dim(L);
    const size_t expected = n_rows * kv_dim;
    if (n_elems != expected)
        return fail(SKV_ERR_DIMENSION, "seed KV: attendu " + std::to_string(expected) + " (=" +
                                           std::to_string(n_rows) + "×" + std::to_string(kv_dim) +
                                           "), reçu " + std::to_string(n_elems));
    if (n_rows > 0 && (!keys || !values)) return fail(SKV_ERR_DEVICE, "seed: pointeur nul");
    SKV_HIP(hipSetDevice(L->ctx->device));
    L->len = 0;
    L->floor_pos = 0;
    if (n_rows == 0) return SKV_OK;
    hipStream_t s = L->ctx->stream;
    // RETI_RUST_KV_BF16_SIM_KONLY / _VONLY (src/decode_resident/attention.rs:573-585): on an
    // f32 cache the seed keeps K alone, or else V alone, at bf16 precision (still stored as f32)
    std::vector<float> rounded;
    if (L->g.f32 && (skv_flag_kv_bf16_sim_konly() || skv_flag_kv_bf16_sim_vonly())) {
        const bool k_only = skv_flag_kv_bf16_sim_konly() != 0; // K wins when both are set, as in the match
        const float *src = k_only ? keys : values;
        rounded.resize(expected);
        for (size_t i = 0; i < expected; ++i) {
            const uint32_t b = (uint32_t)skv_f32_to_bf16_bits(src[i]) << 16;
            std::memcpy(&rounded[i], &b, sizeof(float));
        }
        (k_only ? keys : values) = rounded.data();
    }
    float *stage = nullptr;
    SKV_HIP(hipMalloc((void **)&stage, 2 * expected * sizeof(float)));
    hipError_t e = hipMemcpyAsync(stage, keys, expected * sizeof(float), hipMemcpyHostToDevice, s);
    if (e == hipSuccess)
        e = hipMemcpyAsync(stage + expected, values, expected * sizeof(float), hipMemcpyHostToDevice, s);
    int32_t rc = SKV_OK;
    if (e == hipSuccess) rc = encode_append(L, s, stage, stage + expected, n_rows);
    hipError_t e2 = hipStreamSynchronize(s);
    (void)hipFree(stage);
    if (e != hipSuccess) return fail_hip(e, "seed: copie hôte→device");
    if (rc) return rc;
    if (e2 != hipSuccess) return fail_hip(e2, "seed: synchronisation");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_append_host(skv_layer *L, const float *key, const float *value, size_t n_elems) try {
    if (!L || !key || !value) return fail(SKV_ERR_DEVICE, "append: pointeur nul");
    const size_t kv_dim = skv_kv_dim(L);
    if (n_elems != kv_dim)
        return fail(SKV_ERR_DIMENSION, "append KV: attendu " + std::to_string(kv_dim) + ", reçu " +
                                           std::to_string(n_elems));
    if (L->len >= L->capacity)
        return fail(SKV_ERR_DIMENSION,
                    "append KV: capacité " + std::to_string(L->capacity) + " atteinte (overflow)");
    SKV_HIP(hipSetDevice(L->ctx->device));
    hipStream_t s = L->ctx->stream;
    SKV_HIP(hipMemcpyAsync(L->kv_stage, key, kv_dim * sizeof(float), hipMemcpyHostToDevice, s));
    SKV_HIP(hipMemcpyAsync(L->kv_stage + kv_dim, value, kv_dim * sizeof(float), hipMemcpyHostToDevice, s));
    int32_t rc = encode_append(L, s, L->kv_stage, L->kv_stage + kv_dim, 1);
    if (rc) return rc;
    SKV_HIP(hipStreamSynchronize(s));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_append_device(skv_layer *L, skv_stream stream, const void *k_dev, size_t k_off,
                          const void *v_dev, size_t v_off) try {
    if (!L || !k_dev || !v_dev) return fail(SKV_ERR_DEVICE, "append device: pointeur nul");
    if ((k_off | v_off) & 3) return fail(SKV_ERR_DIMENSION, "append device: offset non aligné f32");
    return encode_append(L, as_stream(stream),
                         reinterpret_cast<const float *>((const char *)k_dev + k_off),
                         reinterpret_cast<const float *>((const char *)v_dev + v_off), 1);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_append_batch_device(skv_layer *L, skv_stream stream, const void *k_dev,
                                const void *v_dev, size_t n_rows) try {
    if (!L || !k_dev || !v_dev) return fail(SKV_ERR_DEVICE, "append batch: pointeur nul");
    if (n_rows == 0) return fail(SKV_ERR_DIMENSION, "cache KV batch attend seq > 0");
    return encode_append(L, as_stream(stream), (const float *)k_dev, (const float *)v_dev, n_rows);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_attention_device(skv_layer *L, skv_stream stream, const float *q_dev, float *out_dev,
                             size_t window_start) try {
    if (!L || !q_dev || !out_dev) return fail(SKV_ERR_DEVICE, "attention device: pointeur nul");
    return encode_attention(L, as_stream(stream), q_dev, out_dev, window_start);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_attention_host(skv_layer *L, const float *q, size_t n_elems, size_t window_start,
                           float *out) try {
    if (!L || !q || !out) return fail(SKV_ERR_DEVICE, "attention: pointeur nul");
    if (L->len == 0) return fail(SKV_ERR_DIMENSION, "attention_decode sur KV vide");
    const size_t q_dim = (size_t)L->g.q_heads * L->g.head_dim;
    if (n_elems != q_dim)
        return fail(SKV_ERR_DIMENSION, "attention_decode: q attendu [" + std::to_string(q_dim) +
                                           "], reçu " + std::to_string(n_elems));
    SKV_HIP(hipSetDevice(L->ctx->device));
    hipStream_t s = L->ctx->stream;
    SKV_HIP(hipMemcpyAsync(L->q_stage, q, q_dim * sizeof(float), hipMemcpyHostToDevice, s));
    int32_t rc = encode_attention(L, s, L->q_stage, L->out_stage, window_start);
    if (rc) return rc;
    SKV_HIP(hipMemcpyAsync(out, L->out_stage, q_dim * sizeof(float), hipMemcpyDeviceToHost, s));
    SKV_HIP(hipStreamSynchronize(s));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_decode_step_device(skv_layer *L, skv_stream stream, const void *k_dev, size_t k_off,
                               const void *v_dev, size_t v_off, const float *q_dev,
                               float *out_dev) try {
    if (!L || !k_dev || !v_dev || !q_dev || !out_dev)
        return fail(SKV_ERR_DEVICE, "decode_step: pointeur nul");
    const bool fused = tuning().fused_append;
    if (!fused || !uses_flash(L) || !fused_append_built(L)) {
        int32_t rc = skv_append_device(L, stream, k_dev, k_off, v_dev, v_off);
        if (rc) return rc;
        const size_t ws = skv_window_start(L->len - 1, L->window);
        return skv_attention_device(L, stream, q_dev, out_dev, ws);
    }
    if ((k_off | v_off) & 3) return fail(SKV_ERR_DIMENSION, "append device: offset non aligné f32");
    if (L->len >= L->capacity)
        return fail(SKV_ERR_DIMENSION, "append KV résident: capacité " +
                                           std::to_string(L->capacity) + " atteinte (overflow)");
    // the attention kernel writes the row itself: advance the bookkeeping first
    const size_t floor_before = L->floor_pos;
    L->len += 1;
    if (L->g.ring_rows > 0 && L->len > (size_t)L->g.ring_rows)
        L->floor_pos = std::max(L->floor_pos, L->len - (size_t)L->g.ring_rows);
    const size_t ws = skv_window_start(L->len - 1, L->window);
    int32_t rc = encode_attention(L, as_stream(stream), q_dev, out_dev, ws,
                                  reinterpret_cast<const float *>((const char *)k_dev + k_off),
                                  reinterpret_cast<const float *>((const char *)v_dev + v_off));
    if (rc) {
        L->len -= 1;
        L->floor_pos = floor_before;
    }
    return rc;
} catch (...) {
    return skv::fail_exception();
}

// skv_decode_step_device with the split partials in the library's static device array
// instead of the layer's own buffers: nothing here allocates or frees.
int32_t skv_decode_step_static_device(skv_layer *L, skv_stream stream, const void *k_dev, size_t k_off,
                                      const void *v_dev, size_t v_off, const float *q_dev,
                                      float *out_dev) try {
    if (!L || !k_dev || !v_dev || !q_dev || !out_dev)
        return fail(SKV_ERR_DEVICE, "decode_step_static: pointeur nul");
    if (!uses_flash(L))
        return fail(SKV_ERR_CONFIG, "decode_step_static: le noyau simple (RETI_RUST_FLASH_SDPA=0) alloue son "
                                    "tampon de scores");
    void *part = L->ctx->static_scratch;
    if (!part) return fail(SKV_ERR_DEVICE, "decode_step_static: tampon statique non résolu");
    if ((k_off | v_off) & 3) return fail(SKV_ERR_DIMENSION, "append device: offset non aligné f32");
    const float *k = reinterpret_cast<const float *>((const char *)k_dev + k_off);
    const float *v = reinterpret_cast<const float *>((const char *)v_dev + v_off);
    hipStream_t s = as_stream(stream);
    if (!tuning().fused_append || !fused_append_built(L)) {
        // separate launches (wide f32 heads have no fused append); on a failure after the
        // append the row stays appended, as with skv_decode_step_device
        int32_t rc = encode_append(L, s, k, v, 1);
        if (rc) return rc;
        return encode_attention(L, s, q_dev, out_dev, skv_window_start(L->len - 1, L->window), nullptr,
                                nullptr, 1, 0.0f, nullptr, part);
    }
    if (L->len >= L->capacity)
        return fail(SKV_ERR_DIMENSION, "append KV résident: capacité " +
                                           std::to_string(L->capacity) + " atteinte (overflow)");
    const size_t floor_before = L->floor_pos;
    L->len += 1;
    if (L->g.ring_rows > 0 && L->len > (size_t)L->g.ring_rows)
        L->floor_pos = std::max(L->floor_pos, L->len - (size_t)L->g.ring_rows);
    int32_t rc = encode_attention(L, s, q_dev, out_dev, skv_window_start(L->len - 1, L->window), k, v, 1,
                                  0.0f, nullptr, part);
    if (rc) {
        L->len -= 1;
        L->floor_pos = floor_before;
    }
    return rc;
} catch (...) {
    return skv::fail_exception();
}

// A chunk of c > 1 rows on a ring layer. The ring holds exactly the window (rounded up to a
// page), so the chunk's own rows overwrite rows its first queries still attend. The chunk
// is therefore attended in two phases around the append: first every query over the rows
// already in the ring (capped at the last old position), then, once the chunk is appended,
// over the chunk's own rows (from its first position up to each query's own). Both phases
// leave (o, m, l) partials; one merge produces the context. c <= ring_rows.
static int32_t ring_chunk(skv_layer *L, hipStream_t s, const float *q, const float *k, const float *v,
                          size_t c, float *out) {
    const Geom &g = L->g;
    const size_t base = L->len;
    const bool two = !g.f32 && prefill_two_tiles(g, L->n_pages);
    const size_t per_wg = g.f32 ? 16 : (size_t)prefill_tile_slots(g.P, two);
    const size_t tiles = (c * (size_t)g.gqa + per_wg - 1) / per_wg * (size_t)g.kv_heads;
    auto launch_chunk = [&](const DecodeArgs &a) { return g.f32 ? launch_f32_split(a, s) : launch_prefill_tiles(a, s); };
    auto splits_for = [&](int n_pages) {
        size_t want = std::max<size_t>((g.f32 ? 2 : 1) * tuning().prefill_wgs / tiles, 1);
        want = std::min<size_t>(want, std::max<size_t>((size_t)n_pages / 8, 1));
        return (int)std::min<size_t>(want, tuning().prefill_max_splits);
    };
    DecodeArgs a1{}, a3{};
    int s1 = 0;
    if (base > 0) { // phase 1, prepared against the ring as it is now
        fill_decode_args(L, q, out, L->floor_pos, nullptr, nullptr, c, tuning().prefill_wgs, a1);
        a1.q_pos0 = (int)base;
        a1.limit_cap = (int)base - 1;
        a1.tiles2 = two ? 1 : 0;
        s1 = splits_for(a1.n_pages);
    }
    const int pages_after = (int)std::min<size_t>((base + c + 15) / 16, (size_t)L->n_pages);
    const int s3 = splits_for(pages_after);
    const int total = s1 + s3;
    if (base > 0) {
        a1.splits = s1;
        a1.split_base = 0;
        a1.splits_total = total;
        int32_t rc = multi_query_partials(L, s, (size_t)total, c, a1);
        if (rc) return rc;
        SKV_HIP(launch_chunk(a1));
    }
    int32_t rc = encode_append(L, s, k, v, c);
    if (rc) return rc;
    fill_decode_args(L, q, out, std::max(base, L->floor_pos), nullptr, nullptr, c, tuning().prefill_wgs, a3);
    a3.q_pos0 = (int)base;
    a3.tiles2 = two ? 1 : 0;
    a3.splits = s3;
    a3.split_base = s1;
    a3.splits_total = total;
    if (total > 1) {
        rc = multi_query_partials(L, s, (size_t)total, c, a3);
        if (rc) return rc;
    }
    SKV_HIP(launch_chunk(a3));
    if (total > 1) SKV_HIP(launch_merge_rows(a3, s));
    return SKV_OK;
}

int32_t skv_prefill_chunk_device(skv_layer *L, skv_stream stream, const float *q_dev,
                                 const void *k_dev, const void *v_dev, size_t n_rows,
                                 float *out_dev) try {
    if (!L || !q_dev || !k_dev || !v_dev || !out_dev)
        return fail(SKV_ERR_DEVICE, "prefill chunk: pointeur nul");
    if (n_rows == 0) return fail(SKV_ERR_DIMENSION, "attention batch cached shapes: seq == 0");
    if (L->len + n_rows > L->capacity)
        return fail(SKV_ERR_DIMENSION, "append KV résident: capacité " +
                                           std::to_string(L->capacity) + " atteinte (overflow)");
    const size_t kv_dim = skv_kv_dim(L), q_dim = (size_t)L->g.q_heads * L->g.head_dim;
    // Ring layers take the chunk in steps of at most the ring's rows (see ring_chunk).
    size_t step = std::min<size_t>(n_rows, 4096);
    if (L->g.ring_rows > 0) step = std::min(step, (size_t)L->g.ring_rows);
    const float *q = q_dev, *k = (const float *)k_dev, *v = (const float *)v_dev;
    float *out = out_dev;
    for (size_t done = 0; done < n_rows; done += step) {
        const size_t c = std::min(step, n_rows - done);
        int32_t rc;
        if (L->g.ring_rows > 0 && c > 1) {
            rc = ring_chunk(L, as_stream(stream), q, k, v, c, out);
            if (rc) return rc;
            q += c * q_dim;
            k += c * kv_dim;
            v += c * kv_dim;
            out += c * q_dim;
            continue;
        }
        rc = encode_append(L, as_stream(stream), k, v, c);
        if (rc) return rc;
        const size_t ws_base = L->g.ring_rows > 0 ? L->floor_pos : 0;
        const size_t first_ws = std::max(ws_base, skv_window_start(L->len - c, L->window));
        if (c == 1) {
            rc = encode_attention(L, as_stream(stream), q, out, first_ws);
        } else {
            rc = encode_attention(L, as_stream(stream), q, out, ws_base, nullptr, nullptr, c);
        }
        if (rc) return rc;
        q += c * q_dim;
        k += c * kv_dim;
        v += c * kv_dim;
        out += c * q_dim;
    }
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prefill_chunk_host(skv_layer *L, const float *q, const float *k, const float *v,
                               size_t n_rows, float *out) try {
    if (!L || !q || !k || !v || !out) return fail(SKV_ERR_DEVICE, "prefill chunk: pointeur nul");
    if (n_rows == 0) return fail(SKV_ERR_DIMENSION, "attention batch cached shapes: seq == 0");
    SKV_HIP(hipSetDevice(L->ctx->device));
    const size_t kv_dim = skv_kv_dim(L), q_dim = (size_t)L->g.q_heads * L->g.head_dim;
    const size_t qb = n_rows * q_dim * sizeof(float), kb = n_rows * kv_dim * sizeof(float);
    char *buf = nullptr;
    SKV_HIP(hipMalloc((void **)&buf, 2 * qb + 2 * kb));
    float *qd = (float *)buf, *od = (float *)(buf + qb), *kd = (float *)(buf + 2 * qb),
          *vd = (float *)(buf + 2 * qb + kb);
    hipStream_t s = L->ctx->stream;
    hipError_t e = hipMemcpyAsync(qd, q, qb, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(kd, k, kb, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(vd, v, kb, hipMemcpyHostToDevice, s);
    int32_t rc = SKV_OK;
    if (e == hipSuccess) rc = skv_prefill_chunk_device(L, s, qd, kd, vd, n_rows, od);
    if (e == hipSuccess && !rc) e = hipMemcpyAsync(out, od, qb, hipMemcpyDeviceToHost, s);
    hipError_t e2 = hipStreamSynchronize(s);
    (void)hipFree(buf);
    if (e != hipSuccess) return fail_hip(e, "prefill chunk: copie");
    if (rc) return rc;
    if (e2 != hipSuccess) return fail_hip(e2, "prefill chunk: synchronisation");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

// ---- the step before the cache: per-head RMSNorm + rotation --------------------------

struct skv_rope {
    CtxRef ctx;
    float *table = nullptr; // [max_positions][rope_dims/2][2]
    size_t max_positions = 0;
    size_t rope_dims = 0;
    int style = 0;
};

int32_t skv_rope_rotations_host(size_t position, size_t rope_dims, size_t frequency_dim, float theta,
                                float position_scale, float *cos_sin_out) try {
    if (!cos_sin_out) return fail(SKV_ERR_DEVICE, "rope: pointeur nul");
    if (rope_dims == 0 || rope_dims % 2 != 0)
        return fail(SKV_ERR_DIMENSION, "RoPE: rope_dims=" + std::to_string(rope_dims) + " doit être pair et non nul");
    if (!(theta > 0.0f)) return fail(SKV_ERR_DIMENSION, "RoPE: theta doit être > 0");
    if (frequency_dim == 0) frequency_dim = rope_dims;
    // rope_rotations (src/decoder/attention_ops.rs:848-887), operation for operation in f32
    volatile float scaled_position = (float)position * position_scale;
    for (size_t pair = 0; pair < rope_dims / 2; ++pair) {
        volatile float exponent = (float)(2 * pair) / (float)frequency_dim;
        volatile float denom = powf(theta, exponent);
        volatile float angle = scaled_position / denom;
        cos_sin_out[2 * pair] = cosf(angle);
        cos_sin_out[2 * pair + 1] = sinf(angle);
    }
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_rope_create(skv_ctx *ctx, size_t max_positions, size_t rope_dims, size_t frequency_dim,
                        float theta, float position_scale, int32_t style, skv_rope **out) try {
    if (!ctx || !out) return fail(SKV_ERR_DEVICE, "skv_rope_create: pointeur nul");
    *out = nullptr;
    if (max_positions == 0 || max_positions > ((size_t)1 << 30))
        return fail(SKV_ERR_CONFIG, "RoPE: nombre de positions invalide");
    if (rope_dims > 512) return fail(SKV_ERR_CONFIG, "RoPE: rope_dims > 512 non supporté");
    if (style != 0 && style != 1) return fail(SKV_ERR_CONFIG, "RoPE: style inconnu");
    // one (cos, sin) pair per position and rotated pair, built on the host: keep it to a
    // size a host vector and a device buffer always hold (1 GiB = 2 M positions at 128 dims)
    if (max_positions * rope_dims > ((size_t)1 << 28))
        return fail(SKV_ERR_CONFIG, "RoPE: table de " + std::to_string(max_positions) + " positions x " +
                                        std::to_string(rope_dims) + " dims au-delà de 1 GiB");
    std::vector<float> host(max_positions * rope_dims);
    for (size_t p = 0; p < max_positions; ++p) {
        int32_t rc = skv_rope_rotations_host(p, rope_dims, frequency_dim, theta, position_scale,
                                             host.data() + p * rope_dims);
        if (rc) return rc;
    }
    SKV_HIP(hipSetDevice(ctx->device));
    skv_rope *r = new skv_rope();
    r->ctx = ctx;
    r->max_positions = max_positions;
    r->rope_dims = rope_dims;
    r->style = style;
    hipError_t e = hipMalloc((void **)&r->table, host.size() * sizeof(float));
    if (e == hipSuccess)
        e = hipMemcpy(r->table, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        if (r->table) (void)hipFree(r->table);
        delete r;
        return fail_hip(e, "RoPE: table des rotations");
    }
    *out = r;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

void skv_rope_destroy(skv_rope *rope) {
    if (!rope) return;
    (void)hipSetDevice(rope->ctx->device);
    (void)hipDeviceSynchronize();
    if (rope->table) (void)hipFree(rope->table);
    delete rope;
}

static int32_t check_rope(const skv_rope *rope, size_t position, size_t head_dim) {
    if (!rope) return SKV_OK;
    if (rope->rope_dims > head_dim)
        return fail(SKV_ERR_DIMENSION, "RoPE: rope_dims=" + std::to_string(rope->rope_dims) +
                                           " > head_dim=" + std::to_string(head_dim));
    if (position >= rope->max_positions)
        return fail(SKV_ERR_DIMENSION, "RoPE: position " + std::to_string(position) +
                                           " hors de la table (" + std::to_string(rope->max_positions) + ")");
    return SKV_OK;
}

int32_t skv_rms_norm_rope_decode_device(skv_ctx *ctx, skv_stream stream, const skv_rope *rope,
                                        size_t position, const float *x_dev, const float *weight_dev,
                                        size_t heads, size_t head_dim, float eps, float *out_dev) try {
    if (!ctx || !x_dev || !out_dev) return fail(SKV_ERR_DEVICE, "rms_norm_rope: pointeur nul");
    if (heads == 0 || head_dim == 0 || head_dim > 512 || heads > 65535)
        return fail(SKV_ERR_DIMENSION, "RMSNorm/RoPE heads invalide");
    int32_t rc = check_rope(rope, position, head_dim);
    if (rc) return rc;
    NormRopeArgs a{};
    a.x = x_dev;
    a.out = out_dev;
    a.weight = weight_dev;
    a.rope = rope ? rope->table + position * rope->rope_dims : nullptr;
    a.heads = (int)heads;
    a.head_dim = (int)head_dim;
    a.rope_dims = rope ? (int)rope->rope_dims : 0;
    a.rope_style = rope ? rope->style : 0;
    a.eps = eps;
    SKV_HIP(launch_norm_rope(a, as_stream(stream)));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_rms_norm_rope_rows_device(skv_ctx *ctx, skv_stream stream, const skv_rope *rope,
                                      size_t position_offset, const float *x_dev, const float *weight_dev,
                                      size_t n_rows, size_t heads, size_t head_dim, float eps,
                                      float *out_dev) try {
    if (!ctx || !x_dev || !out_dev) return fail(SKV_ERR_DEVICE, "rms_norm_rope: pointeur nul");
    if (heads == 0 || head_dim == 0 || head_dim > 512 || heads > 65535)
        return fail(SKV_ERR_DIMENSION, "RMSNorm/RoPE heads invalide");
    if (n_rows == 0) return SKV_OK;
    int32_t rc = check_rope(rope, position_offset + n_rows - 1, head_dim);
    if (rc) return rc;
    const size_t row_elems = heads * head_dim;
    for (size_t first = 0; first < n_rows; first += 65535) { // grid y limit
        const size_t n = std::min<size_t>(65535, n_rows - first);
        NormRopeArgs a{};
        a.x = x_dev + first * row_elems;
        a.out = out_dev + first * row_elems;
        a.weight = weight_dev;
        a.rope = rope ? rope->table + (position_offset + first) * rope->rope_dims : nullptr;
        a.heads = (int)heads;
        a.head_dim = (int)head_dim;
        a.rope_dims = rope ? (int)rope->rope_dims : 0;
        a.rope_style = rope ? rope->style : 0;
        a.eps = eps;
        a.n_rows = (int)n;
        SKV_HIP(launch_norm_rope(a, as_stream(stream)));
    }
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_rms_norm_rope_decode_host(skv_ctx *ctx, const float *x, const float *weight, size_t heads,
                                      size_t head_dim, size_t rope_dims, size_t frequency_dim,
                                      size_t position, float eps, float theta, float position_scale,
                                      int32_t style, float *out) try {
    if (!ctx || !x || !out) return fail(SKV_ERR_DEVICE, "rms_norm_rope: pointeur nul");
    if (heads == 0 || head_dim == 0 || head_dim > 512 || heads > 65535)
        return fail(SKV_ERR_DIMENSION, "RMSNorm/RoPE heads invalide");
    if (rope_dims == 0 || rope_dims > head_dim || rope_dims % 2 != 0)
        return fail(SKV_ERR_DIMENSION, "RMSNorm/RoPE: rope_dims invalide");
    if (style != 0 && style != 1) return fail(SKV_ERR_CONFIG, "RoPE: style inconnu");
    std::vector<float> cs(rope_dims);
    int32_t rc = skv_rope_rotations_host(position, rope_dims, frequency_dim, theta, position_scale, cs.data());
    if (rc) return rc;
    SKV_HIP(hipSetDevice(ctx->device));
    const size_t n = heads * head_dim;
    float *buf = nullptr;
    SKV_HIP(hipMalloc((void **)&buf, (2 * n + head_dim + rope_dims) * sizeof(float)));
    float *xd = buf, *od = buf + n, *wd = buf + 2 * n, *rd = wd + head_dim;
    hipStream_t s = ctx->stream;
    hipError_t e = hipMemcpyAsync(xd, x, n * sizeof(float), hipMemcpyHostToDevice, s);
    if (e == hipSuccess && weight) e = hipMemcpyAsync(wd, weight, head_dim * sizeof(float), hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(rd, cs.data(), rope_dims * sizeof(float), hipMemcpyHostToDevice, s);
    NormRopeArgs a{};
    a.x = xd;
    a.out = od;
    a.weight = weight ? wd : nullptr;
    a.rope = rd;
    a.heads = (int)heads;
    a.head_dim = (int)head_dim;
    a.rope_dims = (int)rope_dims;
    a.rope_style = style;
    a.eps = eps;
    if (e == hipSuccess) e = launch_norm_rope(a, s);
    if (e == hipSuccess) e = hipMemcpyAsync(out, od, n * sizeof(float), hipMemcpyDeviceToHost, s);
    hipError_t e2 = hipStreamSynchronize(s);
    (void)hipFree(buf);
    if (e != hipSuccess) return fail_hip(e, "rms_norm_rope");
    if (e2 != hipSuccess) return fail_hip(e2, "rms_norm_rope: synchronisation");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

static int32_t prekv_step(skv_layer *L, skv_stream stream, const skv_rope *rope, size_t position,
                          const float *q, size_t q_head_stride, const float *gate, const float *k,
                          const float *v, const float *q_norm_w, const float *k_norm_w, float eps,
                          float attn_scalar, float *out_dev) {
    if (!std::isfinite(attn_scalar) || attn_scalar <= 0.0f)
        return fail(SKV_ERR_CONFIG, "scalaire d'attention résident invalide: " + std::to_string(attn_scalar));
    int32_t rc = check_rope(rope, position, (size_t)L->g.head_dim);
    if (rc) return rc;
    if (L->len >= L->capacity)
        return fail(SKV_ERR_DIMENSION, "append KV résident: capacité " +
                                           std::to_string(L->capacity) + " atteinte (overflow)");
    hipStream_t s = as_stream(stream);
    const bool fused = tuning().fused_append;
    if (!fused || !uses_flash(L) || wide_f32_heads(L) || L->g.gqa > 16) {
        // the same step as separate launches: norm + rotation of q and k, append, attention, gate
        NormRopeArgs n{};
        n.x = q;
        n.out = L->q_stage;
        n.weight = q_norm_w;
        n.rope = rope ? rope->table + position * rope->rope_dims : nullptr;
        n.heads = L->g.q_heads;
        n.head_dim = L->g.head_dim;
        n.rope_dims = rope ? (int)rope->rope_dims : 0;
        n.rope_style = rope ? rope->style : 0;
        n.eps = eps;
        n.x_head_stride = (int)q_head_stride;
        SKV_HIP(launch_norm_rope(n, s));
        n.x = k;
        n.out = L->kv_stage;
        n.weight = k_norm_w;
        n.heads = L->g.kv_heads;
        n.x_head_stride = 0;
        SKV_HIP(launch_norm_rope(n, s));
        rc = encode_append(L, s, L->kv_stage, v, 1);
        if (rc) return rc;
        rc = encode_attention(L, s, L->q_stage, out_dev, skv_window_start(L->len - 1, L->window),
                              nullptr, nullptr, 1, attn_scalar);
        if (rc || !gate) return rc;
        GateArgs ga{};
        ga.ctx = out_dev;
        ga.gate = gate;
        ga.out = out_dev;
        ga.heads = L->g.q_heads;
        ga.head_dim = L->g.head_dim;
        ga.gate_head_stride = q_head_stride ? (int)q_head_stride : L->g.head_dim;
        SKV_HIP(launch_gate(ga, s));
        return SKV_OK;
    }
    PreKv pre{};
    pre.rope = rope ? rope->table + position * rope->rope_dims : nullptr;
    pre.q_norm_w = q_norm_w;
    pre.k_norm_w = k_norm_w;
    pre.eps = eps;
    pre.rope_dims = rope ? (int)rope->rope_dims : 0;
    pre.rope_style = rope ? rope->style : 0;
    pre.gate = gate;
    pre.q_head_stride = (int)q_head_stride;
    L->len += 1;
    if (L->g.ring_rows > 0 && L->len > (size_t)L->g.ring_rows)
        L->floor_pos = std::max(L->floor_pos, L->len - (size_t)L->g.ring_rows);
    rc = encode_attention(L, s, q, out_dev, skv_window_start(L->len - 1, L->window), k, v, 1,
                          attn_scalar, &pre);
    if (rc) L->len -= 1;
    return rc;
}

int32_t skv_decode_step_prekv_device(skv_layer *L, skv_stream stream, const skv_rope *rope,
                                     size_t position, const void *q_dev, size_t q_off,
                                     const void *k_dev, size_t k_off, const void *v_dev, size_t v_off,
                                     const float *q_norm_w, const float *k_norm_w, float eps,
                                     float attn_scalar, float *out_dev) try {
    if (!L || !q_dev || !k_dev || !v_dev || !out_dev)
        return fail(SKV_ERR_DEVICE, "decode_step_prekv: pointeur nul");
    if ((q_off | k_off | v_off) & 3) return fail(SKV_ERR_DIMENSION, "decode_step_prekv: offset non aligné f32");
    return prekv_step(L, stream, rope, position,
                      reinterpret_cast<const float *>((const char *)q_dev + q_off), 0, nullptr,
                      reinterpret_cast<const float *>((const char *)k_dev + k_off),
                      reinterpret_cast<const float *>((const char *)v_dev + v_off), q_norm_w,
                      k_norm_w, eps, attn_scalar, out_dev);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_decode_step_gated_device(skv_layer *L, skv_stream stream, const skv_rope *rope,
                                     size_t position, const void *qg_dev, size_t qg_off,
                                     const void *k_dev, size_t k_off, const void *v_dev, size_t v_off,
                                     const float *q_norm_w, const float *k_norm_w, float eps,
                                     float attn_scalar, float *out_dev) try {
    if (!L || !qg_dev || !k_dev || !v_dev || !out_dev)
        return fail(SKV_ERR_DEVICE, "decode_step_gated: pointeur nul");
    if ((qg_off | k_off | v_off) & 3) return fail(SKV_ERR_DIMENSION, "decode_step_gated: offset non aligné f32");
    // split_q_gate (src/decode_resident/kernels.rs:931-946) by addressing: head h holds its
    // head_dim query values at h * 2 * head_dim and its gate values right after them
    const float *qg = reinterpret_cast<const float *>((const char *)qg_dev + qg_off);
    const size_t hd = (size_t)L->g.head_dim;
    return prekv_step(L, stream, rope, position, qg, 2 * hd, qg + hd,
                      reinterpret_cast<const float *>((const char *)k_dev + k_off),
                      reinterpret_cast<const float *>((const char *)v_dev + v_off), q_norm_w,
                      k_norm_w, eps, attn_scalar, out_dev);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_attn_gate_device(skv_ctx *ctx, skv_stream stream, const float *ctx_dev, const float *gate_dev,
                             size_t gate_head_stride, size_t heads, size_t head_dim, float *out_dev) try {
    if (!ctx || !ctx_dev || !gate_dev || !out_dev) return fail(SKV_ERR_DEVICE, "attn_gate: pointeur nul");
    if (heads == 0 || head_dim == 0 || heads * head_dim > ((size_t)1 << 30))
        return fail(SKV_ERR_DIMENSION, "attn_gate: dimensions invalides");
    if (gate_head_stride != 0 && gate_head_stride < head_dim)
        return fail(SKV_ERR_DIMENSION, "attn_gate: pas du gate < head_dim");
    GateArgs ga{};
    ga.ctx = ctx_dev;
    ga.gate = gate_dev;
    ga.out = out_dev;
    ga.heads = (int)heads;
    ga.head_dim = (int)head_dim;
    ga.gate_head_stride = (int)(gate_head_stride ? gate_head_stride : head_dim);
    SKV_HIP(launch_gate(ga, as_stream(stream)));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_decode_step_batch_device(skv_layer *const *seqs, size_t n_seq, skv_stream stream,
                                     const void *const *k_dev, const void *const *v_dev,
                                     const float *const *q_dev, float *const *out_dev) try {
    if (!seqs || !k_dev || !v_dev || !q_dev || !out_dev)
        return fail(SKV_ERR_DEVICE, "decode_step_batch: pointeur nul");
    if (n_seq == 0) return fail(SKV_ERR_DIMENSION, "decode_step_batch: aucune séquence");
    for (size_t i = 0; i < n_seq; ++i) {
        const skv_layer *L = seqs[i];
        if (!L || !k_dev[i] || !v_dev[i] || !q_dev[i] || !out_dev[i])
            return fail(SKV_ERR_DEVICE, "decode_step_batch: pointeur nul (séquence " + std::to_string(i) + ")");
        const Geom &g = L->g, &g0 = seqs[0]->g;
        if (g.q_heads != g0.q_heads || g.kv_heads != g0.kv_heads || g.head_dim != g0.head_dim ||
            (g.ring_rows > 0) != (g0.ring_rows > 0) || g.f32 != g0.f32 || L->window != seqs[0]->window ||
            L->ctx != seqs[0]->ctx)
            return fail(SKV_ERR_DIMENSION, "decode_step_batch: la séquence " + std::to_string(i) +
                                               " n'a pas la géométrie de la séquence 0");
        for (size_t j = 0; j < i; ++j)
            if (seqs[j] == L)
                return fail(SKV_ERR_DIMENSION, "decode_step_batch: séquence " + std::to_string(i) + " en double");
        // nothing is modified unless every sequence can take its row
        if (L->len >= L->capacity)
            return fail(SKV_ERR_DIMENSION, "append KV résident: capacité " + std::to_string(L->capacity) +
                                               " atteinte (overflow), séquence " + std::to_string(i));
    }
    const bool fused = tuning().fused_append;
    if (!fused || !uses_flash(seqs[0]) || seqs[0]->g.gqa > 16 || n_seq == 1 || !fused_append_built(seqs[0])) {
        for (size_t i = 0; i < n_seq; ++i) {
            int32_t rc = skv_decode_step_device(seqs[i], stream, k_dev[i], 0, v_dev[i], 0, q_dev[i], out_dev[i]);
            if (rc) return rc;
        }
        return SKV_OK;
    }
    for (size_t first = 0; first < n_seq; first += SKV_MAX_BATCH) {
        const size_t n = std::min<size_t>(SKV_MAX_BATCH, n_seq - first);
        // the workgroup budget is shared in proportion to the pages each sequence scans
        size_t pages_total = 0;
        for (size_t i = 0; i < n; ++i) {
            const skv_layer *L = seqs[first + i];
            const size_t rows = L->g.ring_rows > 0 ? std::min<size_t>(L->len + 1, (size_t)L->g.ring_rows)
                                                   : L->len + 1 - skv_window_start(L->len, L->window);
            pages_total += (rows + 15) / 16;
        }
        DecodeBatchArgs b{};
        size_t floor_before[SKV_MAX_BATCH];
        for (size_t i = 0; i < n; ++i) {
            skv_layer *L = seqs[first + i];
            // the attention kernel writes the row itself: advance the bookkeeping first
            floor_before[i] = L->floor_pos;
            L->len += 1;
            if (L->g.ring_rows > 0 && L->len > (size_t)L->g.ring_rows)
                L->floor_pos = std::max(L->floor_pos, L->len - (size_t)L->g.ring_rows);
            const size_t ws = skv_window_start(L->len - 1, L->window);
            const size_t rows = L->g.ring_rows > 0 ? std::min<size_t>(L->len, (size_t)L->g.ring_rows) : L->len - ws;
            const size_t share = std::max<size_t>(decode_target_wgs() * ((rows + 15) / 16) / std::max<size_t>(pages_total, 1),
                                                  (size_t)L->g.kv_heads);
            fill_decode_args(L, q_dev[first + i], out_dev[first + i], ws,
                             reinterpret_cast<const float *>(k_dev[first + i]),
                             reinterpret_cast<const float *>(v_dev[first + i]), 1, share, b.seq[i]);
        }
        hipError_t e = launch_decode_batch(b, (int)n, as_stream(stream));
        if (e != hipSuccess) {
            for (size_t i = 0; i < n; ++i) {
                seqs[first + i]->len -= 1;
                seqs[first + i]->floor_pos = floor_before[i];
            }
            return fail_hip(e, "decode_step_batch: lancement");
        }
    }
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_decode_step_layers_device(skv_layer *const *layers, size_t n_layers, skv_stream stream,
                                      const void *const *k_dev, const void *const *v_dev,
                                      const float *const *q_dev, float *const *out_dev) try {
    if (!layers || !k_dev || !v_dev || !q_dev || !out_dev)
        return fail(SKV_ERR_DEVICE, "decode_step_layers: pointeur nul");
    for (size_t i = 0; i < n_layers; ++i) {
        int32_t rc = skv_decode_step_device(layers[i], stream, k_dev[i], 0, v_dev[i], 0, q_dev[i],
                                            out_dev[i]);
        if (rc) return rc;
    }
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

static int32_t check_rows(const skv_layer *L, size_t first, size_t n) {
    if (first + n > L->len)
        return fail(SKV_ERR_DIMENSION, "lecture KV lignes " + std::to_string(first) + ".." +
                                           std::to_string(first + n) + " > len " +
                                           std::to_string(L->len));
    if (L->g.ring_rows > 0 && n > 0 && first < L->floor_pos)
        return fail(SKV_ERR_DIMENSION, "lecture KV: ligne " + std::to_string(first) +
                                           " déjà évincée de l'anneau");
    return SKV_OK;
}

int32_t skv_gather_device(skv_layer *L, skv_stream stream, size_t first, size_t n, void *k_dst,
                          void *v_dst) try {
    if (!L) return fail(SKV_ERR_DEVICE, "gather: pointeur nul");
    int32_t rc = check_rows(L, first, n);
    if (rc) return rc;
    if (n == 0) return SKV_OK;
    GatherArgs a{};
    a.k_pool = L->k_pool;
    a.v_pool = L->v_pool;
    a.table = L->table_dev;
    a.k_dst = (uint16_t *)k_dst;
    a.v_dst = (uint16_t *)v_dst;
    a.first_pos = (long)first;
    a.n_rows = (int)n;
    a.g = L->g;
    SKV_HIP(L->g.f32 ? launch_gather_f32(a, as_stream(stream)) : launch_gather(a, as_stream(stream)));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

// Rows of either storage mode as f32 (bf16 rows widened: exact).
int32_t skv_read_rows_f32(skv_layer *L, size_t first, size_t n, float *k_out, float *v_out) try {
    if (!L) return fail(SKV_ERR_DEVICE, "read_rows: pointeur nul");
    int32_t rc = check_rows(L, first, n);
    if (rc) return rc;
    if (n == 0) return SKV_OK;
    const size_t elems = n * skv_kv_dim(L);
    if (!L->g.f32) {
        std::vector<uint16_t> kb(k_out ? elems : 0), vb(v_out ? elems : 0);
        rc = skv_read_rows(L, first, n, k_out ? kb.data() : nullptr, v_out ? vb.data() : nullptr);
        if (rc) return rc;
        auto widen = [](uint16_t b) {
            const uint32_t u = (uint32_t)b << 16;
            float f;
            std::memcpy(&f, &u, sizeof f);
            return f;
        };
        for (size_t i = 0; i < kb.size(); ++i) k_out[i] = widen(kb[i]);
        for (size_t i = 0; i < vb.size(); ++i) v_out[i] = widen(vb[i]);
        return SKV_OK;
    }
    SKV_HIP(hipSetDevice(L->ctx->device));
    float *tmp = nullptr;
    SKV_HIP(hipMalloc((void **)&tmp, 2 * elems * sizeof(float)));
    hipStream_t s = L->ctx->stream;
    float *kd = tmp, *vd = tmp + elems;
    rc = skv_gather_device(L, s, first, n, k_out ? kd : nullptr, v_out ? vd : nullptr);
    hipError_t e = hipSuccess;
    if (!rc && k_out) e = hipMemcpyAsync(k_out, kd, elems * sizeof(float), hipMemcpyDeviceToHost, s);
    if (!rc && e == hipSuccess && v_out) e = hipMemcpyAsync(v_out, vd, elems * sizeof(float), hipMemcpyDeviceToHost, s);
    hipError_t e2 = hipStreamSynchronize(s);
    (void)hipFree(tmp);
    if (rc) return rc;
    if (e != hipSuccess) return fail_hip(e, "read_rows: copie device→hôte");
    if (e2 != hipSuccess) return fail_hip(e2, "read_rows: synchronisation");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_read_rows(skv_layer *L, size_t first, size_t n, uint16_t *k_out, uint16_t *v_out) try {
    if (!L) return fail(SKV_ERR_DEVICE, "read_rows: pointeur nul");
    if (L->g.f32) return fail(SKV_ERR_CONFIG, "read_rows: cache f32, lire avec skv_read_rows_f32");
    int32_t rc = check_rows(L, first, n);
    if (rc) return rc;
    if (n == 0) return SKV_OK;
    SKV_HIP(hipSetDevice(L->ctx->device));
    const size_t bytes = n * skv_kv_dim(L) * sizeof(uint16_t);
    uint16_t *tmp = nullptr;
    SKV_HIP(hipMalloc((void **)&tmp, 2 * bytes));
    hipStream_t s = L->ctx->stream;
    uint16_t *kd = tmp, *vd = tmp + n * skv_kv_dim(L);
    rc = skv_gather_device(L, s, first, n, k_out ? kd : nullptr, v_out ? vd : nullptr);
    hipError_t e = hipSuccess;
    if (!rc && k_out) e = hipMemcpyAsync(k_out, kd, bytes, hipMemcpyDeviceToHost, s);
    if (!rc && e == hipSuccess && v_out) e = hipMemcpyAsync(v_out, vd, bytes, hipMemcpyDeviceToHost, s);
    hipError_t e2 = hipStreamSynchronize(s);
    (void)hipFree(tmp);
    if (rc) return rc;
    if (e != hipSuccess) return fail_hip(e, "read_rows: copie device→hôte");
    if (e2 != hipSuccess) return fail_hip(e2, "read_rows: synchronisation");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

// ---- measurement aids ---------------------------------------------------------------------
static int32_t probe_read(skv_layer *L, skv_stream stream, bool store_partials) {
    if (!L) return fail(SKV_ERR_DEVICE, "probe: pointeur nul");
    if (L->len == 0) return fail(SKV_ERR_DIMENSION, "probe: cache vide");
    ProbeArgs a{};
    a.k_pool = L->k_pool;
    a.v_pool = L->v_pool;
    a.table = L->table_dev;
    a.sink = nullptr;
    a.n_pages = (int)std::min<size_t>((L->len + 15) / 16, (size_t)L->n_pages);
    a.splits = (int)std::max<size_t>(std::min<size_t>(decode_target_wgs() / (size_t)L->g.kv_heads, (size_t)a.n_pages), 1);
    a.splits = std::min(a.splits, L->max_splits);
    a.g = L->g;
    if (store_partials) {
        // (o[head_dim] per head of the group, rounded down to whole 16-byte units; m and l are 2 of 258 floats)
        a.part = L->part_o;
        a.part_floats = (L->g.gqa * L->g.head_dim) & ~3;
    }
    SKV_HIP(launch_probe_read(a, as_stream(stream)));
    return SKV_OK;
}

int32_t skv_probe_read_pages_device(skv_layer *L, skv_stream stream) try {
    return probe_read(L, stream, false);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_probe_read_store_pages_device(skv_layer *L, skv_stream stream) try {
    return probe_read(L, stream, true);
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_probe_merge_device(skv_layer *L, skv_stream stream, float *out_dev) try {
    if (!L || !out_dev) return fail(SKV_ERR_DEVICE, "probe: pointeur nul");
    if (L->len == 0) return fail(SKV_ERR_DIMENSION, "probe: cache vide");
    if (!uses_flash(L)) return fail(SKV_ERR_CONFIG, "probe: noyau matriciel seulement");
    DecodeArgs a{};
    fill_decode_args(L, nullptr, out_dev, skv_window_start(L->len - 1, L->window), nullptr, nullptr, 1,
                     decode_target_wgs(), a);
    if (a.splits > 1) SKV_HIP(launch_merge(a, as_stream(stream)));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_probe_empty_launch_device(skv_ctx *ctx, skv_stream stream) try {
    if (!ctx) return fail(SKV_ERR_DEVICE, "probe: ctx nul");
    SKV_HIP(launch_probe_empty(as_stream(stream)));
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

} // extern "C"
