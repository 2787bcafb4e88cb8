// Block snapshot / restore of the paged cache, recurrent-state snapshots, and the GPU
// side of the prefix hot cache (a pool of page slots indexed by the chained block
// hash with LRU eviction). Stands in for snapshot/copy/restore_prompt_state_metal
// (src/decoder/generation.rs:2834-2892, 3041-3103), the blits of
// src/metal_backend/linear_attention.rs:3027-3067, 3163-3198, and the GPU half of
// remember_prefix_block / prefill_prompt_state (src/serve/state.rs:560-639).
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "layer.h"
#include "prefix.h"

namespace skv {

// ---- one launch copies up to COPY_MAX_PAGES pages of up to COPY_MAX_LAYERS layers --------
constexpr int COPY_MAX_LAYERS = 48;
constexpr int COPY_MAX_PAGES = 192;

struct CopyLayer {
    uint16_t *k_pool;
    uint16_t *v_pool;
    const int32_t *table;
    uint64_t slot_off;    // byte offset of this layer's K page inside a slot; V follows it
    uint32_t page_bytes;  // bytes of one K (or V) page of this layer
    uint32_t ring_pages;  // 0, or the ring's page count (logical page -> page % ring_pages)
    uint32_t first_page;  // logical pages below this one are skipped (rows a ring no longer holds)
    uint32_t pad;
    uint64_t slot_stride; // bytes between this layer's pages of consecutive slots
};

struct CopyArgs {
    CopyLayer layers[COPY_MAX_LAYERS];
    int32_t layer_page[COPY_MAX_PAGES]; // logical page inside every layer
    int32_t slot[COPY_MAX_PAGES];       // page slot inside the snapshot storage
    uint8_t *base;                      // snapshot storage
    int n_layers;
    int n_pages;
    int to_snapshot; // 1: cache -> storage, 0: storage -> cache
    int layer_major; // workgroup order, see page_copy_kernel
};

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Streams n16 16-byte words from src to dst: eight independent loads in flight per thread,
// then eight stores, all non-temporal (the data is touched once; keeping it out of the
// caches leaves them to the attention kernels and measurably raises copy bandwidth).
__device__ __forceinline__ void copy_stream(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst,
                                            long n16, long first, long stride) {
    long i = first;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u) __builtin_nontemporal_store(v[u], dst + i + u * stride);
    }
    for (; i < n16; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// One workgroup per (page, layer, K|V): a contiguous page_bytes chunk on both sides,
// 16-byte loads, eight in flight per thread. Consecutive workgroups walk the layers of one
// page (the order of a storage slot: the writes of a snapshot are contiguous) or, with
// layer_major, the pages of one layer (the writes of a restore stay inside one layer's pool
// instead of spreading over all of them, worth 6-10 % on launches of 100 pages and more).
__global__ __launch_bounds__(256) void page_copy_kernel(CopyArgs a) {
    const int chunk = blockIdx.x;
    const int kv = chunk & 1;
    const int li = a.layer_major ? (chunk >> 1) / a.n_pages : (chunk >> 1) % a.n_layers;
    const int pi = a.layer_major ? (chunk >> 1) % a.n_pages : (chunk >> 1) / a.n_layers;
    const CopyLayer &L = a.layers[li];
    const uint32_t lp = (uint32_t)a.layer_page[pi];
    if (lp < L.first_page) return;
    const uint32_t tp = L.ring_pages ? lp % L.ring_pages : lp;
    const int page = L.table[tp];
    uint8_t *cache = reinterpret_cast<uint8_t *>(kv ? L.v_pool : L.k_pool) + (size_t)page * L.page_bytes;
    uint8_t *store = a.base + (size_t)a.slot[pi] * L.slot_stride + L.slot_off + (size_t)kv * L.page_bytes;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(a.to_snapshot ? cache : store);
    u32x4 *dst = reinterpret_cast<u32x4 *>(a.to_snapshot ? store : cache);
    copy_stream(src, dst, (long)(L.page_bytes >> 4), threadIdx.x, 256);
}

// ---- flat copies of several device buffers in one launch (recurrent state) ----------------
constexpr int FLAT_MAX = 120;
constexpr uint32_t FLAT_CHUNK16 = 2048; // 16-byte words per workgroup: 32 KiB, eight per thread
struct FlatArgs {
    const uint8_t *src[FLAT_MAX];
    uint8_t *dst[FLAT_MAX];
    uint64_t bytes[FLAT_MAX];
    uint32_t first_chunk[FLAT_MAX + 1]; // running count of 32 KiB chunks: buffer i owns [first_chunk[i], first_chunk[i+1])
    int n;
};

// One workgroup per 32 KiB chunk of one buffer (a buffer of 96 KiB gets three workgroups, one
// of 2 MiB sixty-four: none idles and none loops), eight non-temporal 16-byte loads in flight
// per thread, then the stores.
__global__ __launch_bounds__(256) void flat_copy_kernel(FlatArgs a) {
    const uint32_t chunk = blockIdx.x;
    int lo = 0, hi = a.n - 1; // the buffer that owns the chunk (uniform: scalar loads)
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (a.first_chunk[mid] <= chunk) lo = mid; else hi = mid - 1;
    }
    const int b = lo;
    const uint64_t n = a.bytes[b];
    const long n16 = (long)(n >> 4);
    const long w0 = (long)(chunk - a.first_chunk[b]) * FLAT_CHUNK16;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(a.src[b]);
    u32x4 *dst = reinterpret_cast<u32x4 *>(a.dst[b]);
    const long end = min(w0 + (long)FLAT_CHUNK16, n16);
    if (w0 + (long)FLAT_CHUNK16 <= n16) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + w0 + u * 256 + threadIdx.x);
#pragma unroll
        for (int u = 0; u < 8; ++u) __builtin_nontemporal_store(v[u], dst + w0 + u * 256 + threadIdx.x);
    } else {
        for (long i = w0 + threadIdx.x; i < end; i += 256) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
    }
    if (end == n16) // the chunk that ends the buffer also copies its last bytes, if any
        for (uint64_t i = ((uint64_t)n16 << 4) + threadIdx.x; i < n; i += 256) a.dst[b][i] = a.src[b][i];
}

static int32_t launch_flat(const void *const *src, void *const *dst, const size_t *bytes, size_t n,
                           hipStream_t s) {
    size_t first = 0;
    while (first < n) {
        FlatArgs a{};
        uint64_t chunks = 0;
        int k = 0;
        // as many buffers as fit the argument block and a 32-bit chunk count
        for (; k < FLAT_MAX && first + k < n; ++k) {
            const uint64_t c = std::max<uint64_t>((((uint64_t)bytes[first + k] >> 4) + FLAT_CHUNK16 - 1) / FLAT_CHUNK16, 1);
            if (chunks + c > 0x7fffffffull) break;
            a.src[k] = (const uint8_t *)src[first + k];
            a.dst[k] = (uint8_t *)dst[first + k];
            a.bytes[k] = bytes[first + k];
            if (((uintptr_t)a.src[k] | (uintptr_t)a.dst[k]) & 15)
                return fail(SKV_ERR_DEVICE, "copie d'état: pointeur non aligné sur 16 octets");
            a.first_chunk[k] = (uint32_t)chunks;
            chunks += c;
        }
        if (k == 0) return fail(SKV_ERR_DIMENSION, "copie d'état: tampon trop grand pour un lancement");
        a.first_chunk[k] = (uint32_t)chunks;
        a.n = k;
        hipLaunchKernelGGL(flat_copy_kernel, dim3((unsigned)chunks), dim3(256), 0, s, a);
        SKV_HIP(hipGetLastError());
        first += (size_t)k;
    }
    return SKV_OK;
}

// Shapes of the layers a storage area was laid out for.
struct SlotLayout {
    std::vector<uint32_t> page_bytes; // per layer
    std::vector<uint64_t> shape;      // per layer: what the bytes of a page mean
    std::vector<uint64_t> slot_off;
    std::vector<uint64_t> slot_stride;
    uint64_t slot_bytes = 0;
    bool layer_major = false;

    // kv heads, head_dim and element: two layers whose pages merely have the same size
    // (bf16 at head_dim 256 and f32 at 128, say) must not exchange pages
    static uint64_t shape_of(const skv_layer *L) {
        return ((uint64_t)L->g.kv_heads << 32) | ((uint64_t)L->g.head_dim << 1) | (uint64_t)(L->g.f32 & 1);
    }
    void build(skv_layer *const *layers, size_t n, size_t slots = 0, bool by_layer = false) {
        page_bytes.resize(n);
        shape.resize(n);
        slot_off.resize(n);
        slot_stride.resize(n);
        slot_bytes = 0;
        for (size_t i = 0; i < n; ++i) {
            page_bytes[i] = (uint32_t)((size_t)layers[i]->g.page_elems * sizeof(uint16_t));
            shape[i] = shape_of(layers[i]);
            slot_off[i] = slot_bytes;
            slot_bytes += 2ull * page_bytes[i];
        }
        // Slot-major storage: slot s holds one page of every layer, K then V, contiguously.
        // Layer-major storage (the hot cache's pool and the snapshot objects): a layer's pages
        // of all `slots` slots form one region, so the launches of a restore, which walk layer
        // by layer, read from one region and write into one pool at a time (217-219 us against
        // 228 us for 256 blocks of 36 layers; one-block snapshots cost the same either way).
        layer_major = by_layer;
        for (size_t i = 0; i < n; ++i) {
            slot_stride[i] = by_layer ? 2ull * page_bytes[i] : slot_bytes;
            if (by_layer) slot_off[i] *= slots;
        }
    }
    bool matches(skv_layer *const *layers, size_t n) const {
        if (n != page_bytes.size()) return false;
        for (size_t i = 0; i < n; ++i)
            if (shape[i] != shape_of(layers[i])) return false;
        return true;
    }
};

// Pages in a restore launch from which its workgroups go layer by layer (measured: below
// about 64 pages the slot order is as good or better). SKV_COPY_LAYER_MAJOR_MIN_PAGES
// overrides it; read once per flag generation.
static size_t layer_major_min_pages() {
    thread_local uint64_t seen = 0;
    thread_local size_t value = 64;
    const uint64_t epoch = skv_internal_flags_epoch();
    if (epoch != seen) {
        const char *raw = std::getenv("SKV_COPY_LAYER_MAJOR_MIN_PAGES");
        char *end = nullptr;
        const unsigned long long v = raw && *raw ? std::strtoull(raw, &end, 10) : 64;
        value = raw && *raw && end != raw ? (size_t)v : 64;
        seen = epoch;
    }
    return value;
}

// Copies pages between `layers` and the storage at `base`: logical page layer_pages[i] of
// every layer <-> slot slots[i]. first_page[l] (optional) skips the low pages of layer l.
static int32_t copy_pages(const SlotLayout &lay, uint8_t *base, skv_layer *const *layers,
                          size_t n_layers, const int32_t *layer_pages, const int32_t *slots,
                          size_t n_pages, const uint32_t *first_page, bool to_snapshot,
                          hipStream_t s) {
    for (size_t l0 = 0; l0 < n_layers; l0 += COPY_MAX_LAYERS) {
        const size_t nl = std::min<size_t>(COPY_MAX_LAYERS, n_layers - l0);
        for (size_t p0 = 0; p0 < n_pages; p0 += COPY_MAX_PAGES) {
            CopyArgs a{};
            a.n_layers = (int)nl;
            a.n_pages = (int)std::min<size_t>(COPY_MAX_PAGES, n_pages - p0);
            a.base = base;
            a.to_snapshot = to_snapshot ? 1 : 0;
            a.layer_major = (!to_snapshot || lay.layer_major) && (size_t)a.n_pages >= layer_major_min_pages() ? 1 : 0;
            for (size_t i = 0; i < nl; ++i) {
                skv_layer *L = layers[l0 + i];
                CopyLayer &c = a.layers[i];
                c.k_pool = L->k_pool;
                c.v_pool = L->v_pool;
                c.table = L->table_dev;
                c.slot_off = lay.slot_off[l0 + i];
                c.slot_stride = lay.slot_stride[l0 + i];
                c.page_bytes = lay.page_bytes[l0 + i];
                c.ring_pages = L->g.ring_rows > 0 ? (uint32_t)L->n_pages : 0;
                c.first_page = first_page ? first_page[l0 + i] : 0;
            }
            for (int i = 0; i < a.n_pages; ++i) {
                a.layer_page[i] = layer_pages[p0 + i];
                a.slot[i] = slots[p0 + i];
            }
            hipLaunchKernelGGL(page_copy_kernel, dim3((unsigned)(a.n_pages * a.n_layers * 2)), dim3(256),
                               0, s, a);
            SKV_HIP(hipGetLastError());
        }
    }
    return SKV_OK;
}

static int32_t check_layers(skv_ctx *ctx, skv_layer *const *layers, size_t n_layers) {
    if (!ctx || !layers || n_layers == 0) return fail(SKV_ERR_DEVICE, "snapshot: pointeur nul");
    for (size_t i = 0; i < n_layers; ++i)
        if (!layers[i] || layers[i]->ctx != ctx) return fail(SKV_ERR_DEVICE, "snapshot: couche invalide");
    return SKV_OK;
}

} // namespace skv

using namespace skv;

struct skv_snapshot {
    CtxRef ctx;
    uint8_t *base = nullptr;
    size_t bytes = 0;
    // block snapshots
    SlotLayout layout;
    size_t n_pages = 0;
    // state snapshots
    std::vector<size_t> sizes;   // bytes of each buffer
    std::vector<size_t> offsets; // 256-byte aligned offsets inside `base`
};

static hipStream_t as_stream(skv_stream s) { return reinterpret_cast<hipStream_t>(s); }

struct HotEntry {
    std::vector<int32_t> slots;  // one per 16-token page of the block
    skv_snapshot *state = nullptr; // recurrent state at the block boundary, or null
    size_t bytes = 0;
};

struct skv_hot {
    CtxRef ctx;
    PrefixIndex *index = nullptr;
    SlotLayout layout;
    size_t pages_per_block = 0;
    size_t pool_slots = 0;
    uint8_t *pool = nullptr;
    std::vector<int32_t> free_slots;
    std::unordered_map<uint64_t, HotEntry> entries;
    uint64_t next_id = 1;
    // counters (x-saragossa-reused-prefix-tokens accounting and eviction log, serve/state.rs:59-80, 263-266)
    uint64_t evictions = 0;
    uint64_t skipped = 0;
    // State buffers of evicted entries, kept for the next remember of the same shapes: an
    // eviction then costs neither a device synchronisation nor a free, a remember no
    // allocation (copies into and out of them are ordered by the stream, like the page slots).
    std::vector<skv_snapshot *> spare_states;
};
constexpr size_t HOT_MAX_SPARE_STATES = 4;

static void hot_release(skv_hot *h, uint64_t id) {
    auto it = h->entries.find(id);
    if (it == h->entries.end()) return;
    for (int32_t s : it->second.slots) h->free_slots.push_back(s);
    if (it->second.state) {
        if (h->spare_states.size() < HOT_MAX_SPARE_STATES)
            h->spare_states.push_back(it->second.state);
        else
            skv_snapshot_free(it->second.state);
    }
    h->entries.erase(it);
}

extern "C" {

// ---- block snapshots ----------------------------------------------------------------------
int32_t skv_snapshot_blocks(skv_ctx *ctx, skv_stream stream, skv_layer *const *layers,
                            size_t n_layers, const size_t *block_ids, size_t n_blocks,
                            skv_snapshot **out) try {
    if (!out) return fail(SKV_ERR_DEVICE, "snapshot_blocks: out nul");
    *out = nullptr;
    int32_t rc = check_layers(ctx, layers, n_layers);
    if (rc) return rc;
    if (n_blocks && !block_ids) return fail(SKV_ERR_DEVICE, "snapshot_blocks: block_ids nul");
    std::vector<int32_t> pages(n_blocks), slots(n_blocks);
    for (size_t i = 0; i < n_blocks; ++i) {
        for (size_t l = 0; l < n_layers; ++l) {
            const skv_layer *L = layers[l];
            if (block_ids[i] * 16 >= L->len)
                return fail(SKV_ERR_DIMENSION, "snapshot_blocks: bloc " + std::to_string(block_ids[i]) +
                                                   " au-delà de len " + std::to_string(L->len));
            if (L->g.ring_rows > 0 && block_ids[i] * 16 < L->floor_pos)
                return fail(SKV_ERR_DIMENSION, "snapshot_blocks: bloc déjà évincé de l'anneau");
        }
        pages[i] = (int32_t)block_ids[i];
        slots[i] = (int32_t)i;
    }
    SKV_HIP(hipSetDevice(ctx->device));
    skv_snapshot *snap = new skv_snapshot();
    snap->ctx = ctx;
    snap->layout.build(layers, n_layers, n_blocks, true);
    snap->n_pages = n_blocks;
    snap->bytes = n_blocks * snap->layout.slot_bytes;
    if (snap->bytes) {
        hipError_t e = hipMalloc((void **)&snap->base, snap->bytes);
        if (e != hipSuccess) {
            delete snap;
            return fail_hip(e, "snapshot_blocks: allocation");
        }
        rc = copy_pages(snap->layout, snap->base, layers, n_layers, pages.data(), slots.data(),
                        n_blocks, nullptr, true, as_stream(stream));
        if (rc) {
            skv_snapshot_free(snap);
            return rc;
        }
    }
    *out = snap;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_restore_blocks(skv_ctx *ctx, skv_stream stream, const skv_snapshot *snap,
                           skv_layer *const *layers, size_t n_layers, const size_t *dst_block_ids,
                           size_t n_blocks) try {
    if (!snap) return fail(SKV_ERR_DEVICE, "restore_blocks: snapshot nul");
    if (n_blocks && !dst_block_ids) return fail(SKV_ERR_DEVICE, "restore_blocks: dst_block_ids nul");
    int32_t rc = check_layers(ctx, layers, n_layers);
    if (rc) return rc;
    if (!snap->sizes.empty()) return fail(SKV_ERR_DEVICE, "restore_blocks: snapshot d'état, pas de blocs");
    if (!snap->layout.matches(layers, n_layers))
        return fail(SKV_ERR_DIMENSION, "prefix-cache: snapshots=" + std::to_string(snap->layout.page_bytes.size()) +
                                           " couches=" + std::to_string(n_layers) + " ou formes différentes");
    if (n_blocks != snap->n_pages)
        return fail(SKV_ERR_DIMENSION, "restore_blocks: " + std::to_string(n_blocks) + " blocs, snapshot de " +
                                           std::to_string(snap->n_pages));
    std::vector<int32_t> pages(n_blocks), slots(n_blocks);
    for (size_t i = 0; i < n_blocks; ++i) {
        for (size_t l = 0; l < n_layers; ++l) {
            const skv_layer *L = layers[l];
            const size_t cap_pages = L->g.ring_rows > 0 ? (L->capacity + 15) / 16 : (size_t)L->n_pages;
            if (dst_block_ids[i] >= cap_pages)
                return fail(SKV_ERR_DIMENSION, "restore_blocks: bloc " + std::to_string(dst_block_ids[i]) +
                                                   " > capacité");
        }
        pages[i] = (int32_t)dst_block_ids[i];
        slots[i] = (int32_t)i;
    }
    if (n_blocks == 0) return SKV_OK;
    SKV_HIP(hipSetDevice(ctx->device));
    return copy_pages(snap->layout, snap->base, layers, n_layers, pages.data(), slots.data(), n_blocks,
                      nullptr, false, as_stream(stream));
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_snapshot_clone(skv_ctx *ctx, skv_stream stream, const skv_snapshot *snap,
                           skv_snapshot **out) try {
    if (!ctx || !snap || !out) return fail(SKV_ERR_DEVICE, "snapshot_clone: pointeur nul");
    *out = nullptr;
    SKV_HIP(hipSetDevice(ctx->device));
    skv_snapshot *c = new skv_snapshot(*snap);
    c->base = nullptr;
    if (c->bytes) {
        hipError_t e = hipMalloc((void **)&c->base, c->bytes);
        if (e != hipSuccess) {
            delete c;
            return fail_hip(e, "snapshot_clone: allocation");
        }
        const void *src = snap->base;
        void *dst = c->base;
        int32_t rc = launch_flat(&src, &dst, &c->bytes, 1, as_stream(stream));
        if (rc) {
            skv_snapshot_free(c);
            return rc;
        }
    }
    *out = c;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

size_t skv_snapshot_bytes(const skv_snapshot *snap) { return snap ? snap->bytes : 0; }

void skv_snapshot_free(skv_snapshot *snap) {
    if (!snap) return;
    if (snap->base) {
        (void)hipSetDevice(snap->ctx->device);
        (void)hipDeviceSynchronize(); // copies that read or write it may still be queued
        (void)hipFree(snap->base);
    }
    delete snap;
}

// ---- recurrent-state snapshots ---------------------------------------------------------------
int32_t skv_state_snapshot(skv_ctx *ctx, skv_stream stream, const void *const *dev_ptrs,
                           const size_t *bytes, size_t n, skv_snapshot **out) try {
    if (!ctx || !out || (n && (!dev_ptrs || !bytes))) return fail(SKV_ERR_DEVICE, "state_snapshot: pointeur nul");
    *out = nullptr;
    SKV_HIP(hipSetDevice(ctx->device));
    skv_snapshot *snap = new skv_snapshot();
    snap->ctx = ctx;
    size_t total = 0;
    for (size_t i = 0; i < n; ++i) {
        if (!dev_ptrs[i]) {
            delete snap;
            return fail(SKV_ERR_DEVICE, "state_snapshot: pointeur nul");
        }
        snap->sizes.push_back(bytes[i]);
        snap->offsets.push_back(total);
        total += (bytes[i] + 255) / 256 * 256;
    }
    snap->bytes = total;
    if (total) {
        hipError_t e = hipMalloc((void **)&snap->base, total);
        if (e != hipSuccess) {
            delete snap;
            return fail_hip(e, "state_snapshot: allocation");
        }
        std::vector<void *> dst(n);
        for (size_t i = 0; i < n; ++i) dst[i] = snap->base + snap->offsets[i];
        int32_t rc = launch_flat(dev_ptrs, dst.data(), bytes, n, as_stream(stream));
        if (rc) {
            skv_snapshot_free(snap);
            return rc;
        }
    }
    if (n == 0) snap->sizes.clear();
    *out = snap;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_state_restore(skv_ctx *ctx, skv_stream stream, const skv_snapshot *snap,
                          void *const *dev_ptrs, const size_t *bytes, size_t n) try {
    if (!ctx || !snap || (n && (!dev_ptrs || !bytes))) return fail(SKV_ERR_DEVICE, "state_restore: pointeur nul");
    if (n != snap->sizes.size())
        return fail(SKV_ERR_DIMENSION, "prefix-cache: snapshots=" + std::to_string(snap->sizes.size()) +
                                           " couches=" + std::to_string(n));
    for (size_t i = 0; i < n; ++i)
        if (bytes[i] != snap->sizes[i])
            return fail(SKV_ERR_DIMENSION, "state_restore: taille du tampon " + std::to_string(i) + " différente");
    if (n == 0) return SKV_OK;
    SKV_HIP(hipSetDevice(ctx->device));
    std::vector<const void *> src(n);
    for (size_t i = 0; i < n; ++i) src[i] = snap->base + snap->offsets[i];
    return launch_flat(src.data(), dev_ptrs, bytes, n, as_stream(stream));
} catch (...) {
    return skv::fail_exception();
}

// ---- the hot cache: page pool + index ----------------------------------------------------------
int32_t skv_hot_create(skv_ctx *ctx, size_t block_tokens, size_t capacity_blocks,
                       size_t blocks_per_session, size_t pool_blocks, skv_layer *const *layers,
                       size_t n_layers, skv_hot **out) try {
    if (!out) return fail(SKV_ERR_DEVICE, "hot_create: out nul");
    *out = nullptr;
    int32_t rc = check_layers(ctx, layers, n_layers);
    if (rc) return rc;
    if (block_tokens == 0 || block_tokens % 16 != 0)
        return fail(SKV_ERR_CONFIG, "prefix-cache GPU: block_tokens doit être un multiple de 16");
    SKV_HIP(hipSetDevice(ctx->device));
    skv_hot *h = new skv_hot();
    h->ctx = ctx;
    h->index = new PrefixIndex(block_tokens, capacity_blocks, blocks_per_session);
    h->pages_per_block = block_tokens / 16;
    h->pool_slots = pool_blocks * h->pages_per_block;
    h->layout.build(layers, n_layers, h->pool_slots, true);
    const size_t bytes = h->pool_slots * h->layout.slot_bytes;
    if (bytes) {
        hipError_t e = hipMalloc((void **)&h->pool, bytes);
        if (e != hipSuccess) {
            delete h->index;
            delete h;
            return fail_hip(e, "hot_create: allocation du pool");
        }
    }
    h->free_slots.reserve(h->pool_slots);
    for (size_t i = h->pool_slots; i-- > 0;) h->free_slots.push_back((int32_t)i);
    *out = h;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

void skv_hot_destroy(skv_hot *h) {
    if (!h) return;
    (void)hipSetDevice(h->ctx->device);
    (void)hipDeviceSynchronize();
    for (auto &kv : h->entries)
        if (kv.second.state) skv_snapshot_free(kv.second.state);
    for (skv_snapshot *sp : h->spare_states) skv_snapshot_free(sp);
    if (h->pool) (void)hipFree(h->pool);
    delete h->index;
    delete h;
}

size_t skv_hot_block_tokens(const skv_hot *h) { return h ? h->index->block_tokens() : 0; }
size_t skv_hot_len(const skv_hot *h) { return h ? h->index->len() : 0; }
size_t skv_hot_bytes(const skv_hot *h) { return h ? h->index->bytes() : 0; }
size_t skv_hot_free_blocks(const skv_hot *h) { return h ? h->free_slots.size() / h->pages_per_block : 0; }
size_t skv_hot_pool_blocks(const skv_hot *h) { return h ? h->pool_slots / h->pages_per_block : 0; }
size_t skv_hot_block_bytes(const skv_hot *h) { return h ? h->pages_per_block * h->layout.slot_bytes : 0; }
uint64_t skv_hot_evictions(const skv_hot *h) { return h ? h->evictions : 0; }
uint64_t skv_hot_skipped(const skv_hot *h) { return h ? h->skipped : 0; }

int32_t skv_hot_entry(const skv_hot *h, size_t index, uint8_t session[32], uint8_t hash[32],
                      size_t *tokens, size_t *bytes) try {
    if (!h) return fail(SKV_ERR_DEVICE, "hot_entry: pointeur nul");
    if (!h->index->entry(index, session, hash, tokens, nullptr, bytes))
        return fail(SKV_ERR_DIMENSION, "hot_entry: index " + std::to_string(index) + " hors plage");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_hot_evict_lru(skv_hot *h, int32_t *found, size_t *bytes) try {
    if (!h || !found) return fail(SKV_ERR_DEVICE, "hot_evict_lru: pointeur nul");
    uint64_t id = 0;
    const bool ok = h->index->evict_lru(&id, bytes);
    *found = ok ? 1 : 0;
    if (ok) {
        hot_release(h, id);
        ++h->evictions;
    }
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

// remember_prefix_block (src/serve/state.rs:613-639): snapshot the block that ends at
// `tokens`, evict least-recent blocks while the pool has no room, then insert. When nothing
// is left to evict the block is skipped without an error (*cached = 0).
int32_t skv_hot_remember(skv_hot *h, skv_stream stream, const uint8_t session[32],
                         const uint8_t hash[32], size_t tokens, skv_layer *const *layers,
                         size_t n_layers, const void *const *state_ptrs, const size_t *state_bytes,
                         size_t n_states, int32_t *cached) try {
    if (!h || !session || !hash || !cached) return fail(SKV_ERR_DEVICE, "hot_remember: pointeur nul");
    *cached = 0;
    int32_t rc = check_layers(h->ctx, layers, n_layers);
    if (rc) return rc;
    if (!h->layout.matches(layers, n_layers))
        return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: les couches n'ont pas la forme du pool");
    const size_t bt = h->index->block_tokens();
    if (tokens < bt || tokens % bt != 0)
        return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: tokens=" + std::to_string(tokens) +
                                           " n'est pas une frontière de bloc");
    for (size_t l = 0; l < n_layers; ++l) {
        if (layers[l]->len < tokens)
            return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: couche plus courte que la frontière");
        if (layers[l]->g.ring_rows > 0 && tokens - bt < layers[l]->floor_pos)
            return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: bloc déjà évincé de l'anneau");
    }
    if (h->index->capacity() == 0) return SKV_OK; // insert() of a disabled cache stores nothing
    SKV_HIP(hipSetDevice(h->ctx->device));
    while (h->free_slots.size() < h->pages_per_block) {
        uint64_t id = 0;
        if (!h->index->evict_lru(&id, nullptr)) {
            ++h->skipped;
            return SKV_OK; // nothing left to evict: skip caching, no error
        }
        hot_release(h, id);
        ++h->evictions;
    }
    HotEntry e;
    std::vector<int32_t> pages(h->pages_per_block);
    for (size_t i = 0; i < h->pages_per_block; ++i) {
        e.slots.push_back(h->free_slots.back());
        h->free_slots.pop_back();
        pages[i] = (int32_t)((tokens - bt) / 16 + i);
    }
    rc = copy_pages(h->layout, h->pool, layers, n_layers, pages.data(), e.slots.data(),
                    h->pages_per_block, nullptr, true, as_stream(stream));
    if (!rc && n_states) {
        // a spare buffer of the same shapes, if an eviction left one
        for (size_t i = 0; i < h->spare_states.size() && !e.state; ++i) {
            skv_snapshot *sp = h->spare_states[i];
            if (sp->sizes.size() == n_states && state_bytes && std::equal(sp->sizes.begin(), sp->sizes.end(), state_bytes)) {
                e.state = sp;
                h->spare_states.erase(h->spare_states.begin() + (long)i);
            }
        }
        if (e.state) {
            bool ok = state_ptrs != nullptr;
            std::vector<void *> dst(n_states);
            for (size_t i = 0; i < n_states && ok; ++i) {
                ok = state_ptrs[i] != nullptr;
                dst[i] = e.state->base + e.state->offsets[i];
            }
            rc = ok ? launch_flat(state_ptrs, dst.data(), state_bytes, n_states, as_stream(stream))
                    : fail(SKV_ERR_DEVICE, "state_snapshot: pointeur nul");
            if (rc) {
                h->spare_states.push_back(e.state);
                e.state = nullptr;
            }
        } else {
            rc = skv_state_snapshot(h->ctx, stream, state_ptrs, state_bytes, n_states, &e.state);
        }
    }
    if (rc) {
        for (int32_t s : e.slots) h->free_slots.push_back(s);
        return rc;
    }
    e.bytes = h->pages_per_block * h->layout.slot_bytes + (e.state ? e.state->bytes : 0);
    const uint64_t id = h->next_id++;
    const size_t nbytes = e.bytes;
    h->entries.emplace(id, std::move(e));
    std::vector<uint64_t> dropped;
    h->index->insert(session, hash, tokens, id, nbytes, &dropped);
    for (uint64_t d : dropped) {
        if (d != id) ++h->evictions;
        hot_release(h, d);
    }
    *cached = h->entries.count(id) ? 1 : 0;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

// remember_prefix_block for `n_blocks` consecutive boundaries in one call: block i covers
// rows [first_tokens - block_tokens + i*block_tokens, first_tokens + i*block_tokens) and is
// keyed by hashes[i]. Same evictions and insertions, in the same order, as n_blocks separate
// calls; the page copies of all blocks are queued together. For caches without recurrent
// state (a state exists only at the boundary the decoder is at).
int32_t skv_hot_remember_range(skv_hot *h, skv_stream stream, const uint8_t session[32],
                               const uint8_t *hashes, size_t first_tokens, size_t n_blocks,
                               skv_layer *const *layers, size_t n_layers, size_t *n_cached) try {
    if (!h || !session || (n_blocks && !hashes)) return fail(SKV_ERR_DEVICE, "hot_remember_range: pointeur nul");
    if (n_cached) *n_cached = 0;
    int32_t rc = check_layers(h->ctx, layers, n_layers);
    if (rc) return rc;
    if (!h->layout.matches(layers, n_layers))
        return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: les couches n'ont pas la forme du pool");
    const size_t bt = h->index->block_tokens();
    if (n_blocks == 0) return SKV_OK;
    if (first_tokens < bt || first_tokens % bt != 0)
        return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: tokens=" + std::to_string(first_tokens) +
                                           " n'est pas une frontière de bloc");
    const size_t last_tokens = first_tokens + (n_blocks - 1) * bt;
    for (size_t l = 0; l < n_layers; ++l) {
        if (layers[l]->len < last_tokens)
            return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: couche plus courte que la frontière");
        if (layers[l]->g.ring_rows > 0 && first_tokens - bt < layers[l]->floor_pos)
            return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: bloc déjà évincé de l'anneau");
    }
    if (h->index->capacity() == 0) return SKV_OK;
    SKV_HIP(hipSetDevice(h->ctx->device));
    std::vector<int32_t> pages, slots;
    std::vector<char> pending(h->pool_slots, 0); // slots written by copies not yet queued
    auto flush = [&]() -> int32_t {
        if (pages.empty()) return SKV_OK;
        int32_t r = copy_pages(h->layout, h->pool, layers, n_layers, pages.data(), slots.data(),
                               pages.size(), nullptr, true, as_stream(stream));
        for (int32_t sl : slots) pending[sl] = 0;
        pages.clear();
        slots.clear();
        return r;
    };
    size_t cached = 0;
    // The copies go out in growing batches while the host is still inserting the later
    // blocks into the index, as in skv_hot_match_restore.
    size_t batch_pages = 16;
    for (size_t b = 0; b < n_blocks; ++b) {
        const size_t tokens = first_tokens + b * bt;
        if (pages.size() >= batch_pages) {
            rc = flush();
            if (rc) return rc;
            batch_pages = std::min<size_t>(batch_pages * 5 / 2, COPY_MAX_PAGES);
        }
        bool skipped = false;
        while (h->free_slots.size() < h->pages_per_block) {
            uint64_t id = 0;
            if (!h->index->evict_lru(&id, nullptr)) {
                ++h->skipped;
                skipped = true;
                break;
            }
            hot_release(h, id);
            ++h->evictions;
        }
        if (skipped) continue;
        HotEntry e;
        bool reuse = false;
        for (size_t i = 0; i < h->pages_per_block; ++i) {
            const int32_t sl = h->free_slots.back();
            h->free_slots.pop_back();
            e.slots.push_back(sl);
            reuse = reuse || pending[sl];
        }
        if (reuse) { // a slot freed by an eviction inside this call: its old copy goes first
            rc = flush();
            if (rc) return rc;
        }
        for (size_t i = 0; i < h->pages_per_block; ++i) {
            pages.push_back((int32_t)((tokens - bt) / 16 + i));
            slots.push_back(e.slots[i]);
            pending[e.slots[i]] = 1;
        }
        e.bytes = h->pages_per_block * h->layout.slot_bytes;
        const uint64_t id = h->next_id++;
        const size_t nbytes = e.bytes;
        h->entries.emplace(id, std::move(e));
        std::vector<uint64_t> dropped;
        h->index->insert(session, hashes + 32 * b, tokens, id, nbytes, &dropped);
        for (uint64_t d : dropped) {
            if (d != id) ++h->evictions;
            hot_release(h, d);
        }
        if (h->entries.count(id)) ++cached;
    }
    rc = flush();
    if (rc) return rc;
    if (n_cached) *n_cached = cached;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

// The hit branch of prefill_prompt_state (src/serve/state.rs:574-584): longest chain of
// cached blocks for `tokens`, every matched block's pages copied into the layers' rows
// [0, reused), the recurrent state of the last matched block copied out, len = reused.
int32_t skv_hot_match_restore(skv_hot *h, skv_stream stream, const uint8_t root[32],
                              const uint64_t *tokens, size_t n_tokens, skv_layer *const *layers,
                              size_t n_layers, void *const *state_ptrs, const size_t *state_bytes,
                              size_t n_states, size_t *reused_tokens, uint8_t hash_out[32]) try {
    if (!h || !root || !reused_tokens || (n_tokens && !tokens))
        return fail(SKV_ERR_DEVICE, "hot_match_restore: pointeur nul");
    *reused_tokens = 0;
    int32_t rc = check_layers(h->ctx, layers, n_layers);
    if (rc) return rc;
    if (!h->layout.matches(layers, n_layers))
        return fail(SKV_ERR_DIMENSION, "prefix-cache GPU: les couches n'ont pas la forme du pool");
    size_t min_capacity = (size_t)-1;
    bool any_ring = false;
    for (size_t l = 0; l < n_layers; ++l) {
        min_capacity = std::min(min_capacity, layers[l]->capacity);
        any_ring = any_ring || layers[l]->g.ring_rows > 0;
    }
    SKV_HIP(hipSetDevice(h->ctx->device));
    // The chain of SHA-256 digests is inherently serial on the host (about 0.3 us per
    // block); the walk therefore proceeds in growing batches and the pages of each batch
    // are put in flight while the next one is being hashed. Ring layers need the final
    // length to know which rows still fit, so for them the walk finishes first.
    PrefixHit hit{};
    std::vector<uint64_t> chain;
    PrefixIndex::Walk walk;
    h->index->match_start(&walk, root);
    std::vector<int32_t> pages, slots;
    size_t done_blocks = 0; // blocks whose copies have been queued
    size_t batch = any_ring ? (size_t)-1 : 16;
    const size_t bt = h->index->block_tokens();
    // Once the first batch of copies is queued the layers' rows are being overwritten: an
    // error after that point leaves every layer empty (len 0) rather than with its old length
    // over rows that are no longer its own.
    auto fail_emptied = [&](int32_t code) {
        if (done_blocks > 0)
            for (size_t l = 0; l < n_layers; ++l) {
                layers[l]->len = 0;
                layers[l]->floor_pos = 0;
            }
        return code;
    };
    for (;;) {
        const size_t got = h->index->match_more(&walk, root, tokens, n_tokens, batch, &hit, &chain);
        if (chain.size() * bt > min_capacity)
            return fail_emptied(fail(SKV_ERR_DIMENSION, "seed KV " + std::to_string(chain.size() * bt) +
                                                            " > capacité " + std::to_string(min_capacity)));
        if (got == 0) break;
        if (!any_ring) {
            pages.clear();
            slots.clear();
            for (size_t b = done_blocks; b < chain.size(); ++b) {
                const HotEntry &e = h->entries.at(chain[b]);
                for (size_t i = 0; i < e.slots.size(); ++i) {
                    pages.push_back((int32_t)(b * h->pages_per_block + i));
                    slots.push_back(e.slots[i]);
                }
            }
            rc = copy_pages(h->layout, h->pool, layers, n_layers, pages.data(), slots.data(),
                            pages.size(), nullptr, false, as_stream(stream));
            done_blocks = chain.size();
            if (rc) return fail_emptied(rc);
            // Hashing a block takes about 0.29 us, copying it (Qwen3-4B shape) about 0.72 us plus
            // 6 us per launch: a batch four times the last is hashed while the last is copied, and
            // a 4096-token prefix goes out in three launches (16, 64, 176 blocks).
            batch = std::min<size_t>(batch * 4, COPY_MAX_PAGES);
        }
        if (!walk.alive) break;
    }
    if (chain.empty()) return SKV_OK;
    const HotEntry &last = h->entries.at(chain.back());
    if (n_states && !last.state)
        return fail_emptied(fail(SKV_ERR_DIMENSION, "prefix-cache: snapshots=0 couches=" + std::to_string(n_states)));
    const size_t reused = hit.tokens;
    std::vector<uint32_t> first_page(n_layers, 0);
    if (any_ring) {
        for (size_t b = 0; b < chain.size(); ++b) {
            const HotEntry &e = h->entries.at(chain[b]);
            for (size_t i = 0; i < e.slots.size(); ++i) {
                pages.push_back((int32_t)(b * h->pages_per_block + i));
                slots.push_back(e.slots[i]);
            }
        }
        for (size_t l = 0; l < n_layers; ++l) {
            const skv_layer *L = layers[l];
            if (L->g.ring_rows > 0 && reused > (size_t)L->g.ring_rows)
                first_page[l] = (uint32_t)((reused - (size_t)L->g.ring_rows + 15) / 16);
        }
        rc = copy_pages(h->layout, h->pool, layers, n_layers, pages.data(), slots.data(), pages.size(),
                        first_page.data(), false, as_stream(stream));
        done_blocks = chain.size();
        if (rc) return fail_emptied(rc);
    }
    if (n_states) {
        rc = skv_state_restore(h->ctx, stream, last.state, state_ptrs, state_bytes, n_states);
        if (rc) return fail_emptied(rc);
    }
    for (size_t l = 0; l < n_layers; ++l) {
        skv_layer *L = layers[l];
        L->len = reused;
        L->floor_pos = (size_t)first_page[l] * 16;
    }
    *reused_tokens = reused;
    if (hash_out) std::memcpy(hash_out, hit.hash, 32);
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

// ---- the decoder's own whole-prompt cache ---------------------------------------------------
// prefix_cache_get / prefix_cache_put (src/decoder/generation.rs:2998-3025, 3105-3139): a few
// whole prompts (RETI_RUST_PREFIX_CACHE_CAP, default 4), newest first, each with the K/V rows of
// every layer and the model's opaque state buffers (final hidden state, recurrent states); a
// request whose prompt starts with a cached prompt resumes from the longest such entry. An
// entry here is a block snapshot of the prompt's pages plus a state snapshot; a hit copies them
// into the caller's layers, so what the caller then appends never touches the entry (the
// reference clones for the same reason, generation.rs:3009).
} // extern "C"

struct PromptEntry {
    std::vector<uint64_t> tokens;
    // per layer: logical pages below this one are not in the snapshot (a ring layer whose
    // prompt was longer than the ring no longer held them; the reference clones the whole
    // cache, generation.rs:3105-3139, but its sliding layers never attend those rows again)
    std::vector<uint32_t> first_page;
    skv_snapshot *pages = nullptr;
    skv_snapshot *state = nullptr;
    size_t bytes = 0;
};

struct skv_prompt_cache {
    CtxRef ctx;
    size_t capacity = 0;
    std::vector<PromptEntry> entries; // index 0 = most recent
};

static void prompt_entry_free(PromptEntry &e) {
    skv_snapshot_free(e.pages);
    skv_snapshot_free(e.state);
    e.pages = e.state = nullptr;
}

// longest_prefix_entry_index (src/decoder/generation.rs:190-204): the first of the longest
// entries whose tokens the prompt starts with; -1 = none (an empty entry never matches).
static long longest_prefix_entry_index(const std::vector<PromptEntry> &entries, const uint64_t *prompt, size_t n) {
    long best = -1;
    size_t best_len = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
        const std::vector<uint64_t> &t = entries[i].tokens;
        if (t.size() > best_len && t.size() <= n && std::equal(t.begin(), t.end(), prompt)) {
            best = (long)i;
            best_len = t.size();
        }
    }
    return best;
}

extern "C" {

int32_t skv_prompt_cache_create(skv_ctx *ctx, size_t capacity, skv_prompt_cache **out) try {
    if (!ctx || !out) return fail(SKV_ERR_DEVICE, "prompt_cache_create: pointeur nul");
    skv_prompt_cache *c = new skv_prompt_cache();
    c->ctx = ctx;
    c->capacity = capacity;
    *out = c;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prompt_cache_from_runtime_flags(skv_ctx *ctx, skv_prompt_cache **out) try {
    // RETI_RUST_PREFIX_CACHE=0 switches the cache off (generation.rs:2781-2784): capacity 0
    return skv_prompt_cache_create(ctx, skv_flag_prefix_cache_enabled() ? skv_flag_prefix_cache_capacity() : 0, out);
} catch (...) {
    return skv::fail_exception();
}

void skv_prompt_cache_destroy(skv_prompt_cache *c) {
    if (!c) return;
    for (PromptEntry &e : c->entries) prompt_entry_free(e);
    delete c;
}

size_t skv_prompt_cache_len(const skv_prompt_cache *c) { return c ? c->entries.size() : 0; }
size_t skv_prompt_cache_capacity(const skv_prompt_cache *c) { return c ? c->capacity : 0; }
size_t skv_prompt_cache_bytes(const skv_prompt_cache *c) {
    size_t b = 0;
    if (c)
        for (const PromptEntry &e : c->entries) b += e.bytes;
    return b;
}

int32_t skv_prompt_cache_entry(const skv_prompt_cache *c, size_t index, size_t *n_tokens, uint64_t *tokens_out,
                               size_t tokens_cap) try {
    if (!c || !n_tokens) return fail(SKV_ERR_DEVICE, "prompt_cache_entry: pointeur nul");
    if (index >= c->entries.size()) return fail(SKV_ERR_DIMENSION, "prompt_cache_entry: indice hors plage");
    const std::vector<uint64_t> &t = c->entries[index].tokens;
    *n_tokens = t.size();
    if (tokens_out) std::copy(t.begin(), t.begin() + std::min(tokens_cap, t.size()), tokens_out);
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prompt_cache_put(skv_prompt_cache *c, skv_stream stream, const uint64_t *tokens, size_t n_tokens,
                             skv_layer *const *layers, size_t n_layers, const void *const *state_ptrs,
                             const size_t *state_bytes, size_t n_states) try {
    if (!c || (n_tokens && !tokens)) return fail(SKV_ERR_DEVICE, "prompt_cache_put: pointeur nul");
    if (c->capacity == 0) return SKV_OK;
    int32_t rc = check_layers(c->ctx, layers, n_layers);
    if (rc) return rc;
    for (size_t l = 0; l < n_layers; ++l)
        if (layers[l]->len != n_tokens)
            return fail(SKV_ERR_DIMENSION, "prompt_cache_put: la couche " + std::to_string(l) + " tient " +
                                               std::to_string(layers[l]->len) + " lignes pour un prompt de " +
                                               std::to_string(n_tokens));
    // the snapshots first: a failure leaves the cache as it was
    PromptEntry e;
    e.tokens.assign(tokens, tokens + n_tokens);
    const size_t n_blocks = (n_tokens + 15) / 16;
    // a ring layer holds positions floor_pos .. len-1: its whole pages from the first one that
    // starts at or after floor_pos (the page that straddles floor_pos already holds newer rows
    // in its low slots; its surviving rows lie behind every window the layer can still serve
    // as long as the ring keeps 16 rows or more behind the window)
    e.first_page.assign(n_layers, 0);
    for (size_t l = 0; l < n_layers; ++l)
        if (layers[l]->g.ring_rows > 0) e.first_page[l] = (uint32_t)((layers[l]->floor_pos + 15) / 16);
    {
        SKV_HIP(hipSetDevice(c->ctx->device));
        skv_snapshot *snap = new skv_snapshot();
        snap->ctx = c->ctx;
        snap->layout.build(layers, n_layers, n_blocks, true);
        snap->n_pages = n_blocks;
        snap->bytes = n_blocks * snap->layout.slot_bytes;
        if (snap->bytes) {
            hipError_t he = hipMalloc((void **)&snap->base, snap->bytes);
            if (he != hipSuccess) {
                delete snap;
                return fail_hip(he, "prompt_cache_put: allocation");
            }
            std::vector<int32_t> pages(n_blocks), slots(n_blocks);
            for (size_t i = 0; i < n_blocks; ++i) pages[i] = slots[i] = (int32_t)i;
            rc = copy_pages(snap->layout, snap->base, layers, n_layers, pages.data(), slots.data(), n_blocks,
                            e.first_page.data(), true, as_stream(stream));
            if (rc) {
                skv_snapshot_free(snap);
                return rc;
            }
        }
        e.pages = snap;
    }
    rc = skv_state_snapshot(c->ctx, stream, state_ptrs, state_bytes, n_states, &e.state);
    if (rc) {
        prompt_entry_free(e);
        return rc;
    }
    e.bytes = skv_snapshot_bytes(e.pages) + skv_snapshot_bytes(e.state);
    for (size_t i = 0; i < c->entries.size(); ++i) {
        if (c->entries[i].tokens == e.tokens) {
            prompt_entry_free(c->entries[i]);
            c->entries.erase(c->entries.begin() + (long)i);
            break;
        }
    }
    c->entries.insert(c->entries.begin(), std::move(e));
    while (c->entries.size() > c->capacity) {
        prompt_entry_free(c->entries.back());
        c->entries.pop_back();
    }
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prompt_cache_get(skv_prompt_cache *c, skv_stream stream, const uint64_t *prompt, size_t n_prompt,
                             skv_layer *const *layers, size_t n_layers, void *const *state_ptrs,
                             const size_t *state_bytes, size_t n_states, size_t *cached_tokens) try {
    if (!c || !cached_tokens || (n_prompt && !prompt)) return fail(SKV_ERR_DEVICE, "prompt_cache_get: pointeur nul");
    *cached_tokens = 0;
    const long index = longest_prefix_entry_index(c->entries, prompt, n_prompt);
    if (index < 0) return SKV_OK;
    int32_t rc = check_layers(c->ctx, layers, n_layers);
    if (rc) return rc;
    const PromptEntry &hit = c->entries[(size_t)index];
    const size_t cached = hit.tokens.size();
    // every check before the first copy is queued: a failure leaves the layers untouched
    for (size_t l = 0; l < n_layers; ++l)
        if (layers[l]->capacity < cached)
            return fail(SKV_ERR_DIMENSION, "prompt_cache_get: capacité " + std::to_string(layers[l]->capacity) +
                                               " < préfixe en cache " + std::to_string(cached));
    if (hit.state && n_states != hit.state->sizes.size())
        return fail(SKV_ERR_DIMENSION, "prefix-cache: snapshots=" + std::to_string(hit.state->sizes.size()) +
                                           " couches=" + std::to_string(n_states));
    for (size_t i = 0; i < n_states; ++i)
        if (!state_ptrs || !state_bytes || state_bytes[i] != hit.state->sizes[i])
            return fail(SKV_ERR_DIMENSION, "prompt_cache_get: taille du tampon d'état " + std::to_string(i) + " différente");
    const size_t n_blocks = hit.pages ? hit.pages->n_pages : 0;
    if (n_blocks && (hit.first_page.size() != n_layers || !hit.pages->layout.matches(layers, n_layers)))
        return fail(SKV_ERR_DIMENSION, "prefix-cache: snapshots=" + std::to_string(hit.first_page.size()) +
                                           " couches=" + std::to_string(n_layers) + " ou formes différentes");
    // where each layer's restored pages start: what the entry holds, and no more than the
    // destination's own ring can take
    std::vector<uint32_t> first_page(n_layers, 0);
    for (size_t l = 0; l < n_layers && n_blocks; ++l) {
        const skv_layer *L = layers[l];
        first_page[l] = hit.first_page[l];
        if (L->g.ring_rows == 0) {
            if (first_page[l] > 0)
                return fail(SKV_ERR_DIMENSION, "prompt_cache_get: l'entrée ne tient que la fenêtre de la couche " +
                                                   std::to_string(l) + ", la couche de destination n'est pas un anneau");
        } else if (cached > (size_t)L->g.ring_rows) {
            first_page[l] = std::max(first_page[l], (uint32_t)((cached - (size_t)L->g.ring_rows + 15) / 16));
        }
    }
    if (n_blocks) {
        SKV_HIP(hipSetDevice(c->ctx->device));
        std::vector<int32_t> pages(n_blocks), slots(n_blocks);
        for (size_t i = 0; i < n_blocks; ++i) pages[i] = slots[i] = (int32_t)i;
        rc = copy_pages(hit.pages->layout, hit.pages->base, layers, n_layers, pages.data(), slots.data(), n_blocks,
                        first_page.data(), false, as_stream(stream));
        if (rc) return rc;
    }
    rc = skv_state_restore(c->ctx, stream, hit.state, state_ptrs, state_bytes, n_states);
    if (rc) return rc;
    for (size_t l = 0; l < n_layers; ++l) {
        layers[l]->len = cached;
        layers[l]->floor_pos = (size_t)first_page[l] * 16;
    }
    // the hit becomes the most recent entry (generation.rs:3007-3012)
    if (index > 0) std::rotate(c->entries.begin(), c->entries.begin() + index, c->entries.begin() + index + 1);
    *cached_tokens = cached;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

} // extern "C"
