// Host-side state of a context and of one layer's paged cache, shared by the entry points.
#pragma once

#include <atomic>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "skv_internal.h"

using skv::Geom;

struct skv_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    void *static_scratch = nullptr; // this device's copy of the library's static scratch array
    // Split-K partials of multi-query launches (chunked prefill), one buffer per stream the
    // context has seen such a launch on, grown on demand: launches on one stream are ordered by
    // it, launches on different streams never share a buffer. At most MQ_SCRATCH_STREAMS
    // entries: a caller that makes a stream per request would otherwise leave one buffer per
    // dead stream behind; past that the least recently used entry is dropped (after a device
    // synchronisation: its stream may no longer exist). The map is guarded by arena_mu; the
    // waits, frees and allocations happen outside it. Calls on ONE stream must come from one
    // thread at a time (as a stream's owner issues its work anyway).
    struct MqScratch {
        void *ptr = nullptr;
        size_t bytes = 0;
        uint64_t used = 0; // value of mq_clock at the last use
    };
    static constexpr size_t MQ_SCRATCH_STREAMS = 8;
    std::map<hipStream_t, MqScratch> mq_scratch;
    uint64_t mq_clock = 0;
    // Device buffers of destroyed layers, kept for the next layer that needs about as much:
    // the stand-in for the arena DecodeResidentState leases its buffers from
    // (src/decode_resident/arena.rs:116-211). A server creates and drops one cache per layer
    // and request; without this every request pays hundreds of allocations and frees.
    std::mutex arena_mu;
    std::multimap<size_t, void *> arena_free; // by size in bytes
    size_t arena_bytes = 0;                   // held in arena_free
    size_t arena_cap = 0;                     // most it may hold (SKV_ARENA_MAX_MB, default 4096)
    // One reference for the owner plus one per layer, rope table, snapshot and hot cache made
    // from the context: skv_ctx_destroy gives the context's device memory back and drops the
    // owner's reference, the struct itself goes with the last object that points at it, so a
    // binding whose finalisers run in any order never touches freed memory.
    std::atomic<int> refs{1};
    bool closed = false; // after skv_ctx_destroy: arena_put frees instead of keeping
};

namespace skv {
// A buffer of at least `bytes` from the context's arena (one whose size is within a quarter
// above the need) or from hipMalloc; *got is its real size, to hand back with arena_put.
hipError_t arena_get(skv_ctx *ctx, size_t bytes, void **ptr, size_t *got);
// Returns a buffer to the arena, or frees it when the arena is full. The caller has made
// sure the device no longer uses it.
void arena_put(skv_ctx *ctx, void *ptr, size_t bytes);
void ctx_release(skv_ctx *ctx);

// The context pointer of an object made from a context; holds one of its references.
class CtxRef {
  public:
    CtxRef() = default;
    CtxRef(const CtxRef &o) { *this = o.p_; }
    CtxRef &operator=(const CtxRef &o) { return *this = o.p_; }
    ~CtxRef() {
        if (p_) ctx_release(p_);
    }
    CtxRef &operator=(skv_ctx *c) {
        if (c) c->refs.fetch_add(1, std::memory_order_relaxed);
        if (p_) ctx_release(p_);
        p_ = c;
        return *this;
    }
    skv_ctx *operator->() const { return p_; }
    operator skv_ctx *() const { return p_; }

  private:
    skv_ctx *p_ = nullptr;
};
} // namespace skv

struct skv_layer {
    skv::CtxRef ctx;
    Geom g{};
    size_t capacity = 0;
    size_t len = 0;
    size_t window = 0;    // 0 = full cache
    size_t floor_pos = 0; // ring layers: oldest position still held
    int n_pages = 0;
    uint16_t *k_pool = nullptr;
    uint16_t *v_pool = nullptr;
    int32_t *table_dev = nullptr;
    std::vector<int32_t> table;
    // split-K partials
    int max_splits = 1;
    float *part_o = nullptr;
    float *part_m = nullptr;
    float *part_l = nullptr;
    // staging for the synchronous host entry points
    float *q_stage = nullptr;   // [q_dim]
    float *out_stage = nullptr; // [q_dim]
    float *kv_stage = nullptr;  // [2*kv_dim]
    float *scores = nullptr;    // plain kernel: [q_heads][capacity], allocated on first use
    size_t scores_cap = 0;
    std::vector<std::pair<void *, size_t>> leased; // buffers from the context's arena, with their sizes
};

// flags.cpp: generation counter of the cached runtime flags
uint64_t skv_internal_flags_epoch();
