// Host-side state of a context and of one layer's paged cache, shared by the entry points.
#pragma once

#include <vector>

#include "skv_internal.h"

using skv::Geom;

struct skv_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    void *mq_scratch = nullptr; // split-K partials of multi-query launches, grown on demand
    size_t mq_bytes = 0;
};

struct skv_layer {
    skv_ctx *ctx = nullptr;
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
};

// flags.cpp: generation counter of the cached runtime flags
uint64_t skv_internal_flags_epoch();
