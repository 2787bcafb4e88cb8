// Runtime kill-switches of the KV path, read from the environment like the
// reference does (src/runtime_flags.rs:25-44; src/decode_resident/utils.rs:182-286).
// Each getter is frozen at its first read; skv_flags_reload() drops the frozen
// values and exists for tests only.
#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <optional>
#include <string>

#include "skv_internal.h"

namespace {

std::mutex g_mu;
uint64_t g_epoch = 1;

std::string trim(const char *s) {
    std::string v(s ? s : "");
    size_t b = 0, e = v.size();
    while (b < e && std::isspace((unsigned char)v[b])) ++b;
    while (e > b && std::isspace((unsigned char)v[e - 1])) --e;
    return v.substr(b, e - b);
}

bool ieq(const std::string &a, const char *b) {
    if (a.size() != std::strlen(b)) return false;
    for (size_t i = 0; i < a.size(); ++i)
        if (std::tolower((unsigned char)a[i]) != b[i]) return false;
    return true;
}

// env_flag_value (src/runtime_flags.rs:32-44)
std::optional<bool> flag_value(const char *raw) {
    const std::string v = trim(raw);
    if (v == "1" || ieq(v, "true") || ieq(v, "on")) return true;
    if (v == "0" || ieq(v, "false") || ieq(v, "off")) return false;
    return std::nullopt;
}

bool env_flag(const char *name, bool dflt) {
    const char *raw = std::getenv(name);
    if (!raw) return dflt;
    return flag_value(raw).value_or(dflt);
}

// value.trim().parse::<usize>().ok(): decimal digits only (an optional leading '+').
std::optional<size_t> parse_usize(const char *raw, bool do_trim) {
    if (!raw) return std::nullopt;
    std::string v = do_trim ? trim(raw) : std::string(raw);
    size_t i = 0;
    if (!v.empty() && v[0] == '+') i = 1;
    if (i >= v.size()) return std::nullopt;
    size_t out = 0;
    for (; i < v.size(); ++i) {
        if (v[i] < '0' || v[i] > '9') return std::nullopt;
        size_t d = (size_t)(v[i] - '0');
        if (out > (SIZE_MAX - d) / 10) return std::nullopt;
        out = out * 10 + d;
    }
    return out;
}

template <typename T> struct Once {
    uint64_t epoch = 0;
    T value{};
    template <typename F> T get(F f) {
        std::lock_guard<std::mutex> lk(g_mu);
        if (epoch != g_epoch) {
            value = f();
            epoch = g_epoch;
        }
        return value;
    }
};

Once<int> f_flash, f_2pass, f_res_full, f_res, f_serve_prefix, f_prefix, f_kv_bf16, f_sim_k, f_sim_v, f_pipeline,
    f_mem_guard, f_oom_guard;
Once<size_t> f_2pass_min, f_block_tokens, f_cache_blocks, f_per_session, f_prefix_cap, f_chunk, f_par_threshold,
    f_split_min;
Once<uint64_t> f_mem_cap, f_mem_headroom, f_serve_cap, f_serve_headroom;

// `.ok().and_then(|value| value.trim().parse::<u64>().ok())`
std::optional<uint64_t> env_u64(const char *name) {
    auto v = parse_usize(std::getenv(name), true);
    return v.has_value() ? std::optional<uint64_t>((uint64_t)*v) : std::nullopt;
}

} // namespace

extern "C" {

int32_t skv_env_flag(const char *name, int32_t default_value) {
    return env_flag(name, default_value != 0) ? 1 : 0;
}

int32_t skv_env_flag_value(const char *value) {
    auto v = flag_value(value);
    return v.has_value() ? (*v ? 1 : 0) : -1;
}

int32_t skv_flag_kv_bf16_for(int32_t sampled) {
    // -1 = no override
    int ov = f_kv_bf16.get([] {
        const char *raw = std::getenv("RETI_RUST_KV_BF16");
        if (!raw) return -1;
        auto v = flag_value(raw);
        return v.has_value() ? (*v ? 1 : 0) : -1;
    });
    return ov >= 0 ? ov : (sampled != 0);
}

int32_t skv_flag_flash_sdpa_enabled(void) {
    return f_flash.get([] { return (int)env_flag("RETI_RUST_FLASH_SDPA", true); });
}
int32_t skv_flag_sdpa_2pass_enabled(void) {
    return f_2pass.get([] { return (int)env_flag("RETI_RUST_SDPA_2PASS", true); });
}
size_t skv_flag_sdpa_2pass_min_len(void) {
    // `.and_then(|value| value.parse().ok())`: no trim here in the reference.
    return f_2pass_min.get([] {
        return parse_usize(std::getenv("RETI_RUST_SDPA_2PASS_MIN_LEN"), false).value_or(2048);
    });
}
size_t skv_effective_split_min_len(void) {
    // The reference's default switch-over (2048 rows, src/decode_resident/utils.rs:270-278) was
    // tuned for Apple GPUs; an explicit RETI_RUST_SDPA_2PASS_MIN_LEN is honoured as it is, the
    // default here is 128 because one workgroup per kv head leaves most compute units idle.
    return f_split_min.get([] {
        const char *raw = std::getenv("RETI_RUST_SDPA_2PASS_MIN_LEN");
        return raw ? parse_usize(raw, false).value_or(2048) : (size_t)128;
    });
}
int32_t skv_flag_kv_bf16_sim_konly(void) {
    return f_sim_k.get([] { return (int)env_flag("RETI_RUST_KV_BF16_SIM_KONLY", false); });
}
int32_t skv_flag_kv_bf16_sim_vonly(void) {
    return f_sim_v.get([] { return (int)env_flag("RETI_RUST_KV_BF16_SIM_VONLY", false); });
}
size_t skv_flag_attention_par_threshold(void) {
    return f_par_threshold.get(
        [] { return parse_usize(std::getenv("RETI_RUST_ATTENTION_PAR_THRESHOLD"), true).value_or(128); });
}
int32_t skv_flag_decode_pipeline(void) {
    return f_pipeline.get([] { return (int)env_flag("RETI_RUST_DECODE_PIPELINE", true); });
}
size_t skv_sdpa_2pass_blocks(size_t len) {
    size_t raw = std::max<size_t>(len / 128, 1);
    size_t rounded = (raw + 31) / 32 * 32;
    return std::min<size_t>(std::max<size_t>(rounded, 32), 1024);
}
int32_t skv_flag_decode_resident_full(void) {
    return f_res_full.get([] { return (int)env_flag("RETI_RUST_DECODE_RESIDENT_FULL", true); });
}
int32_t skv_flag_decode_resident(void) {
    return f_res.get([] { return (int)env_flag("RETI_RUST_DECODE_RESIDENT", false); });
}
int32_t skv_flag_serve_prefix_cache_enabled(void) {
    return f_serve_prefix.get([] { return (int)env_flag("RETI_SERVE_PREFIX_CACHE", true); });
}
size_t skv_flag_serve_prefix_block_tokens(void) {
    return f_block_tokens.get([] {
        auto v = parse_usize(std::getenv("RETI_SERVE_PREFIX_BLOCK_TOKENS"), true);
        return (v.has_value() && *v > 0) ? *v : (size_t)256;
    });
}
size_t skv_flag_serve_prefix_cache_blocks(void) {
    return f_cache_blocks.get(
        [] { return parse_usize(std::getenv("RETI_SERVE_PREFIX_CACHE_BLOCKS"), true).value_or(128); });
}
size_t skv_flag_serve_prefix_blocks_per_session(void) {
    size_t dflt = skv_flag_serve_prefix_cache_blocks();
    return f_per_session.get([dflt] {
        return parse_usize(std::getenv("RETI_SERVE_PREFIX_BLOCKS_PER_SESSION"), true).value_or(dflt);
    });
}
int32_t skv_flag_prefix_cache_enabled(void) {
    return f_prefix.get([] { return (int)env_flag("RETI_RUST_PREFIX_CACHE", true); });
}
size_t skv_flag_prefix_cache_capacity(void) {
    return f_prefix_cap.get(
        [] { return parse_usize(std::getenv("RETI_RUST_PREFIX_CACHE_CAP"), true).value_or(4); });
}
int32_t skv_flag_memory_guard_enabled(void) {
    return f_mem_guard.get([] { return (int)env_flag("RETI_MEMORY_GUARD", true); });
}
int32_t skv_flag_serve_oom_guard_enabled(void) {
    // memory_guard_enabled() && env_flag("RETI_SERVE_OOM_GUARD", true)
    const int guard = skv_flag_memory_guard_enabled();
    return f_oom_guard.get([guard] { return (int)(guard && env_flag("RETI_SERVE_OOM_GUARD", true)); });
}
uint64_t skv_flag_memory_static_cap_bytes(void) {
    // Option<u64> with zero filtered out: 0 = no cap
    return f_mem_cap.get([] { return env_u64("RETI_MEMORY_CAP_BYTES").value_or(0); });
}
uint64_t skv_flag_memory_headroom_bytes(void) {
    return f_mem_headroom.get([] { return env_u64("RETI_MEMORY_HEADROOM_BYTES").value_or(2ull * 1024 * 1024 * 1024); });
}
uint64_t skv_flag_serve_memory_static_cap_bytes(void) {
    return f_serve_cap.get([] { return env_u64("RETI_SERVE_MEMORY_CAP_BYTES").value_or(0); });
}
uint64_t skv_flag_serve_memory_headroom_bytes(void) {
    return f_serve_headroom.get(
        [] { return env_u64("RETI_SERVE_MEMORY_HEADROOM_BYTES").value_or(2ull * 1024 * 1024 * 1024); });
}
size_t skv_flag_prefill_chunk(void) {
    return f_chunk.get([] {
        // the alias is consulted only when the first variable is absent, not when it fails to parse
        const char *raw = std::getenv("RETI_RUST_PREFILL_CHUNK");
        if (!raw) raw = std::getenv("RETI_RUST_PREFILL_STEP_SIZE");
        return parse_usize(raw, true).value_or(0);
    });
}

} // extern "C"

// Generation of the cached flag values: callers that cache their own environment-derived
// settings re-read them when it changes.
uint64_t skv_internal_flags_epoch() {
    std::lock_guard<std::mutex> lk(g_mu);
    return g_epoch;
}

extern "C" {

void skv_flags_reload(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    ++g_epoch;
}

size_t skv_window_start(size_t position, size_t window) {
    if (window == 0) return 0;
    return position + 1 > window ? position + 1 - window : 0;
}

int32_t skv_resident_capacity(size_t prefill_len, size_t max_new_tokens, size_t draft_headroom,
                              size_t *capacity) {
    size_t a = 0, b = 0;
    if (!capacity || __builtin_add_overflow(prefill_len, max_new_tokens, &a) ||
        __builtin_add_overflow(a, draft_headroom, &b))
        return 0;
    *capacity = b;
    return 1;
}

int32_t skv_resident_kv_bytes(size_t capacity, const size_t *kv_dims, size_t n_layers, size_t elem_bytes,
                              uint64_t *bytes) {
    // checked_bytes(&[2, capacity, kv_dim], size_of::<f32>()) summed with saturating_add
    // (src/decoder/resident/setup.rs:906-917); an overflowing product is the reference's
    // "KV résident déborde"
    if (!bytes || (n_layers && !kv_dims)) return 0;
    uint64_t total = 0;
    for (size_t i = 0; i < n_layers; ++i) {
        uint64_t b = 2;
        if (__builtin_mul_overflow(b, (uint64_t)capacity, &b) || __builtin_mul_overflow(b, (uint64_t)kv_dims[i], &b) ||
            __builtin_mul_overflow(b, (uint64_t)elem_bytes, &b))
            return 0;
        total = total > UINT64_MAX - b ? UINT64_MAX : total + b;
    }
    *bytes = total;
    return 1;
}

int32_t skv_memory_projection(uint64_t current, uint64_t reserved, uint64_t requested, uint64_t limit,
                              uint64_t *projected, uint64_t *available) {
    // projection_with_reserved + projection_over_limit (src/memory_guard.rs:334-362)
    auto sat = [](uint64_t a, uint64_t b) { return a > UINT64_MAX - b ? UINT64_MAX : a + b; };
    const uint64_t before = sat(current, reserved);
    const uint64_t proj = sat(before, requested);
    if (projected) *projected = proj;
    if (available) *available = limit > before ? limit - before : 0;
    return proj > limit ? 1 : 0;
}

uint16_t skv_f32_to_bf16_bits(float value) {
    uint32_t bits;
    std::memcpy(&bits, &value, 4);
    uint32_t lsb = (bits >> 16) & 1u;
    return (uint16_t)((bits + 0x7fffu + lsb) >> 16);
}

} // extern "C"
