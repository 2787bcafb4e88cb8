// Host side of the prefix hot cache: SHA-256 chained block keys and the LRU index,
// the stand-in for BlockHash and BlockAwarePrefixCache (src/serve/cache.rs:1-220).
//
// The reference keeps a Vec with index 0 = most recently used and scans it linearly.
// Here the same order lives in a doubly linked list with a hash map from
// (session, hash, tokens) to the list node, so lookup, touch and global eviction
// are O(1); every observable order (what a match leaves behind, which entry a
// per-session or global eviction removes) is the reference's.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <list>
#include <string>
#include <unordered_map>
#include <vector>

#include "prefix.h"

#if defined(__x86_64__)
#include <immintrin.h>
#endif

namespace skv {

// ---- SHA-256 (FIPS 180-4) ------------------------------------------------------------
namespace {

const uint32_t K256[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5,
    0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174,
    0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da,
    0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967,
    0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
    0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
    0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3,
    0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};

inline uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }

} // namespace

void Sha256::reset() {
    static const uint32_t H0[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a,
                                   0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    std::memcpy(h_, H0, sizeof(H0));
    len_ = 0;
    fill_ = 0;
}

#if defined(__x86_64__)
// One or more 64-byte blocks with the x86 SHA extensions (sha256rnds2 / sha256msg1 /
// sha256msg2), used when the host CPU has them. Same function as the portable code below;
// both are checked against FIPS 180-4 vectors.
__attribute__((target("sha,sse4.1,ssse3"))) static void sha256_blocks_ni(uint32_t state[8],
                                                                         const uint8_t *data) {
    const __m128i mask = _mm_set_epi64x(0x0c0d0e0f08090a0bLL, 0x0405060700010203LL);
    __m128i tmp = _mm_loadu_si128(reinterpret_cast<const __m128i *>(&state[0]));
    __m128i st1 = _mm_loadu_si128(reinterpret_cast<const __m128i *>(&state[4]));
    tmp = _mm_shuffle_epi32(tmp, 0xB1);              // CDAB
    st1 = _mm_shuffle_epi32(st1, 0x1B);              // EFGH
    __m128i st0 = _mm_alignr_epi8(tmp, st1, 8);      // ABEF
    st1 = _mm_blend_epi16(st1, tmp, 0xF0);           // CDGH
    const __m128i abef = st0, cdgh = st1;
    __m128i m[4];
    for (int i = 0; i < 4; ++i)
        m[i] = _mm_shuffle_epi8(_mm_loadu_si128(reinterpret_cast<const __m128i *>(data + 16 * i)), mask);
    for (int i = 0; i < 16; ++i) {
        const int cur = i & 3;
        __m128i msg = _mm_add_epi32(m[cur], _mm_loadu_si128(reinterpret_cast<const __m128i *>(&K256[4 * i])));
        st1 = _mm_sha256rnds2_epu32(st1, st0, msg);
        if (i >= 3 && i < 15) { // message words of the group after next
            const __m128i t = _mm_alignr_epi8(m[cur], m[(cur + 3) & 3], 4);
            m[(cur + 1) & 3] = _mm_sha256msg2_epu32(_mm_add_epi32(m[(cur + 1) & 3], t), m[cur]);
        }
        msg = _mm_shuffle_epi32(msg, 0x0E);
        st0 = _mm_sha256rnds2_epu32(st0, st1, msg);
        if (i >= 1 && i < 13) m[(cur + 3) & 3] = _mm_sha256msg1_epu32(m[(cur + 3) & 3], m[cur]);
    }
    st0 = _mm_add_epi32(st0, abef);
    st1 = _mm_add_epi32(st1, cdgh);
    tmp = _mm_shuffle_epi32(st0, 0x1B);              // FEBA
    st1 = _mm_shuffle_epi32(st1, 0xB1);              // DCHG
    st0 = _mm_blend_epi16(tmp, st1, 0xF0);           // DCBA
    st1 = _mm_alignr_epi8(st1, tmp, 8);              // HGFE
    _mm_storeu_si128(reinterpret_cast<__m128i *>(&state[0]), st0);
    _mm_storeu_si128(reinterpret_cast<__m128i *>(&state[4]), st1);
}

static bool have_sha_ni() {
    static const bool ok = [] {
        const char *force = std::getenv("SKV_SHA_PORTABLE");
        if (force && force[0] == '1') return false;
        return __builtin_cpu_supports("sha") && __builtin_cpu_supports("sse4.1") &&
               __builtin_cpu_supports("ssse3");
    }();
    return ok;
}
#endif

void Sha256::block(const uint8_t *p) {
#if defined(__x86_64__)
    if (have_sha_ni()) {
        sha256_blocks_ni(h_, p);
        return;
    }
#endif
    uint32_t w[64];
    for (int i = 0; i < 16; ++i)
        w[i] = ((uint32_t)p[4 * i] << 24) | ((uint32_t)p[4 * i + 1] << 16) |
               ((uint32_t)p[4 * i + 2] << 8) | (uint32_t)p[4 * i + 3];
    for (int i = 16; i < 64; ++i) {
        const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
        const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
        w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = h_[0], b = h_[1], c = h_[2], d = h_[3], e = h_[4], f = h_[5], g = h_[6], h = h_[7];
    for (int i = 0; i < 64; ++i) {
        const uint32_t S1 = rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25);
        const uint32_t ch = (e & f) ^ (~e & g);
        const uint32_t t1 = h + S1 + ch + K256[i] + w[i];
        const uint32_t S0 = rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22);
        const uint32_t mj = (a & b) ^ (a & c) ^ (b & c);
        const uint32_t t2 = S0 + mj;
        h = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
    }
    h_[0] += a; h_[1] += b; h_[2] += c; h_[3] += d; h_[4] += e; h_[5] += f; h_[6] += g; h_[7] += h;
}

void Sha256::update(const void *data, size_t n) {
    const uint8_t *p = static_cast<const uint8_t *>(data);
    len_ += n;
    if (fill_) {
        const size_t take = std::min(n, (size_t)64 - fill_);
        std::memcpy(buf_ + fill_, p, take);
        fill_ += take;
        p += take;
        n -= take;
        if (fill_ == 64) {
            block(buf_);
            fill_ = 0;
        }
    }
    while (n >= 64) {
        block(p);
        p += 64;
        n -= 64;
    }
    if (n) {
        std::memcpy(buf_, p, n);
        fill_ = n;
    }
}

void Sha256::finish(uint8_t out[32]) {
    const uint64_t bits = len_ * 8;
    uint8_t pad[72] = {0x80};
    const size_t padlen = (fill_ < 56 ? 56 : 120) - fill_;
    uint8_t lenb[8];
    for (int i = 0; i < 8; ++i) lenb[i] = (uint8_t)(bits >> (56 - 8 * i));
    update(pad, padlen);
    update(lenb, 8);
    for (int i = 0; i < 8; ++i) {
        out[4 * i] = (uint8_t)(h_[i] >> 24);
        out[4 * i + 1] = (uint8_t)(h_[i] >> 16);
        out[4 * i + 2] = (uint8_t)(h_[i] >> 8);
        out[4 * i + 3] = (uint8_t)h_[i];
    }
}

// BlockHash::chain (src/serve/cache.rs:36-46): SHA-256(prev32 || each token as u64 LE).
void hash_chain(const uint8_t prev[32], const uint64_t *tokens, size_t n, uint8_t out[32]) {
    Sha256 h;
    h.update(prev, 32);
#if defined(__BYTE_ORDER__) && __BYTE_ORDER__ == __ORDER_LITTLE_ENDIAN__
    h.update(tokens, n * sizeof(uint64_t)); // already u64 little-endian in memory
#else
    for (size_t i = 0; i < n; ++i) {
        uint8_t le[8];
        for (int b = 0; b < 8; ++b) le[b] = (uint8_t)(tokens[i] >> (8 * b));
        h.update(le, 8);
    }
#endif
    h.finish(out);
}

// ---- the index ------------------------------------------------------------------------
struct PrefixIndex::Impl {
    struct Key {
        uint8_t session[32];
        uint8_t hash[32];
        size_t tokens;
        bool operator==(const Key &o) const {
            return tokens == o.tokens && !std::memcmp(session, o.session, 32) &&
                   !std::memcmp(hash, o.hash, 32);
        }
    };
    struct KeyHash {
        size_t operator()(const Key &k) const {
            // the digest is already uniform: fold a few of its bytes with the session's
            uint64_t a, b;
            std::memcpy(&a, k.hash, 8);
            std::memcpy(&b, k.session + 8, 8);
            return (size_t)(a ^ (b * 0x9E3779B97F4A7C15ull) ^ (uint64_t)k.tokens);
        }
    };
    struct Node {
        Key key;
        uint64_t payload;
        size_t bytes;
    };
    struct SessionHash {
        size_t operator()(const std::string &s) const { return std::hash<std::string>()(s); }
    };
    std::list<Node> lru; // front = most recently used
    std::unordered_map<Key, std::list<Node>::iterator, KeyHash> map;
    std::unordered_map<std::string, size_t> per_session_count;

    static std::string skey(const uint8_t s[32]) { return std::string((const char *)s, 32); }

    void erase(std::list<Node>::iterator it) {
        auto c = per_session_count.find(skey(it->key.session));
        if (c != per_session_count.end() && --c->second == 0) per_session_count.erase(c);
        map.erase(it->key);
        lru.erase(it);
    }
};

PrefixIndex::PrefixIndex(size_t block_tokens, size_t capacity, size_t per_session)
    : block_tokens_(block_tokens < 1 ? 1 : block_tokens), capacity_(capacity),
      per_session_(per_session), impl_(new Impl()) {}

PrefixIndex::~PrefixIndex() { delete impl_; }

size_t PrefixIndex::len() const { return impl_->lru.size(); }

size_t PrefixIndex::bytes() const {
    size_t total = 0;
    for (const auto &n : impl_->lru) total += n.bytes;
    return total;
}

size_t PrefixIndex::session_block_count(const uint8_t session[32]) const {
    auto c = impl_->per_session_count.find(Impl::skey(session));
    return c == impl_->per_session_count.end() ? 0 : c->second;
}

// match_prefix (src/serve/cache.rs:121-151): walk whole blocks, stop at the first miss,
// move every hit to the front in walk order, report the last hit.
bool PrefixIndex::match(const uint8_t root[32], const uint64_t *tokens, size_t n, PrefixHit *hit,
                        std::vector<uint64_t> *chain) {
    if (chain) chain->clear();
    Walk w;
    match_start(&w, root);
    return match_more(&w, root, tokens, n, (size_t)-1, hit, chain) > 0;
}

void PrefixIndex::match_start(Walk *w, const uint8_t root[32]) const {
    std::memcpy(w->previous, root, 32);
    w->index = 0;
    w->alive = capacity_ != 0;
}

size_t PrefixIndex::match_more(Walk *w, const uint8_t root[32], const uint64_t *tokens, size_t n,
                               size_t max_blocks, PrefixHit *hit, std::vector<uint64_t> *chain) {
    if (!w->alive) return 0;
    const size_t blocks = n / block_tokens_; // chunks_exact
    size_t matched = 0;
    while (matched < max_blocks) {
        if (w->index >= blocks) {
            w->alive = false;
            break;
        }
        Impl::Key key;
        std::memcpy(key.session, root, 32);
        hash_chain(w->previous, tokens + w->index * block_tokens_, block_tokens_, key.hash);
        key.tokens = (w->index + 1) * block_tokens_;
        auto it = impl_->map.find(key);
        if (it == impl_->map.end()) {
            w->alive = false;
            break;
        }
        impl_->lru.splice(impl_->lru.begin(), impl_->lru, it->second); // remove + insert(0)
        const Impl::Node &node = *it->second;
        if (hit) {
            hit->tokens = node.key.tokens;
            std::memcpy(hit->hash, node.key.hash, 32);
            hit->payload = node.payload;
            hit->matched_blocks = w->index + 1;
        }
        if (chain) chain->push_back(node.payload);
        std::memcpy(w->previous, key.hash, 32);
        ++w->index;
        ++matched;
    }
    return matched;
}

// insert (src/serve/cache.rs:154-193). Payloads that leave the index (a replaced equal
// key, the session's least recent entry, the global least recent entry) go to `dropped`
// in that order.
size_t PrefixIndex::insert(const uint8_t session[32], const uint8_t hash[32], size_t tokens,
                           uint64_t payload, size_t bytes, std::vector<uint64_t> *dropped) {
    if (capacity_ == 0) {
        if (dropped) dropped->push_back(payload); // a disabled cache stores nothing: hand it back
        return 0;
    }
    Impl::Key key;
    std::memcpy(key.session, session, 32);
    std::memcpy(key.hash, hash, 32);
    key.tokens = tokens;
    auto it = impl_->map.find(key);
    if (it != impl_->map.end()) {
        if (dropped) dropped->push_back(it->second->payload);
        impl_->erase(it->second);
    }
    impl_->lru.push_front(Impl::Node{key, payload, bytes});
    impl_->map[key] = impl_->lru.begin();
    ++impl_->per_session_count[Impl::skey(session)];
    while (session_block_count(session) > per_session_) {
        // evict_lru_session_block: rposition -> the session's entry closest to the back
        auto r = impl_->lru.end();
        bool gone = false;
        while (r != impl_->lru.begin()) {
            --r;
            if (!std::memcmp(r->key.session, session, 32)) {
                if (dropped) dropped->push_back(r->payload);
                impl_->erase(r);
                gone = true;
                break;
            }
        }
        if (!gone) break;
    }
    while (impl_->lru.size() > capacity_) {
        auto last = std::prev(impl_->lru.end());
        if (dropped) dropped->push_back(last->payload);
        impl_->erase(last);
    }
    return bytes;
}

// evict_lru_block (src/serve/cache.rs:196-198)
bool PrefixIndex::evict_lru(uint64_t *payload, size_t *bytes) {
    if (impl_->lru.empty()) return false;
    auto last = std::prev(impl_->lru.end());
    if (payload) *payload = last->payload;
    if (bytes) *bytes = last->bytes;
    impl_->erase(last);
    return true;
}

bool PrefixIndex::entry(size_t index, uint8_t session[32], uint8_t hash[32], size_t *tokens,
                        uint64_t *payload, size_t *bytes) const {
    if (index >= impl_->lru.size()) return false;
    auto it = impl_->lru.begin();
    std::advance(it, (long)index);
    if (session) std::memcpy(session, it->key.session, 32);
    if (hash) std::memcpy(hash, it->key.hash, 32);
    if (tokens) *tokens = it->key.tokens;
    if (payload) *payload = it->payload;
    if (bytes) *bytes = it->bytes;
    return true;
}

} // namespace skv

using namespace skv;

struct skv_prefix {
    PrefixIndex index;
    skv_prefix(size_t bt, size_t cap, size_t per) : index(bt, cap, per) {}
};

extern "C" {

void skv_hash_root(uint8_t out[32]) { std::memset(out, 0, 32); }

void skv_hash_for_session(const char *key, size_t key_len, uint8_t out[32]) {
    if (!key || key_len == 0) {
        std::memset(out, 0, 32);
        return;
    }
    Sha256 h;
    h.update(key, key_len);
    h.finish(out);
}

void skv_hash_chain(const uint8_t previous[32], const uint64_t *tokens, size_t n, uint8_t out[32]) {
    hash_chain(previous, tokens, n, out);
}

int32_t skv_prefix_create(size_t block_tokens, size_t capacity, size_t blocks_per_session,
                          skv_prefix **out) try {
    if (!out) return fail(SKV_ERR_DEVICE, "skv_prefix_create: out nul");
    *out = new skv_prefix(block_tokens, capacity, blocks_per_session);
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prefix_from_runtime_flags(skv_prefix **out) try {
    return skv_prefix_create(skv_flag_serve_prefix_block_tokens(), skv_flag_serve_prefix_cache_blocks(),
                             skv_flag_serve_prefix_blocks_per_session(), out);
} catch (...) {
    return skv::fail_exception();
}

void skv_prefix_destroy(skv_prefix *cache) { delete cache; }

size_t skv_prefix_block_tokens(const skv_prefix *c) { return c ? c->index.block_tokens() : 0; }
size_t skv_prefix_capacity(const skv_prefix *c) { return c ? c->index.capacity() : 0; }
size_t skv_prefix_len(const skv_prefix *c) { return c ? c->index.len() : 0; }
size_t skv_prefix_bytes(const skv_prefix *c) { return c ? c->index.bytes() : 0; }
size_t skv_prefix_session_block_count(const skv_prefix *c, const uint8_t session[32]) {
    return c ? c->index.session_block_count(session) : 0;
}

int32_t skv_prefix_match(skv_prefix *c, const uint8_t root[32], const uint64_t *tokens, size_t n,
                         int32_t *found, skv_hit *hit, uint64_t *chain_payloads, size_t chain_cap) try {
    if (!c || !root || !found || (n && !tokens)) return fail(SKV_ERR_DEVICE, "prefix_match: pointeur nul");
    PrefixHit h{};
    std::vector<uint64_t> chain;
    const bool ok = c->index.match(root, tokens, n, &h, &chain);
    *found = ok ? 1 : 0;
    if (ok && hit) {
        hit->tokens = h.tokens;
        std::memcpy(hit->hash, h.hash, 32);
        hit->payload = h.payload;
        hit->matched_blocks = h.matched_blocks;
    }
    if (chain_payloads)
        for (size_t i = 0; i < chain.size() && i < chain_cap; ++i) chain_payloads[i] = chain[i];
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prefix_insert(skv_prefix *c, const uint8_t session[32], const uint8_t hash[32],
                          size_t tokens, uint64_t payload, size_t bytes, uint64_t *dropped,
                          size_t dropped_cap, size_t *n_dropped, size_t *bytes_out) try {
    if (!c || !session || !hash) return fail(SKV_ERR_DEVICE, "prefix_insert: pointeur nul");
    if (dropped && dropped_cap < 4)
        return fail(SKV_ERR_DIMENSION, "prefix_insert: dropped doit offrir au moins 4 places");
    std::vector<uint64_t> gone;
    const size_t b = c->index.insert(session, hash, tokens, payload, bytes, &gone);
    if (dropped)
        for (size_t i = 0; i < gone.size() && i < dropped_cap; ++i) dropped[i] = gone[i];
    if (n_dropped) *n_dropped = gone.size();
    if (bytes_out) *bytes_out = b;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prefix_evict_lru(skv_prefix *c, int32_t *found, uint64_t *payload, size_t *bytes) try {
    if (!c || !found) return fail(SKV_ERR_DEVICE, "prefix_evict_lru: pointeur nul");
    *found = c->index.evict_lru(payload, bytes) ? 1 : 0;
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

int32_t skv_prefix_entry(const skv_prefix *c, size_t index, uint8_t session[32], uint8_t hash[32],
                         size_t *tokens, uint64_t *payload, size_t *bytes) try {
    if (!c) return fail(SKV_ERR_DEVICE, "prefix_entry: pointeur nul");
    if (!c->index.entry(index, session, hash, tokens, payload, bytes))
        return fail(SKV_ERR_DIMENSION, "prefix_entry: index " + std::to_string(index) + " hors plage");
    return SKV_OK;
} catch (...) {
    return skv::fail_exception();
}

} // extern "C"
