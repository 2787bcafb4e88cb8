// SHA-256 chained block keys and the LRU index of the prefix hot cache (host only).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <vector>

#include "skv_internal.h"

namespace skv {

class Sha256 {
  public:
    Sha256() { reset(); }
    void reset();
    void update(const void *data, size_t n);
    void finish(uint8_t out[32]);

  private:
    void block(const uint8_t *p);
    uint32_t h_[8];
    uint64_t len_;
    uint8_t buf_[64];
    size_t fill_;
};

void hash_chain(const uint8_t prev[32], const uint64_t *tokens, size_t n, uint8_t out[32]);

struct PrefixHit {
    size_t tokens;
    uint8_t hash[32];
    uint64_t payload;
    size_t matched_blocks;
};

// BlockAwarePrefixCache (src/serve/cache.rs:72-219) with opaque 64-bit payloads in
// place of the owned prompt state.
class PrefixIndex {
  public:
    PrefixIndex(size_t block_tokens, size_t capacity, size_t per_session);
    ~PrefixIndex();
    PrefixIndex(const PrefixIndex &) = delete;
    PrefixIndex &operator=(const PrefixIndex &) = delete;

    size_t block_tokens() const { return block_tokens_; }
    size_t capacity() const { return capacity_; }
    size_t len() const;
    size_t bytes() const;
    size_t session_block_count(const uint8_t session[32]) const;
    bool match(const uint8_t root[32], const uint64_t *tokens, size_t n, PrefixHit *hit,
               std::vector<uint64_t> *chain);
    // The same walk in steps, so that a caller can act on the first matched blocks while
    // the rest of the chain is still being hashed. match_more() appends to `chain` and
    // returns how many further blocks matched (fewer than max_blocks: the walk is over).
    struct Walk {
        uint8_t previous[32];
        size_t index = 0;
        bool alive = true;
    };
    void match_start(Walk *w, const uint8_t root[32]) const;
    size_t match_more(Walk *w, const uint8_t root[32], const uint64_t *tokens, size_t n,
                      size_t max_blocks, PrefixHit *hit, std::vector<uint64_t> *chain);
    size_t insert(const uint8_t session[32], const uint8_t hash[32], size_t tokens,
                  uint64_t payload, size_t bytes, std::vector<uint64_t> *dropped);
    bool evict_lru(uint64_t *payload, size_t *bytes);
    bool entry(size_t index, uint8_t session[32], uint8_t hash[32], size_t *tokens,
               uint64_t *payload, size_t *bytes) const;

  private:
    struct Impl;
    size_t block_tokens_, capacity_, per_session_;
    Impl *impl_;
};

} // namespace skv
