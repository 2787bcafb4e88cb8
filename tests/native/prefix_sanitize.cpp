// Host-side soak of the prefix index and the SHA-256 chain under AddressSanitizer and
// UBSan: random inserts, matches, evictions and incremental walks against a plain
// vector model of BlockAwarePrefixCache (src/serve/cache.rs:72-219). Built and run by
// tests/test_native_sanitize.py with g++; no GPU involved.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "prefix.h"

using namespace skv;

struct Entry {
    uint8_t session[32], hash[32];
    size_t tokens;
    uint64_t payload;
    size_t bytes;
};

static bool same(const uint8_t *a, const uint8_t *b) { return std::memcmp(a, b, 32) == 0; }

int main() {
    std::mt19937_64 rng(7);
    const size_t bt = 4, cap = 24, per = 10;
    PrefixIndex index(bt, cap, per);
    std::vector<Entry> model; // index 0 = most recent
    uint8_t roots[3][32];
    for (int r = 0; r < 3; ++r) {
        std::memset(roots[r], 0, 32);
        roots[r][0] = (uint8_t)r;
    }
    uint64_t next_payload = 1;
    for (int op = 0; op < 20000; ++op) {
        const int r = (int)(rng() % 3);
        // prompts share prefixes: tokens drawn from a tiny alphabet
        const size_t n = 1 + rng() % 30;
        std::vector<uint64_t> toks(n);
        for (auto &t : toks) t = rng() % 2;
        const int kind = (int)(rng() % 10);
        if (kind < 5) { // walk the chain and remember every boundary, like a prefill
            uint8_t h[32];
            std::memcpy(h, roots[r], 32);
            for (size_t b = 0; (b + 1) * bt <= n; ++b) {
                uint8_t nh[32];
                hash_chain(h, toks.data() + b * bt, bt, nh);
                std::memcpy(h, nh, 32);
                std::vector<uint64_t> dropped;
                index.insert(roots[r], h, (b + 1) * bt, next_payload, 100 + b, &dropped);
                // model: drop equal key, push front, per-session cap, global cap
                std::vector<uint64_t> want_dropped;
                for (size_t i = 0; i < model.size(); ++i)
                    if (same(model[i].session, roots[r]) && same(model[i].hash, h) && model[i].tokens == (b + 1) * bt) {
                        want_dropped.push_back(model[i].payload);
                        model.erase(model.begin() + (long)i);
                        break;
                    }
                Entry e{};
                std::memcpy(e.session, roots[r], 32);
                std::memcpy(e.hash, h, 32);
                e.tokens = (b + 1) * bt;
                e.payload = next_payload++;
                e.bytes = 100 + b;
                model.insert(model.begin(), e);
                for (;;) {
                    size_t count = 0;
                    for (auto &m : model) count += same(m.session, roots[r]);
                    if (count <= per) break;
                    for (size_t i = model.size(); i-- > 0;)
                        if (same(model[i].session, roots[r])) {
                            want_dropped.push_back(model[i].payload);
                            model.erase(model.begin() + (long)i);
                            break;
                        }
                }
                while (model.size() > cap) {
                    want_dropped.push_back(model.back().payload);
                    model.pop_back();
                }
                if (dropped != want_dropped) {
                    std::printf("op %d: dropped payloads differ\n", op);
                    return 1;
                }
            }
        } else if (kind < 8) { // match, once in one go and once in steps on a second index state
            PrefixHit hit{};
            std::vector<uint64_t> chain;
            const bool found = index.match(roots[r], toks.data(), n, &hit, &chain);
            // model walk
            uint8_t h[32];
            std::memcpy(h, roots[r], 32);
            size_t matched = 0;
            uint64_t last_payload = 0;
            for (size_t b = 0; (b + 1) * bt <= n; ++b) {
                uint8_t nh[32];
                hash_chain(h, toks.data() + b * bt, bt, nh);
                std::memcpy(h, nh, 32);
                size_t at = model.size();
                for (size_t i = 0; i < model.size(); ++i)
                    if (same(model[i].session, roots[r]) && same(model[i].hash, h) && model[i].tokens == (b + 1) * bt) {
                        at = i;
                        break;
                    }
                if (at == model.size()) break;
                Entry e = model[at];
                model.erase(model.begin() + (long)at);
                model.insert(model.begin(), e);
                last_payload = e.payload;
                ++matched;
            }
            if (found != (matched > 0) || (found && (hit.tokens != matched * bt || hit.payload != last_payload ||
                                                     hit.matched_blocks != matched || chain.size() != matched))) {
                std::printf("op %d: match differs (found %d, matched %zu)\n", op, (int)found, matched);
                return 1;
            }
        } else { // evict
            uint64_t payload = 0;
            size_t bytes = 0;
            const bool got = index.evict_lru(&payload, &bytes);
            if (got != !model.empty() || (got && (payload != model.back().payload || bytes != model.back().bytes))) {
                std::printf("op %d: eviction differs\n", op);
                return 1;
            }
            if (got) model.pop_back();
        }
        if (index.len() != model.size()) {
            std::printf("op %d: len %zu vs %zu\n", op, index.len(), model.size());
            return 1;
        }
        size_t total = 0;
        for (auto &m : model) total += m.bytes;
        if (index.bytes() != total) {
            std::printf("op %d: bytes differ\n", op);
            return 1;
        }
        if (op % 97 == 0) // full order check
            for (size_t i = 0; i < model.size(); ++i) {
                uint8_t s[32], h[32];
                size_t tokens = 0, bytes = 0;
                uint64_t payload = 0;
                if (!index.entry(i, s, h, &tokens, &payload, &bytes) || payload != model[i].payload ||
                    tokens != model[i].tokens || !same(h, model[i].hash)) {
                    std::printf("op %d: order differs at %zu\n", op, i);
                    return 1;
                }
            }
    }
    // SHA-256 known answer (FIPS 180-4, "abc") through the portable and the accelerated path
    for (int portable = 0; portable < 2; ++portable) {
        setenv("SKV_SHA_PORTABLE", portable ? "1" : "0", 1);
        Sha256 sha;
        sha.update("abc", 3);
        uint8_t out[32];
        sha.finish(out);
        const uint8_t want[4] = {0xba, 0x78, 0x16, 0xbf};
        if (std::memcmp(out, want, 4) != 0) {
            std::printf("sha256(abc) wrong\n");
            return 1;
        }
    }
    std::printf("ok\n");
    return 0;
}

// The library's error sink lives with the device code; this host-only build supplies its own.
namespace skv {
int32_t fail(int32_t code, const std::string &message) {
    std::printf("error %d: %s\n", code, message.c_str());
    return code;
}
} // namespace skv
