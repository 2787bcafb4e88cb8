"""Prefix hot cache, host side: the native SHA-256 chain and LRU index against the
reference's own tests (src/serve/cache.rs:281-493), against hashlib, and differentially
against the pure-Python restatement of the reference's Vec semantics. No GPU."""
import hashlib
import struct

import numpy as np
import pytest

import saragossa_amd as skv
from oracle import prefix_cache as pc
from saragossa_amd import BlockAwarePrefixCache, BlockHash


class State:
    """Stand-in for CausalDecoderPromptState: position() and a deep clone."""

    def __init__(self, position):
        self._p = position

    def position(self):
        return self._p

    def clone(self):
        return State(self._p)


# ---- hashing -----------------------------------------------------------------------------
def test_sha256_matches_hashlib_for_all_paddings():
    prev = bytes(range(32))
    for n in list(range(0, 20)) + [31, 32, 255, 256, 1000]:
        tokens = [(i * 2654435761 + 7) % (2 ** 64) for i in range(n)]
        want = hashlib.sha256(prev + b"".join(struct.pack("<Q", t) for t in tokens)).digest()
        assert BlockHash.chain(prev, tokens) == want == pc.hash_chain(prev, tokens)
    for key in ["a", "alpha", "x" * 55, "x" * 56, "x" * 63, "x" * 64, "x" * 65, "é🙂" * 40]:
        assert BlockHash.for_session(key) == hashlib.sha256(key.encode()).digest()
    # FIPS 180-4 known answers
    assert BlockHash.for_session("abc").hex() == \
        "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad"


def test_chained_hash_depends_on_previous_block():
    # src/serve/cache.rs:281-288
    first = BlockHash.chain(BlockHash.root(), [1, 2])
    assert BlockHash.chain(first, [3, 4]) != BlockHash.chain(BlockHash.root(), [3, 4])


def test_session_roots_are_deterministic_and_disjoint():
    # src/serve/cache.rs:290-298
    assert BlockHash.for_session("alpha") == BlockHash.for_session("alpha")
    assert BlockHash.for_session("alpha") != BlockHash.for_session("beta")


def test_absent_session_keeps_global_root_byte_identity():
    # src/serve/cache.rs:300-309
    assert BlockHash.for_session(None) == BlockHash.root() == bytes(32)
    assert BlockHash.for_session("") == BlockHash.root()
    assert BlockHash.chain(BlockHash.for_session(None), [1, 2, 3]) == \
        BlockHash.chain(BlockHash.root(), [1, 2, 3])


# ---- index: the reference's tests -----------------------------------------------------------
def test_prefix_cache_matches_longest_chain():
    # src/serve/cache.rs:311-339
    cache = BlockAwarePrefixCache(2, 8)
    root = BlockHash.root()
    first = BlockHash.chain(root, [1, 2])
    second = BlockHash.chain(first, [3, 4])
    cache.insert(root, first, 2, State(2), None)
    cache.insert(root, second, 4, State(4), None)
    hit = cache.match_prefix(root, [1, 2, 3, 4, 5])
    assert hit is not None
    assert hit.tokens == 4 and hit.hash == second and hit.state.position() == 4


def test_prefix_cache_evicts_lru_block():
    # src/serve/cache.rs:341-374: evicting block 1 strands its descendants
    cache = BlockAwarePrefixCache(1, 2)
    root = BlockHash.root()
    first = BlockHash.chain(root, [1])
    second = BlockHash.chain(first, [2])
    third = BlockHash.chain(second, [3])
    for h, n in [(first, 1), (second, 2), (third, 3)]:
        cache.insert(root, h, n, State(n), None)
    assert cache.match_prefix(root, [1]) is None
    assert cache.match_prefix(root, [1, 2, 3]) is None
    assert len(cache) == 2


def test_default_session_cap_keeps_global_lru_eviction_order():
    # src/serve/cache.rs:376-417
    cache = BlockAwarePrefixCache(1, 2)
    alpha, beta = BlockHash.for_session("agent-a"), BlockHash.for_session("agent-b")
    beta_first = BlockHash.chain(beta, [9])
    alpha_first = BlockHash.chain(alpha, [1])
    alpha_second = BlockHash.chain(alpha_first, [2])
    cache.insert(beta, beta_first, 1, State(1), None)
    cache.insert(alpha, alpha_first, 1, State(1), None)
    cache.insert(alpha, alpha_second, 2, State(2), None)
    assert [e["hash"] for e in cache.entries] == [alpha_second, alpha_first]
    assert cache.match_prefix(beta, [9]) is None


def test_reduced_session_cap_evicts_only_that_session_first():
    # src/serve/cache.rs:419-461
    cache = BlockAwarePrefixCache(1, 2, 1)
    alpha, beta = BlockHash.for_session("agent-a"), BlockHash.for_session("agent-b")
    beta_first = BlockHash.chain(beta, [9])
    alpha_first = BlockHash.chain(alpha, [1])
    alpha_second = BlockHash.chain(alpha_first, [2])
    cache.insert(beta, beta_first, 1, State(1), None)
    cache.insert(alpha, alpha_first, 1, State(1), None)
    cache.insert(alpha, alpha_second, 2, State(2), None)
    assert [e["hash"] for e in cache.entries] == [alpha_second, beta_first]
    assert cache.match_prefix(beta, [9]).hash == beta_first
    assert cache.session_block_count(alpha) == 1


def test_prefix_cache_does_not_match_across_sessions():
    # src/serve/cache.rs:463-493
    cache = BlockAwarePrefixCache(2, 8)
    alpha, beta = BlockHash.for_session("agent-a"), BlockHash.for_session("agent-b")
    first = BlockHash.chain(alpha, [1, 2])
    second = BlockHash.chain(first, [3, 4])
    cache.insert(alpha, first, 2, State(2), None)
    cache.insert(alpha, second, 4, State(4), None)
    assert first != BlockHash.chain(beta, [1, 2])
    assert cache.match_prefix(beta, [1, 2, 3, 4]) is None
    assert cache.match_prefix(alpha, [1, 2, 3, 4]).tokens == 4


# ---- index: semantics the reference's Vec has and an idiomatic LRU gets wrong ---------------
def test_match_leaves_chain_in_reverse_walk_order_and_clones_state():
    cache = BlockAwarePrefixCache(1, 8)
    root = BlockHash.root()
    hs, prev = [], root
    for i in range(4):
        prev = BlockHash.chain(prev, [i])
        hs.append(prev)
        cache.insert(root, prev, i + 1, State(i + 1), None)
    other = BlockHash.chain(root, [77])
    cache.insert(root, other, 1, State(1), None)
    hit = cache.match_prefix(root, [0, 1, 2])           # b1..b3 hit
    assert hit.tokens == 3 and hit.matched_blocks == 3
    assert [e["hash"] for e in cache.entries] == [hs[2], hs[1], hs[0], other, hs[3]]
    assert hit.state is not cache.entries[0]["state"]    # the hit carries a clone


def test_equal_hash_different_tokens_are_distinct_and_reinsert_refreshes():
    cache = BlockAwarePrefixCache(1, 8, state_bytes=lambda s, m: s.position() * 10)
    root = BlockHash.root()
    h = BlockHash.chain(root, [5])
    assert cache.insert(root, h, 1, State(1), None) == 10
    cache.insert(root, h, 2, State(2), None)             # same digest, other length
    assert len(cache) == 2 and cache.estimated_bytes() == 30
    cache.insert(root, h, 1, State(7), None)             # refresh: replaced, moved to front
    assert len(cache) == 2 and cache.entries[0]["tokens"] == 1
    assert cache.estimated_bytes() == 90
    assert cache.evict_lru_block() == 20 and cache.evict_lru_block() == 70
    assert cache.evict_lru_block() is None


def test_capacity_zero_disables_and_block_tokens_floor():
    cache = BlockAwarePrefixCache(0, 0)
    assert cache.block_tokens() == 1                      # block_tokens.max(1)
    root = BlockHash.root()
    assert cache.insert(root, BlockHash.chain(root, [1]), 1, State(1), None) == 0
    assert len(cache) == 0 and cache.match_prefix(root, [1]) is None


def test_partial_trailing_block_is_ignored():
    cache = BlockAwarePrefixCache(4, 8)
    root = BlockHash.root()
    h = BlockHash.chain(root, [1, 2, 3, 4])
    cache.insert(root, h, 4, State(4), None)
    assert cache.match_prefix(root, [1, 2, 3]) is None            # chunks_exact: no whole block
    assert cache.match_prefix(root, [1, 2, 3, 4, 5, 6, 7]).tokens == 4


@pytest.mark.parametrize("seed", range(6))
def test_native_index_equals_python_restatement_under_random_ops(seed):
    """Differential run against the list-based restatement of the reference: same hits,
    same order, same byte totals after every operation."""
    rng = np.random.default_rng(seed)
    bt = int(rng.integers(1, 4))
    cap = int(rng.integers(1, 12))
    per = int(rng.integers(1, cap + 1))
    sb = lambda s, m: s.position() * 3 + 1
    a = BlockAwarePrefixCache(bt, cap, per, state_bytes=sb)
    b = pc.BlockAwarePrefixCache(bt, cap, per, state_bytes=sb)
    sessions = [None, "s1", "s2"]
    prompts = [list(rng.integers(0, 3, size=rng.integers(1, 5) * bt)) for _ in range(6)]
    for _ in range(300):
        op = rng.integers(0, 10)
        sk = sessions[rng.integers(0, 3)]
        root = BlockHash.for_session(sk)
        assert root == pc.hash_for_session(sk)
        toks = [int(t) for t in prompts[rng.integers(0, len(prompts))]]
        if op < 5:                                         # insert every block boundary prefix
            n_blocks = int(rng.integers(1, len(toks) // bt + 1))
            h = root
            for i in range(n_blocks):
                h = BlockHash.chain(h, toks[i * bt:(i + 1) * bt])
            n = n_blocks * bt
            assert a.insert(root, h, n, State(n), None) == b.insert(root, h, n, State(n), None)
        elif op < 9:
            extra = [int(t) for t in rng.integers(0, 3, size=rng.integers(0, bt))]
            ha, hb = a.match_prefix(root, toks + extra), b.match_prefix(root, toks + extra)
            assert (ha is None) == (hb is None)
            if ha is not None:
                assert (ha.tokens, ha.hash, ha.state.position()) == \
                       (hb.tokens, hb.hash, hb.state.position())
        else:
            assert a.evict_lru_block() == b.evict_lru_block()
        assert [(e["session"], e["hash"], e["tokens"], e["bytes"]) for e in a.entries] == \
               [(e.session, e.hash, e.tokens, e.bytes) for e in b.entries]
        assert a.estimated_bytes() == b.estimated_bytes()


# ---- the block-boundary algorithm and the whole-prompt cache (oracle self-checks) -----------
class FakeDecoder(pc.PromptDecoder):
    """Prompt state = the list of tokens consumed; lets the boundary algorithm be checked
    for the invariant "state after a hit + extend == state of a cold prefill"."""

    class S(list):
        def clone(self):
            return FakeDecoder.S(self)

    def __init__(self):
        self.calls = []

    def prefill_uncached(self, tokens):
        self.calls.append(("prefill", len(tokens)))
        return FakeDecoder.S(tokens)

    def extend(self, state, tokens):
        self.calls.append(("extend", len(tokens)))
        state.extend(tokens)


def test_prefill_prompt_state_boundary_algorithm():
    # src/serve/state.rs:560-611
    dec = FakeDecoder()
    cache = pc.BlockAwarePrefixCache(4, 16)
    prompt = list(range(11))
    state, reused = pc.prefill_prompt_state(cache, dec, prompt, "sess")
    assert state == prompt and reused == 0
    assert dec.calls == [("prefill", 4), ("extend", 4), ("extend", 3)]
    assert [e.tokens for e in cache.entries] == [8, 4]
    dec.calls.clear()
    state, reused = pc.prefill_prompt_state(cache, dec, prompt + [99, 98], "sess")
    assert state == prompt + [99, 98] and reused == 8
    assert dec.calls == [("extend", 4), ("extend", 1)]     # block 3 completes, then the tail
    assert [e.tokens for e in cache.entries] == [12, 8, 4]
    # a prompt shorter than one block bypasses the cache; another session does not hit
    dec.calls.clear()
    state, reused = pc.prefill_prompt_state(cache, dec, [0, 1, 2], "sess")
    assert reused == 0 and dec.calls == [("prefill", 3)]
    _, reused = pc.prefill_prompt_state(cache, dec, prompt, "other")
    assert reused == 0
    # disabled
    _, reused = pc.prefill_prompt_state(cache, dec, prompt, "sess", enabled=False)
    assert reused == 0


def test_remember_prefix_block_evicts_then_skips_without_error():
    # src/serve/state.rs:613-639 with an injected footprint probe (memory_guard.rs:298-309)
    dec = FakeDecoder()
    cache = pc.BlockAwarePrefixCache(1, 8, state_bytes=lambda s, m: 10)
    root = pc.hash_root()
    for i in range(3):
        cache.insert(root, pc.hash_chain(root, [i]), 1, FakeDecoder.S([i]), None)
    budget = 30
    over = lambda extra: cache.estimated_bytes() + extra > budget
    assert pc.remember_prefix_block(cache, dec, root, pc.hash_chain(root, [9]), 1,
                                    FakeDecoder.S([9]), over)
    assert len(cache.entries) == 3 and cache.entries[0].hash == pc.hash_chain(root, [9])
    assert all(e.hash != pc.hash_chain(root, [0]) for e in cache.entries)   # LRU victim
    budget = 5                                                             # nothing can fit
    assert not pc.remember_prefix_block(cache, dec, root, pc.hash_chain(root, [8]), 1,
                                        FakeDecoder.S([8]), over)
    assert len(cache.entries) == 0                                         # evicted all, skipped


def test_whole_prompt_cache_longest_prefix_and_truncate():
    # src/decoder/generation.rs:190-204, 2998-3025, 3105-3139
    assert pc.longest_prefix_entry_index([[1, 2], [1, 2, 3], [9]], [1, 2, 3, 4]) == 1
    assert pc.longest_prefix_entry_index([[1, 2, 3, 4, 5]], [1, 2, 3]) is None
    assert pc.longest_prefix_entry_index([[], [1]], [1]) == 1      # len must exceed best_len 0
    c = pc.WholePromptCache(capacity=2)
    ext = lambda st, toks: st.extend(toks)
    c.put([1, 2], FakeDecoder.S([1, 2]))
    c.put([7], FakeDecoder.S([7]))
    got = c.get([1, 2, 3], ext)
    assert got == [1, 2, 3]
    assert [e[0] for e in c.entries] == [[1, 2, 3], [1, 2]]         # extended entry put first, cap 2
    assert c.get([5], ext) is None
