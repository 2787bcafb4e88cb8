"""Pure-Python restatement of the reference's prefix hot cache (TEST INFRASTRUCTURE ONLY).

Follows src/serve/cache.rs:1-220 (hash chain, LRU ``Vec`` semantics) and
src/serve/state.rs:560-639 (block-boundary prefill and remember-with-eviction),
plus the decoder-internal whole-prompt cache of src/decoder/generation.rs:190-204,
2998-3025, 3105-3139. SHA-256 comes from ``hashlib`` (FIPS 180-4), an
implementation independent of the one in the product library; the reference uses
the ``sha2`` crate 0.10.9 (Cargo.lock:1739-1741). The reference's tests hold no
absolute digest, so the framing (32-byte previous hash, then each token as u64
little-endian) is pinned by src/serve/cache.rs:36-46 alone.

The LRU is a Python ``list`` used exactly like the reference's ``Vec``: index 0 is
the most recently used entry, ``pop()`` removes the least recently used one.
"""
from __future__ import annotations

import hashlib
import struct
from dataclasses import dataclass, field
from typing import Any, Callable, List, Optional, Sequence, Tuple


def hash_root() -> bytes:
    """BlockHash::root (src/serve/cache.rs:16-18)."""
    return bytes(32)


def hash_for_session(session_key: Optional[str]) -> bytes:
    """BlockHash::for_session (src/serve/cache.rs:22-32): empty or absent key -> root."""
    if not session_key:
        return hash_root()
    return hashlib.sha256(session_key.encode("utf-8")).digest()


def hash_chain(previous: bytes, tokens: Sequence[int]) -> bytes:
    """BlockHash::chain (src/serve/cache.rs:36-46)."""
    h = hashlib.sha256()
    h.update(previous)
    for token in tokens:
        h.update(struct.pack("<Q", token))
    return h.digest()


@dataclass
class Entry:
    session: bytes
    hash: bytes
    tokens: int
    state: Any
    metal: Any
    bytes: int


@dataclass
class Hit:
    tokens: int
    hash: bytes
    state: Any
    metal: Any


def _clone(obj):
    return obj.clone() if hasattr(obj, "clone") else obj


class BlockAwarePrefixCache:
    """BlockAwarePrefixCache (src/serve/cache.rs:72-219).

    ``state_bytes(state, metal)`` plays the part of ``estimated_cpu_bytes() +
    estimated_bytes()`` (src/serve/cache.rs:172-174).
    """

    def __init__(self, block_tokens: int, capacity: int, blocks_per_session: Optional[int] = None,
                 state_bytes: Callable[[Any, Any], int] = lambda s, m: 0):
        self.block_tokens = max(block_tokens, 1)
        self.capacity = capacity
        self.blocks_per_session = capacity if blocks_per_session is None else blocks_per_session
        self.entries: List[Entry] = []
        self._state_bytes = state_bytes

    def match_prefix(self, root: bytes, tokens: Sequence[int]) -> Optional[Hit]:
        """src/serve/cache.rs:121-151."""
        if self.capacity == 0:
            return None
        previous = root
        best = None
        bt = self.block_tokens
        for index in range(len(tokens) // bt):  # chunks_exact
            block = tokens[index * bt:(index + 1) * bt]
            h = hash_chain(previous, block)
            expected_tokens = (index + 1) * bt
            entry_index = next((i for i, e in enumerate(self.entries)
                                if e.session == root and e.hash == h
                                and e.tokens == expected_tokens), None)
            if entry_index is None:
                break
            entry = self.entries.pop(entry_index)
            hit = Hit(entry.tokens, entry.hash, _clone(entry.state), _clone(entry.metal))
            self.entries.insert(0, entry)
            previous = h
            best = hit
        return best

    def insert(self, session: bytes, h: bytes, tokens: int, state: Any, metal: Any) -> int:
        """src/serve/cache.rs:154-193."""
        if self.capacity == 0:
            return 0
        index = next((i for i, e in enumerate(self.entries)
                      if e.session == session and e.hash == h and e.tokens == tokens), None)
        if index is not None:
            self.entries.pop(index)
        nbytes = self._state_bytes(state, metal)
        self.entries.insert(0, Entry(session, h, tokens, state, metal, nbytes))
        while self.session_block_count(session) > self.blocks_per_session:
            if self.evict_lru_session_block(session) is None:
                break
        while len(self.entries) > self.capacity:
            self.entries.pop()
        return nbytes

    def evict_lru_block(self) -> Optional[int]:
        """src/serve/cache.rs:196-198."""
        if not self.entries:
            return None
        return self.entries.pop().bytes

    def estimated_bytes(self) -> int:
        """src/serve/cache.rs:202-204."""
        return sum(e.bytes for e in self.entries)

    def session_block_count(self, session: bytes) -> int:
        return sum(1 for e in self.entries if e.session == session)

    def evict_lru_session_block(self, session: bytes) -> Optional[int]:
        """src/serve/cache.rs:213-219: rposition -> the session's least recent entry."""
        for i in range(len(self.entries) - 1, -1, -1):
            if self.entries[i].session == session:
                return self.entries.pop(i).bytes
        return None


class PromptDecoder:
    """The four decoder calls the boundary algorithm makes, to be supplied by a test.

    prefill_uncached(tokens) -> state            src/decoder/generation.rs:2803-2809
    extend(state, tokens) -> None (in place)     src/decoder/generation.rs:2816-2827
    snapshot_metal(state) -> metal               src/decoder/generation.rs:2834-2849
    copy_metal(metal) -> metal                   src/decoder/generation.rs:2856-2871
    restore_metal(state, metal) -> None          src/decoder/generation.rs:2878-2892
    """

    def prefill_uncached(self, tokens): raise NotImplementedError
    def extend(self, state, tokens): raise NotImplementedError
    def snapshot_metal(self, state): return None
    def copy_metal(self, metal): return metal
    def restore_metal(self, state, metal): return None


def remember_prefix_block(cache: BlockAwarePrefixCache, decoder: PromptDecoder, session: bytes,
                          h: bytes, tokens: int, state: Any,
                          over_limit: Callable[[int], bool]) -> bool:
    """remember_prefix_block (src/serve/state.rs:613-639). Returns False when the
    block was skipped because nothing was left to evict (no error)."""
    metal = decoder.snapshot_metal(state)
    additional = cache._state_bytes(state, metal)
    while over_limit(additional):
        if cache.evict_lru_block() is None:
            return False
    cache.insert(session, h, tokens, _clone(state), metal)
    return True


def prefill_prompt_state(cache: BlockAwarePrefixCache, decoder: PromptDecoder,
                         tokens: Sequence[int], session_key: Optional[str],
                         over_limit: Callable[[int], bool] = lambda extra: False,
                         enabled: bool = True) -> Tuple[Any, int]:
    """LoadedModel::prefill_prompt_state (src/serve/state.rs:560-611).

    Returns (state, reused_prefix_tokens)."""
    if not enabled:
        return decoder.prefill_uncached(tokens), 0
    bt = cache.block_tokens
    full_block_tokens = len(tokens) // bt * bt
    root = hash_for_session(session_key)
    hit = cache.match_prefix(root, tokens)
    reused = hit.tokens if hit is not None else 0
    if hit is not None:
        state = hit.state
        metal = decoder.copy_metal(hit.metal)
        decoder.restore_metal(state, metal)
        consumed, h = hit.tokens, hit.hash
    elif full_block_tokens >= bt:
        first = tokens[:bt]
        state = decoder.prefill_uncached(first)
        h = hash_chain(root, first)
        remember_prefix_block(cache, decoder, root, h, bt, state, over_limit)
        consumed = bt
    else:
        return decoder.prefill_uncached(tokens), 0
    while consumed + bt <= full_block_tokens:
        nxt = consumed + bt
        block = tokens[consumed:nxt]
        decoder.extend(state, block)
        h = hash_chain(h, block)
        remember_prefix_block(cache, decoder, root, h, nxt, state, over_limit)
        consumed = nxt
    if consumed < len(tokens):
        decoder.extend(state, tokens[consumed:])
    return state, reused


# ---- decoder-internal whole-prompt prefix cache -----------------------------

def longest_prefix_entry_index(entries: Sequence[Sequence[int]], prompt: Sequence[int]):
    """longest_prefix_entry_index (src/decoder/generation.rs:190-204); entries are token lists."""
    best, best_len = None, 0
    for index, toks in enumerate(entries):
        n = len(toks)
        if n > best_len and n <= len(prompt) and list(prompt[:n]) == list(toks):
            best, best_len = index, n
    return best


@dataclass
class WholePromptCache:
    """prefix_cache_get / prefix_cache_put (src/decoder/generation.rs:2998-3025, 3105-3139)."""

    capacity: int = 4
    entries: List[Tuple[List[int], Any]] = field(default_factory=list)

    def get(self, prompt: Sequence[int], extend: Callable[[Any, Sequence[int]], None]):
        index = longest_prefix_entry_index([e[0] for e in self.entries], prompt)
        if index is None:
            return None
        entry = self.entries.pop(index)
        cached_len = len(entry[0])
        output = _clone(entry[1])
        self.entries.insert(0, entry)
        if cached_len < len(prompt):
            extend(output, prompt[cached_len:])
            self.put(prompt, output)
        return output

    def put(self, prompt: Sequence[int], state: Any) -> None:
        if self.capacity == 0:
            return
        index = next((i for i, e in enumerate(self.entries) if e[0] == list(prompt)), None)
        if index is not None:
            self.entries.pop(index)
        self.entries.insert(0, (list(prompt), _clone(state)))
        del self.entries[self.capacity:]
