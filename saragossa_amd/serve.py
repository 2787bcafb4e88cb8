"""Host mirror of the serve-side prompt path: LoadedModel::prefill_prompt_state and its
helpers (src/serve/state.rs:560-646) over the GPU hot cache.

The reference clones whole prompt states at every block boundary; here a boundary stores
the pages of its own block in the hot cache's pool and a hit gathers the chain's blocks back
into the session's paged caches. The control flow (what is matched, what is prefilled, what
is remembered, in which order blocks are evicted) is the reference's.
"""
from __future__ import annotations

from typing import Callable, Optional, Sequence

from . import flags
from .prefix import BlockHash, HotCache


class LoadedModelKv:
    """The KV half of LoadedModel (src/serve/state.rs:392-646).

    ``prefill_rows(first, last)`` is the decoder's part: it must run the model over the
    prompt positions [first, last) and append their K/V rows to ``layers`` (for instance
    with ``encode_prefill_rows``); it stands for prefill_prompt_state_uncached /
    extend_prompt_state (src/decoder/generation.rs:2803-2827).
    """

    def __init__(self, hot: HotCache, enabled: Optional[bool] = None):
        self.hot = hot
        # RETI_SERVE_PREFIX_CACHE kill-switch (src/runtime_flags.rs:681-684)
        self.enabled = flags.serve_prefix_cache_enabled() if enabled is None else enabled

    def prefill_prompt_state(self, tokens: Sequence[int], session_key: Optional[str], layers,
                             prefill_rows: Callable[[int, int], None], stream=None,
                             blocks_per_chunk: int = 1) -> int:
        """Returns reused_prefix_tokens. ``blocks_per_chunk`` > 1 prefills that many hash
        blocks per call and remembers them together (same cache contents and order)."""
        n = len(tokens)
        if not self.enabled:
            for kv in layers:
                kv.truncate(0)
            prefill_rows(0, n)
            return 0
        bt = self.hot.block_tokens()
        full_block_tokens = n // bt * bt
        root = BlockHash.for_session(session_key)
        reused, h = self.hot.match_restore(root, tokens, layers, stream=stream)
        if reused:
            consumed = reused
        elif full_block_tokens >= bt:
            for kv in layers:
                kv.truncate(0)
            prefill_rows(0, bt)
            h = BlockHash.chain(root, tokens[:bt])
            self.remember_prefix_block(root, h, bt, layers, stream)
            consumed = bt
        else:
            for kv in layers:
                kv.truncate(0)
            prefill_rows(0, n)
            return 0
        step = max(1, blocks_per_chunk) * bt
        while consumed + bt <= full_block_tokens:
            nxt = min(consumed + step, full_block_tokens)
            prefill_rows(consumed, nxt)
            hashes = []
            for b in range(consumed, nxt, bt):
                h = BlockHash.chain(h, tokens[b:b + bt])
                hashes.append(h)
            if len(hashes) == 1:
                self.remember_prefix_block(root, h, nxt, layers, stream)
            else:
                self.hot.remember_prefix_blocks(root, hashes, consumed + bt, layers, stream=stream)
            consumed = nxt
        if consumed < n:
            prefill_rows(consumed, n)
        return reused

    def remember_prefix_block(self, session: bytes, h: bytes, tokens: int, layers, stream=None) -> bool:
        """remember_prefix_block (src/serve/state.rs:613-639): the pool is the byte budget."""
        return self.hot.remember_prefix_block(session, h, tokens, layers, stream=stream)

    def prefix_cache_bytes(self) -> int:
        return self.hot.estimated_bytes()

    def evict_prefix_block(self) -> Optional[int]:
        return self.hot.evict_lru_block()
