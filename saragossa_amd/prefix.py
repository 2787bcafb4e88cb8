"""Host mirror of the serve-side prefix hot cache (src/serve/cache.rs, src/serve/state.rs).

``BlockAwarePrefixCache`` binds the native index and keeps the Python objects the
reference stores by value (prompt state, device snapshot) in a side table keyed by the
payload id, so that its method signatures are the reference's. ``HotCache`` is the GPU
form: a pool of page slots filled and drained by copy kernels.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Any, Callable, List, Optional, Sequence

import numpy as np

from ._lib import check, lib


def _tok(tokens) -> np.ndarray:
    return np.ascontiguousarray(tokens, dtype=np.uint64)


def _buf32():
    return (C.c_uint8 * 32)()


def _in32(b: bytes):
    assert len(b) == 32
    return (C.c_uint8 * 32).from_buffer_copy(b)


class BlockHash:
    """BlockHash (src/serve/cache.rs:10-47)."""

    @staticmethod
    def root() -> bytes:
        out = _buf32()
        lib().skv_hash_root(out)
        return bytes(out)

    @staticmethod
    def for_session(session_key: Optional[str]) -> bytes:
        out = _buf32()
        key = (session_key or "").encode("utf-8")
        lib().skv_hash_for_session(key if key else None, len(key), out)
        return bytes(out)

    @staticmethod
    def chain(previous: bytes, tokens: Sequence[int]) -> bytes:
        t = _tok(tokens)
        out = _buf32()
        lib().skv_hash_chain(_in32(previous), t.ctypes.data_as(C.c_void_p), t.size, out)
        return bytes(out)


class _Hit(C.Structure):
    _fields_ = [("tokens", C.c_size_t), ("hash", C.c_uint8 * 32), ("payload", C.c_uint64),
                ("matched_blocks", C.c_size_t)]


@dataclass
class PrefixBlockHit:
    """PrefixBlockHit (src/serve/cache.rs:50-60)."""
    tokens: int
    hash: bytes
    state: Any
    metal: Any
    matched_blocks: int = 0


def _clone(obj):
    return obj.clone() if hasattr(obj, "clone") else obj


class BlockAwarePrefixCache:
    """BlockAwarePrefixCache (src/serve/cache.rs:72-219)."""

    def __init__(self, block_tokens: int, capacity: int, blocks_per_session: Optional[int] = None,
                 state_bytes: Callable[[Any, Any], int] = lambda s, m: 0, _handle=None):
        self._l = lib()
        if _handle is None:
            h = C.c_void_p()
            per = capacity if blocks_per_session is None else blocks_per_session
            check(self._l.skv_prefix_create(block_tokens, capacity, per, C.byref(h)))
            _handle = h
        self._h = _handle
        self._objs = {}
        self._next = 1
        self._state_bytes = state_bytes

    @classmethod
    def from_runtime_flags(cls, **kw) -> "BlockAwarePrefixCache":
        h = C.c_void_p()
        check(lib().skv_prefix_from_runtime_flags(C.byref(h)))
        return cls(0, 0, _handle=h, **kw)

    def __del__(self):
        if getattr(self, "_h", None):
            self._l.skv_prefix_destroy(self._h)
            self._h = None

    def block_tokens(self) -> int:
        return self._l.skv_prefix_block_tokens(self._h)

    def capacity(self) -> int:
        return self._l.skv_prefix_capacity(self._h)

    def __len__(self) -> int:
        return self._l.skv_prefix_len(self._h)

    def estimated_bytes(self) -> int:
        return self._l.skv_prefix_bytes(self._h)

    def session_block_count(self, session: bytes) -> int:
        return self._l.skv_prefix_session_block_count(self._h, _in32(session))

    def match_prefix(self, root: bytes, tokens: Sequence[int]) -> Optional[PrefixBlockHit]:
        t = _tok(tokens)
        found, hit = C.c_int32(), _Hit()
        check(self._l.skv_prefix_match(self._h, _in32(root), t.ctypes.data_as(C.c_void_p), t.size,
                                       C.byref(found), C.byref(hit), None, 0))
        if not found.value:
            return None
        state, metal = self._objs[hit.payload]
        return PrefixBlockHit(hit.tokens, bytes(hit.hash), _clone(state), _clone(metal),
                              hit.matched_blocks)

    def insert(self, session: bytes, hash_: bytes, tokens: int, state: Any, metal: Any) -> int:
        pid = self._next
        self._next += 1
        self._objs[pid] = (state, metal)
        dropped = (C.c_uint64 * 8)()
        n_dropped, bytes_out = C.c_size_t(), C.c_size_t()
        check(self._l.skv_prefix_insert(self._h, _in32(session), _in32(hash_), tokens, pid,
                                        self._state_bytes(state, metal), dropped, 8,
                                        C.byref(n_dropped), C.byref(bytes_out)))
        for i in range(n_dropped.value):
            self._objs.pop(dropped[i], None)
        return bytes_out.value

    def evict_lru_block(self) -> Optional[int]:
        found, payload, nbytes = C.c_int32(), C.c_uint64(), C.c_size_t()
        check(self._l.skv_prefix_evict_lru(self._h, C.byref(found), C.byref(payload),
                                           C.byref(nbytes)))
        if not found.value:
            return None
        self._objs.pop(payload.value, None)
        return nbytes.value

    @property
    def entries(self) -> List[dict]:
        """The reference tests' view of `cache.entries` (index 0 = most recent)."""
        out = []
        for i in range(len(self)):
            s, h = _buf32(), _buf32()
            tok, payload, nbytes = C.c_size_t(), C.c_uint64(), C.c_size_t()
            check(self._l.skv_prefix_entry(self._h, i, s, h, C.byref(tok), C.byref(payload),
                                           C.byref(nbytes)))
            out.append({"session": bytes(s), "hash": bytes(h), "tokens": tok.value,
                        "bytes": nbytes.value, "state": self._objs[payload.value][0]})
        return out


class Snapshot:
    """CausalDecoderPromptMetalSnapshot (src/decoder.rs:266-290): owned device copy."""

    def __init__(self, ctx, handle):
        self._ctx, self._l, self._h = ctx, lib(), handle

    def estimated_bytes(self) -> int:
        return self._l.skv_snapshot_bytes(self._h)

    def clone(self, stream=None) -> "Snapshot":
        h = C.c_void_p()
        check(self._l.skv_snapshot_clone(self._ctx._h, stream, self._h, C.byref(h)))
        return Snapshot(self._ctx, h)

    def close(self):
        if getattr(self, "_h", None):
            self._l.skv_snapshot_free(self._h)
            self._h = None

    def __del__(self):
        self.close()


_LAYER_ARRAYS: dict = {}


def _layer_array(layers):
    """The handles of `layers` as a C array. A server passes the same set of layers at every
    block boundary, so the last few arrays are kept (keyed by the handles themselves)."""
    key = tuple(l._h.value for l in layers)
    arr = _LAYER_ARRAYS.get(key)
    if arr is None:
        if len(_LAYER_ARRAYS) >= 16:
            _LAYER_ARRAYS.clear()
        arr = _LAYER_ARRAYS[key] = (C.c_void_p * len(key))(*key)
    return arr


def _ptr_arrays(ptrs, sizes):
    n = len(ptrs)
    return (C.c_void_p * n)(*ptrs), (C.c_size_t * n)(*sizes), n


def snapshot_blocks(ctx, layers, block_ids, stream=None) -> Snapshot:
    ids = (C.c_size_t * len(block_ids))(*block_ids)
    h = C.c_void_p()
    check(lib().skv_snapshot_blocks(ctx._h, stream, _layer_array(layers), len(layers), ids,
                                    len(block_ids), C.byref(h)))
    return Snapshot(ctx, h)


def restore_blocks(ctx, snapshot: Snapshot, layers, dst_block_ids, stream=None) -> None:
    ids = (C.c_size_t * len(dst_block_ids))(*dst_block_ids)
    check(lib().skv_restore_blocks(ctx._h, stream, snapshot._h, _layer_array(layers), len(layers),
                                   ids, len(dst_block_ids)))


def state_snapshot(ctx, ptrs, sizes, stream=None) -> Snapshot:
    pa, sa, n = _ptr_arrays(ptrs, sizes)
    h = C.c_void_p()
    check(lib().skv_state_snapshot(ctx._h, stream, pa, sa, n, C.byref(h)))
    return Snapshot(ctx, h)


def state_restore(ctx, snapshot: Snapshot, ptrs, sizes, stream=None) -> None:
    pa, sa, n = _ptr_arrays(ptrs, sizes)
    check(lib().skv_state_restore(ctx._h, stream, snapshot._h, pa, sa, n))


class HotCache:
    """GPU prefix hot cache: page pool + chained-hash LRU index (src/serve/state.rs:560-646)."""

    def __init__(self, ctx, block_tokens, capacity_blocks, pool_blocks, layers,
                 blocks_per_session=None):
        self._ctx, self._l = ctx, lib()
        h = C.c_void_p()
        per = capacity_blocks if blocks_per_session is None else blocks_per_session
        check(self._l.skv_hot_create(ctx._h, block_tokens, capacity_blocks, per, pool_blocks,
                                     _layer_array(layers), len(layers), C.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._l.skv_hot_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def block_tokens(self): return self._l.skv_hot_block_tokens(self._h)
    def __len__(self): return self._l.skv_hot_len(self._h)
    def estimated_bytes(self): return self._l.skv_hot_bytes(self._h)
    def free_blocks(self): return self._l.skv_hot_free_blocks(self._h)
    def pool_blocks(self): return self._l.skv_hot_pool_blocks(self._h)
    def block_bytes(self): return self._l.skv_hot_block_bytes(self._h)
    def evictions(self): return self._l.skv_hot_evictions(self._h)
    def skipped(self): return self._l.skv_hot_skipped(self._h)

    def remember_prefix_block(self, session: bytes, hash_: bytes, tokens: int, layers,
                              state_ptrs=(), state_sizes=(), stream=None) -> bool:
        pa, sa, n = _ptr_arrays(list(state_ptrs), list(state_sizes))
        cached = C.c_int32()
        check(self._l.skv_hot_remember(self._h, stream, _in32(session), _in32(hash_), tokens,
                                       _layer_array(layers), len(layers), pa if n else None,
                                       sa if n else None, n, C.byref(cached)))
        return bool(cached.value)

    def remember_prefix_blocks(self, session: bytes, hashes, first_tokens: int, layers,
                               stream=None) -> int:
        """remember_prefix_block for consecutive boundaries; returns how many were kept."""
        blob = b"".join(hashes)
        buf = (C.c_uint8 * len(blob)).from_buffer_copy(blob) if blob else None
        kept = C.c_size_t()
        check(self._l.skv_hot_remember_range(self._h, stream, _in32(session), buf, first_tokens,
                                             len(hashes), _layer_array(layers), len(layers),
                                             C.byref(kept)))
        return kept.value

    def match_restore(self, root: bytes, tokens, layers, state_ptrs=(), state_sizes=(),
                      stream=None):
        """Returns (reused_tokens, hash of the last reused block or None)."""
        t = _tok(tokens)
        pa, sa, n = _ptr_arrays(list(state_ptrs), list(state_sizes))
        reused, hout = C.c_size_t(), _buf32()
        check(self._l.skv_hot_match_restore(self._h, stream, _in32(root),
                                            t.ctypes.data_as(C.c_void_p), t.size,
                                            _layer_array(layers), len(layers), pa if n else None,
                                            sa if n else None, n, C.byref(reused), hout))
        return reused.value, (bytes(hout) if reused.value else None)

    def evict_lru_block(self) -> Optional[int]:
        found, nbytes = C.c_int32(), C.c_size_t()
        check(self._l.skv_hot_evict_lru(self._h, C.byref(found), C.byref(nbytes)))
        return nbytes.value if found.value else None

    @property
    def entries(self) -> List[dict]:
        out = []
        for i in range(len(self)):
            s, h = _buf32(), _buf32()
            tok, nbytes = C.c_size_t(), C.c_size_t()
            check(self._l.skv_hot_entry(self._h, i, s, h, C.byref(tok), C.byref(nbytes)))
            out.append({"session": bytes(s), "hash": bytes(h), "tokens": tok.value,
                        "bytes": nbytes.value})
        return out


class WholePromptCache:
    """The decoder's own whole-prompt prefix cache on the GPU: prefix_cache_get /
    prefix_cache_put (src/decoder/generation.rs:2998-3025, 3105-3139). ``capacity`` None takes
    RETI_RUST_PREFIX_CACHE / RETI_RUST_PREFIX_CACHE_CAP (src/runtime_flags.rs:665-678)."""

    def __init__(self, ctx, capacity: Optional[int] = None):
        self._ctx, self._l = ctx, lib()
        h = C.c_void_p()
        if capacity is None:
            check(self._l.skv_prompt_cache_from_runtime_flags(ctx._h, C.byref(h)))
        else:
            check(self._l.skv_prompt_cache_create(ctx._h, capacity, C.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._l.skv_prompt_cache_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def __len__(self): return self._l.skv_prompt_cache_len(self._h)
    def capacity(self): return self._l.skv_prompt_cache_capacity(self._h)
    def estimated_bytes(self): return self._l.skv_prompt_cache_bytes(self._h)

    @property
    def entries(self) -> List[List[int]]:
        """Token lists of the entries, most recent first."""
        out = []
        for i in range(len(self)):
            n = C.c_size_t()
            check(self._l.skv_prompt_cache_entry(self._h, i, C.byref(n), None, 0))
            buf = np.empty(n.value, dtype=np.uint64)
            check(self._l.skv_prompt_cache_entry(self._h, i, C.byref(n), buf.ctypes.data_as(C.c_void_p), n.value))
            out.append([int(t) for t in buf])
        return out

    def put(self, prompt, layers, state_ptrs=(), state_sizes=(), stream=None) -> None:
        t = _tok(prompt)
        pa, sa, n = _ptr_arrays(list(state_ptrs), list(state_sizes))
        check(self._l.skv_prompt_cache_put(self._h, stream, t.ctypes.data_as(C.c_void_p), t.size,
                                           _layer_array(layers), len(layers), pa if n else None,
                                           sa if n else None, n))

    def lookup(self, prompt, layers, state_ptrs=(), state_sizes=(), stream=None) -> int:
        """The restore half of prefix_cache_get: tokens of the longest cached prefix now in
        ``layers`` (0 = miss)."""
        t = _tok(prompt)
        pa, sa, n = _ptr_arrays(list(state_ptrs), list(state_sizes))
        cached = C.c_size_t()
        check(self._l.skv_prompt_cache_get(self._h, stream, t.ctypes.data_as(C.c_void_p), t.size,
                                           _layer_array(layers), len(layers), pa if n else None,
                                           sa if n else None, n, C.byref(cached)))
        return cached.value

    def get(self, prompt, layers, extend: Callable[[int, int], None], state_ptrs=(), state_sizes=(),
            stream=None) -> Optional[int]:
        """prefix_cache_get (generation.rs:2998-3025): on a hit the layers hold the whole prompt
        afterwards (``extend(first, last)`` runs the model over the suffix and appends its rows,
        then the whole prompt is put) and the cached length is returned; None on a miss."""
        cached = self.lookup(prompt, layers, state_ptrs, state_sizes, stream)
        if cached == 0:
            return None
        if cached < len(prompt):
            extend(cached, len(prompt))
            self.put(prompt, layers, state_ptrs, state_sizes, stream)
        return cached
