"""MI355X-native KV-cache hot path of saragossa: thin Python host mirror over the C ABI.

The product is ``libsaragossa_kv.so`` (hand-written gfx950 kernels behind
``include/saragossa_kv.h``). This package only binds it with ctypes and mirrors
the reference's Rust method names so the parity tests read like the reference's
own tests. There is no CPU fallback: without the library, or without a GPU,
every compute call raises.
"""
from ._lib import (KvError, DimensionError, ConfigError, DeviceError, MemoryGuardError, lib, lib_path,
                   DTYPE_BF16, DTYPE_F32, PAGE_ROWS)
from .kv import (DecodeResidentState, FullAttentionState, RopeTable, encode_decode_step_batch,
                 rope_rotations)
from . import flags
from .serve import LoadedModelKv
from .prefix import (BlockHash, BlockAwarePrefixCache, PrefixBlockHit, HotCache, Snapshot, WholePromptCache,
                     snapshot_blocks, restore_blocks, state_snapshot, state_restore)

__all__ = ["KvError", "DimensionError", "ConfigError", "DeviceError", "MemoryGuardError", "lib", "lib_path",
           "DecodeResidentState", "FullAttentionState", "encode_decode_step_batch", "RopeTable", "rope_rotations", "flags", "DTYPE_BF16", "DTYPE_F32",
           "PAGE_ROWS", "BlockHash", "BlockAwarePrefixCache", "PrefixBlockHit", "HotCache",
           "LoadedModelKv", "Snapshot", "WholePromptCache", "snapshot_blocks", "restore_blocks", "state_snapshot", "state_restore"]
