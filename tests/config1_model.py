"""The CPU oracle's KV path for the random-init decoder of config1_hip.py: BASELINE configs[1]
is checked by running greedy decode with the KV path served either by the HIP library
(config1_hip.py) or by the classes below; everything else is the same torch code in both arms,
so only the attention arithmetic differs."""
from __future__ import annotations

import numpy as np
import torch

import oracle
from config1_hip import (Config, HipKv, HipKvF32, HipKvPre, Weights, forward, greedy, norm_rope,  # noqa: F401
                         rms_norm)


class OracleKv:
    """KV path on the CPU oracle with K/V rounded to bf16 at append (mode bf16r)."""
    MODE = "bf16r"

    def __init__(self, cfg, capacity=None, state=None, seed=0):
        self.lay = oracle.layout(cfg.q_heads, cfg.kv_heads, cfg.head_dim)
        self.caches = [oracle.LayerKvCache(self.MODE) for _ in range(cfg.layers)]

    def attend(self, li, q, k, v):
        qn, kn, vn = q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()
        if qn.shape[0] == 1:
            out = oracle.decode_step(self.caches[li], kn[0], vn[0], qn[0], self.lay)[None]
        else:
            out = oracle.cached_attention_prefill_rows(qn, kn, vn, self.caches[li], self.lay)
        return torch.from_numpy(out).cuda()

    def contents(self, li):
        return self.caches[li].keys(), self.caches[li].values()


class OracleKvF32(OracleKv):
    """The CPU path as it is: f32 rows."""
    MODE = "f32"


def norm_rope_cpu(x, heads, cfg, position):
    """rms_norm_rope_heads_at on the CPU oracle (unit norm weights), rows at position.."""
    ones = np.ones(cfg.head_dim, np.float32)
    return oracle.rms_norm_rope_heads_at(x.cpu().numpy(), heads, cfg.head_dim, cfg.head_dim, ones,
                                         cfg.eps, cfg.theta, position)


class OracleKvPre(OracleKv):
    """The CPU path end to end for the attention block: rms_norm_rope_heads_at, append,
    cached_attention_one."""
    raw_qk = True

    def __init__(self, cfg, capacity=None, state=None, seed=0):
        super().__init__(cfg, capacity, state, seed)
        self.cfg = cfg

    def attend_raw(self, li, q_raw, k_raw, v, position):
        q = torch.from_numpy(norm_rope_cpu(q_raw, self.cfg.q_heads, self.cfg, position)).cuda()
        k = torch.from_numpy(norm_rope_cpu(k_raw, self.cfg.kv_heads, self.cfg, position)).cuda()
        return self.attend(li, q, k, v)


