"""A random-init Qwen3-shaped decoder for BASELINE configs[1], with its KV path (append +
attention, chunked prefill over the cache) on the HIP library. Everything that is not the KV
path (embedding, RMSNorm, the q/k/v/o and MLP projections, q/k norm + rotate-half RoPE,
lm_head, first-max argmax) is plain torch fp32 on the GPU; layer wiring follows the reference's
CPU forward (src/decoder/attention.rs:621-712, src/decoder/attention_ops.rs:223-322,
src/decoder/generation.rs:336-362). Used by the end-to-end leg of bench.py and, next to the CPU
oracle's KV path (config1_model.py), by the greedy-parity test. Nothing here touches the oracle."""
from __future__ import annotations

import numpy as np
import torch

import saragossa_amd as skv  # noqa: F401  (the KV classes take a DecodeResidentState from it)


class Config:
    def __init__(self, layers=36, hidden=2560, q_heads=32, kv_heads=8, head_dim=128, mlp=9728,
                 vocab=151936, theta=1.0e6, eps=1.0e-6):
        self.__dict__.update(locals())
        del self.__dict__["self"]


class Weights:
    """N(0, 0.02) projections, unit norms, tied lm_head; generated on the GPU from a seed."""

    def __init__(self, cfg: Config, seed: int):
        g = torch.Generator(device="cuda").manual_seed(seed)
        r = lambda *s: torch.randn(*s, device="cuda", dtype=torch.float32, generator=g) * 0.02
        q_dim, kv_dim = cfg.q_heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim
        self.embed = r(cfg.vocab, cfg.hidden)
        self.layers = []
        for _ in range(cfg.layers):
            self.layers.append(dict(wq=r(q_dim, cfg.hidden), wk=r(kv_dim, cfg.hidden),
                                    wv=r(kv_dim, cfg.hidden), wo=r(cfg.hidden, q_dim),
                                    wg=r(cfg.mlp, cfg.hidden), wu=r(cfg.mlp, cfg.hidden),
                                    wd=r(cfg.hidden, cfg.mlp)))
        self.ones_h = torch.ones(cfg.hidden, device="cuda")
        self.ones_d = torch.ones(cfg.head_dim, device="cuda")


def rms_norm(x, w, eps):
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def norm_rope(x, heads, head_dim, w, eps, theta, positions):
    """Per-head RMSNorm then rotate-half RoPE at `positions` (rms_norm_rope_heads_at)."""
    s = x.shape[0]
    xh = rms_norm(x.view(s, heads, head_dim), w, eps)
    half = head_dim // 2
    inv = theta ** (-torch.arange(0, half, device=x.device, dtype=torch.float32) * 2.0 / head_dim)
    ang = positions.to(torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = xh[..., :half], xh[..., half:]
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1).reshape(s, heads * head_dim)


class HipKv:
    """KV path on the HIP library: paged bf16 caches behind permuted block tables."""
    ELEMENT = "bf16"

    def __init__(self, cfg, capacity, state, seed=0):
        rng = np.random.default_rng(seed)
        self.layers = []
        make = state.full_attention_f32 if self.ELEMENT == "f32" else state.full_attention_bf16
        for _ in range(cfg.layers):
            kv = make(capacity, cfg.q_heads, cfg.kv_heads, cfg.head_dim)
            kv.set_block_table(rng.permutation(kv.pages()).astype(np.int32))
            self.layers.append(kv)
        self.stream = torch.cuda.current_stream().cuda_stream

    def attend(self, li, q, k, v):
        out = torch.empty_like(q)
        kv = self.layers[li]
        if q.shape[0] == 1:
            kv.encode_decode_step(self.stream, k.data_ptr(), 0, v.data_ptr(), 0, q.data_ptr(),
                                  out.data_ptr())
        else:
            kv.encode_prefill_rows(self.stream, q.data_ptr(), k.data_ptr(), v.data_ptr(), q.shape[0],
                                   out.data_ptr())
        return out

    def contents(self, li):
        return self.layers[li].read_rows_f32()


class HipKvF32(HipKv):
    """The same with the f32 element: the reference's choice for greedy decoding."""
    ELEMENT = "f32"


class HipKvPre(HipKv):
    """As HipKv, but a decode token hands the raw q and k projections to the library, which
    applies the q/k norms and the rotation itself (the fused step before the cache), and prefill
    chunks go through the library's multi-row norm + rotation; the other arm takes both from
    the CPU oracle."""
    raw_qk = True

    def __init__(self, cfg, capacity, state, seed=0):
        super().__init__(cfg, capacity, state, seed)
        self.cfg = cfg
        self.state = state
        self.rope = state.rope_table(capacity, cfg.head_dim, cfg.theta)
        self.ones = torch.ones(cfg.head_dim, device="cuda")

    def attend_raw(self, li, q_raw, k_raw, v, position):
        cfg = self.cfg
        if q_raw.shape[0] == 1:
            out = torch.empty_like(q_raw)
            self.layers[li].encode_decode_step_prekv(
                self.stream, self.rope, position, q_raw.data_ptr(), 0, k_raw.data_ptr(), 0,
                v.data_ptr(), 0, self.ones.data_ptr(), self.ones.data_ptr(), cfg.eps,
                float(cfg.head_dim), out.data_ptr())
            return out
        # a prefill chunk: the library's multi-row norm + rotation, then chunked prefill
        q, k = torch.empty_like(q_raw), torch.empty_like(k_raw)
        n = q_raw.shape[0]
        self.state.encode_rms_norm_rope_rows(self.stream, self.rope, position, q_raw.data_ptr(),
                                             self.ones.data_ptr(), n, cfg.q_heads, cfg.head_dim, cfg.eps,
                                             q.data_ptr())
        self.state.encode_rms_norm_rope_rows(self.stream, self.rope, position, k_raw.data_ptr(),
                                             self.ones.data_ptr(), n, cfg.kv_heads, cfg.head_dim, cfg.eps,
                                             k.data_ptr())
        return self.attend(li, q, k, v)


def forward(cfg, w, kv, tokens, position):
    """Runs `tokens` (a chunk, or one token) at positions position.. and returns the last
    row's logits."""
    ids = torch.as_tensor(tokens, device="cuda", dtype=torch.long)
    pos = torch.arange(position, position + ids.numel(), device="cuda")
    x = w.embed[ids]
    for li, lw in enumerate(w.layers):
        h = rms_norm(x, w.ones_h, cfg.eps)
        v = (h @ lw["wv"].T).contiguous()
        if getattr(kv, "raw_qk", False):
            ctx = kv.attend_raw(li, (h @ lw["wq"].T).contiguous(), (h @ lw["wk"].T).contiguous(), v,
                                position)
        else:
            q = norm_rope(h @ lw["wq"].T, cfg.q_heads, cfg.head_dim, w.ones_d, cfg.eps, cfg.theta, pos)
            k = norm_rope(h @ lw["wk"].T, cfg.kv_heads, cfg.head_dim, w.ones_d, cfg.eps, cfg.theta, pos)
            ctx = kv.attend(li, q.contiguous(), k.contiguous(), v)
        x = x + ctx @ lw["wo"].T
        h2 = rms_norm(x, w.ones_h, cfg.eps)
        x = x + (torch.nn.functional.silu(h2 @ lw["wg"].T) * (h2 @ lw["wu"].T)) @ lw["wd"].T
    final = rms_norm(x[-1:], w.ones_h, cfg.eps)
    return (final @ w.embed.T)[0]


def greedy(cfg, w, kv, prompt, n_new, chunk):
    """Chunked prefill over the cache, then n_new greedy steps. Returns (ids, top-1 minus
    top-2 margin per step, logits per step on the CPU)."""
    position = 0
    logits = None
    for i in range(0, len(prompt), chunk):
        part = prompt[i:i + chunk]
        logits = forward(cfg, w, kv, part, position)
        position += len(part)
    ids, margins, all_logits = [], [], []
    for _ in range(n_new):
        top = torch.topk(logits, 2)
        # first-max argmax (src/sampling.rs:49-62): torch.argmax returns the first maximal index
        tok = int(torch.argmax(logits))
        ids.append(tok)
        margins.append(float(top.values[0] - top.values[1]))
        all_logits.append(logits[:4096].cpu().numpy().copy())
        logits = forward(cfg, w, kv, [tok], position)
        position += 1
    return ids, margins, all_logits
