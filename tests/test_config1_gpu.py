"""BASELINE configs[1]: random-init Qwen3-4B-shaped decoder, chunked prefill over the cache,
then greedy decode; token ids with the HIP KV path must equal the ids with the CPU oracle's
KV path, and the caches must hold the same rows. The "kv-path" arm runs at full size: 36
layers, 2048-token prompt in 512-row chunks, 256 greedy steps (about a minute per arm, nearly all
of it the oracle's per-row CPU prefill). All three arms run at full size; SKV_REDUCED_CONFIG1=1
cuts the "fused-pre-kv" and "f32-element" arms to 12 of the 36 layers and a 1024-token prompt
for a quick run."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

from config1_model import (Config, HipKv, HipKvF32, HipKvPre, OracleKv, OracleKvF32, OracleKvPre,  # noqa: E402
                           Weights, greedy)

FULL = os.environ.get("SKV_REDUCED_CONFIG1") != "1"


@pytest.mark.timeout(900)
@pytest.mark.parametrize("hip_cls,ora_cls", [(HipKv, OracleKv), (HipKvPre, OracleKvPre), (HipKvF32, OracleKvF32)],
                         ids=["kv-path", "fused-pre-kv", "f32-element"])
def test_config1_greedy_ids_match_oracle(state, hip_cls, ora_cls):
    """ids "fused-pre-kv": decode tokens additionally run the q/k norms and the rotation
    inside the library's fused step (device) against rms_norm_rope_heads_at (CPU).
    "f32-element": both arms keep f32 rows, as the reference does for greedy decoding."""
    full = FULL or hip_cls is HipKv
    cfg = Config() if full else Config(layers=12)
    n_prompt, n_new, chunk = (2048, 256, 512) if full else (1024, 96, 256)
    w = Weights(cfg, seed=1)
    prompt = [int(t) for t in np.random.default_rng(1).integers(0, cfg.vocab, size=n_prompt)]
    cap = n_prompt + n_new
    with torch.no_grad():
        hip = hip_cls(cfg, cap, state)
        ids_hip, margins, logits_hip = greedy(cfg, w, hip, prompt, n_new, chunk)
        ora = ora_cls(cfg)
        ids_ora, _, logits_ora = greedy(cfg, w, ora, prompt, n_new, chunk)
    print(f"config1 {'full' if full else 'reduced'}: min top-1/top-2 margin {min(margins):.3e}, "
          f"max |logit diff| {max(float(np.abs(a - b).max()) for a, b in zip(logits_hip, logits_ora)):.3e}")
    first_diff = next((i for i, (a, b) in enumerate(zip(ids_hip, ids_ora)) if a != b), None)
    if first_diff is not None:
        print(f"first differing step {first_diff}: margin there {margins[first_diff]:.3e}")
    assert ids_hip == ids_ora
    assert len(set(ids_hip)) > 1          # not a degenerate constant continuation
    # Cache contents after the run. Layer 0's K/V depend on the embeddings only, so both arms
    # append the same f32 rows and the caches must agree bit for bit. Deeper layers receive
    # hidden states that already carry the arms' last-bit attention differences; bf16 rounding
    # of K/V amplifies those (a 1e-6 change tips a rounding now and then, the tipped element
    # moves the next layer's scores by 1e-4), so there the appended inputs themselves differ and
    # only closeness is checked.
    for li in sorted({0, cfg.layers // 2, cfg.layers - 1}):
        gk, gv = hip.contents(li)
        ok, ov = ora.contents(li)
        assert gk.shape == ok.shape == (cap, cfg.kv_heads * cfg.head_dim)
        if li == 0:
            assert np.array_equal(gk, ok) and np.array_equal(gv, ov)
        else:
            for g, o in ((gk, ok), (gv, ov)):
                assert np.abs(g - o).max() <= 0.1 and np.abs(g - o).mean() <= 1e-3
