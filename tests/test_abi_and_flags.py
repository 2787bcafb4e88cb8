"""The C-ABI library loads without a GPU, exports every symbol the header declares, and its
runtime flags parse like the reference's (src/runtime_flags.rs:25-44;
src/decode_resident/utils.rs:288-317). No compute calls here."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

import saragossa_amd as skv
from saragossa_amd import _lib, flags

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "saragossa_kv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(skv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = header_symbols()
    assert len(names) > 60
    dll = ctypes.CDLL(skv.lib_path())
    missing = [n for n in names if not hasattr(dll, n)]
    assert not missing, missing
    # the Python binding covers the whole header too
    unbound = [n for n in names if n not in _lib.SIGNATURES]
    assert not unbound, unbound
    assert skv.lib().skv_abi_version() == 1


def test_no_gpu_means_a_loud_error_not_a_fallback():
    try:
        import torch
        if torch.cuda.is_available():
            pytest.skip("a GPU is present")
    except ImportError:
        pass
    with pytest.raises(skv.DeviceError):
        skv.DecodeResidentState(0)


def test_product_package_never_imports_the_oracle():
    src = os.path.join(ROOT, "saragossa_amd")
    for dirpath, _, files in os.walk(src):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "skvo_" not in text and \
                    "from oracle" not in text, f


def test_env_flag_value_forms():
    # src/decode_resident/utils.rs:292-303
    for on in ["1", "true", "TRUE", "on", "On", " 1 "]:
        assert flags.env_flag_value(on) is True, on
    for off in ["0", "false", "FALSE", "off", "Off", " 0 "]:
        assert flags.env_flag_value(off) is False, off
    for none in ["", "2", "bf16", "yes", "no"]:
        assert flags.env_flag_value(none) is None, none


def _flags_in_subprocess(env):
    code = ("import json, saragossa_amd.flags as f; print(json.dumps(dict("
            "bf16_s=f.kv_bf16_for(True), bf16_g=f.kv_bf16_for(False), flash=f.flash_sdpa_enabled(),"
            "twopass=f.sdpa_2pass_enabled(), minlen=f.sdpa_2pass_min_len(),"
            "full=f.decode_resident_full_enabled(), res=f.decode_resident_enabled(),"
            "serve=f.serve_prefix_cache_enabled(), bt=f.serve_prefix_block_tokens(),"
            "blocks=f.serve_prefix_cache_blocks(), per=f.serve_prefix_blocks_per_session(),"
            "pc=f.prefix_cache_enabled(), cap=f.prefix_cache_capacity(), chunk=f.prefill_chunk_size(),"
            "split=f.effective_split_min_len(), simk=f.kv_bf16_sim_konly(), simv=f.kv_bf16_sim_vonly(),"
            "par=f.attention_parallel_threshold(), pipe=f.decode_pipeline_enabled(),"
            "guard=f.memory_guard_enabled(), oom=f.serve_oom_guard_enabled(), mcap=f.memory_static_cap_bytes(),"
            "mhead=f.memory_headroom_bytes(), scap=f.serve_memory_static_cap_bytes(),"
            "shead=f.serve_memory_headroom_bytes())))")
    full_env = {k: v for k, v in os.environ.items() if not k.startswith("RETI_")}
    full_env.update(env)
    full_env["PYTHONPATH"] = ROOT
    out = subprocess.run([sys.executable, "-c", code], env=full_env, capture_output=True, text=True,
                         check=True).stdout
    import json
    return json.loads(out.strip().splitlines()[-1])


def test_flag_defaults_match_the_reference():
    d = _flags_in_subprocess({})
    assert d == dict(bf16_s=True, bf16_g=False, flash=True, twopass=True, minlen=2048, full=True,
                     res=False, serve=True, bt=256, blocks=128, per=128, pc=True, cap=4, chunk=0,
                     split=128, simk=False, simv=False, par=128, pipe=True,
                     guard=True, oom=True, mcap=None, mhead=2 << 30, scap=None, shead=2 << 30)


def test_flag_overrides_and_precedence():
    # explicit RETI_RUST_KV_BF16 always wins (utils.rs:305-316); per-session cap defaults to capacity
    d = _flags_in_subprocess({"RETI_RUST_KV_BF16": "0", "RETI_RUST_FLASH_SDPA": "off",
                              "RETI_RUST_SDPA_2PASS": "FALSE", "RETI_RUST_SDPA_2PASS_MIN_LEN": "512",
                              "RETI_SERVE_PREFIX_BLOCK_TOKENS": "16",
                              "RETI_SERVE_PREFIX_CACHE_BLOCKS": "9", "RETI_RUST_PREFIX_CACHE_CAP": " 2 ",
                              "RETI_RUST_PREFILL_STEP_SIZE": "512", "RETI_SERVE_PREFIX_CACHE": "0"})
    assert (d["bf16_s"], d["bf16_g"]) == (False, False)
    assert (d["flash"], d["twopass"], d["minlen"]) == (False, False, 512)
    assert d["split"] == 512       # an explicit switch-over length is what the library uses
    assert (d["bt"], d["blocks"], d["per"], d["cap"], d["chunk"], d["serve"]) == (16, 9, 9, 2, 512, False)
    d = _flags_in_subprocess({"RETI_RUST_KV_BF16": "1", "RETI_SERVE_PREFIX_BLOCK_TOKENS": "0",
                              "RETI_SERVE_PREFIX_BLOCKS_PER_SESSION": "3",
                              "RETI_RUST_PREFILL_CHUNK": "x", "RETI_RUST_PREFILL_STEP_SIZE": "64",
                              "RETI_RUST_FLASH_SDPA": "maybe"})
    assert (d["bf16_s"], d["bf16_g"]) == (True, True)
    assert d["bt"] == 256          # zero is filtered out (runtime_flags.rs:727-736)
    assert d["per"] == 3
    assert d["chunk"] == 0         # the alias is only read when the first variable is absent
    assert d["flash"] is True      # unparsable -> default


def test_flags_are_frozen_until_reload():
    os.environ.pop("RETI_RUST_SDPA_2PASS", None)
    flags.reload()
    assert flags.sdpa_2pass_enabled() is True
    os.environ["RETI_RUST_SDPA_2PASS"] = "0"
    try:
        assert flags.sdpa_2pass_enabled() is True      # OnceLock semantics
        flags.reload()
        assert flags.sdpa_2pass_enabled() is False
    finally:
        os.environ.pop("RETI_RUST_SDPA_2PASS", None)
        flags.reload()


def test_integer_helpers_match_the_oracle():
    import oracle
    for n in [0, 1, 127, 128, 2047, 2048, 4096, 8193, 32768, 33000, 131072, 10 ** 7]:
        assert flags.sdpa_2pass_blocks(n) == oracle.sdpa_2pass_blocks(n)
    for pos, w in [(0, 0), (0, 4), (3, 4), (4, 4), (1023, 1024), (1024, 1024), (70000, 1024)]:
        assert flags.window_start(pos, w) == oracle.window_start(pos, w)
    big = 2 ** 64 - 1
    for a, b, c in [(0, 0, 0), (2048, 256, 0), (2048, 256, 4), (big, 0, 0), (big, 1, 0), (big - 5, 3, 3)]:
        try:
            want = oracle.resident_capacity(a, b, c)
        except oracle.OracleError:
            want = None
        assert flags.resident_capacity(a, b, c) == want
    for x in [1.0039062, -0.33325195, 42.125, 0.0, 1e-40, 3.3895314e38]:
        assert flags.f32_to_bf16_bits(x) == int(oracle.f32_to_bf16_bits([x])[0])


def test_diagnostic_and_host_loop_flags():
    # src/decode_resident/utils.rs:245-256; src/runtime_flags.rs:309-313, 641-649
    d = _flags_in_subprocess({"RETI_RUST_KV_BF16_SIM_KONLY": "1", "RETI_RUST_KV_BF16_SIM_VONLY": "on",
                              "RETI_RUST_ATTENTION_PAR_THRESHOLD": " 4096 ", "RETI_RUST_DECODE_PIPELINE": "0",
                              "RETI_RUST_SDPA_2PASS_MIN_LEN": "junk"})
    assert (d["simk"], d["simv"], d["par"], d["pipe"]) == (True, True, 4096, False)
    assert d["split"] == 2048 and d["minlen"] == 2048   # set but unparsable: the reference's default
    d = _flags_in_subprocess({"RETI_RUST_ATTENTION_PAR_THRESHOLD": "-1", "RETI_RUST_DECODE_PIPELINE": "x"})
    assert (d["par"], d["pipe"]) == (128, True)


def test_memory_projection_is_the_reference_guard_arithmetic():
    # check_allocation_accepts_boundary_and_rejects_overflow (src/memory_guard.rs:748-766):
    # current 100, cap 150: 50 passes, 51 is refused with available 50 and projected 151
    assert flags.memory_projection(100, 0, 50, 150) == (False, 150, 50)
    assert flags.memory_projection(100, 0, 51, 150) == (True, 151, 50)
    # reservations_are_counted_until_drop (memory_guard.rs:768-786): 100 + 60 reserved, cap 180
    assert flags.memory_projection(100, 60, 20, 180)[0] is False
    assert flags.memory_projection(100, 60, 21, 180)[0] is True
    big = 2 ** 64 - 1
    assert flags.memory_projection(big, 5, 7, big) == (False, big, 0)      # saturating adds
    assert flags.memory_projection(10, 0, 1, 5) == (True, 11, 0)           # available floors at 0


def test_resident_kv_bytes_and_layer_bytes():
    # check_resident_full_decode_allocation (src/decoder/resident/setup.rs:897-917): 2 * capacity *
    # kv_dim * size_of::<f32>() per full-attention layer
    assert flags.resident_kv_bytes(2304, [1024] * 36) == 36 * 2 * 2304 * 1024 * 4
    assert flags.resident_kv_bytes(10, []) == 0
    assert flags.resident_kv_bytes(2 ** 62, [1024]) is None              # "KV résident déborde"
    # what skv_layer_create takes: whole pages of K and V, table, split partials, staging rows
    bf = flags.layer_bytes(32768 + 300, 16, 2, 256, skv.DTYPE_BF16)
    f32 = flags.layer_bytes(32768 + 300, 16, 2, 256, skv.DTYPE_F32)
    pages = (32768 + 300 + 15) // 16
    pools = 2 * pages * 2 * 256 * 16 * 2
    partials = 512 * 16 * (256 + 2) * 4   # the most splits a launch can take
    assert pools + partials <= bf < pools + partials + 2 ** 16
    assert 2 * pools + partials <= f32 < 2 * pools + partials + 2 ** 16
    # a ring layer's size follows its window (plus 32 rows of slack), not its capacity
    ring = flags.layer_bytes(65536, 16, 8, 256, skv.DTYPE_BF16, 1024)
    assert 2 * 66 * 8 * 256 * 16 * 2 < ring < 2 * 66 * 8 * 256 * 16 * 2 * 1.2
    # padded head_dim: 80 -> 128
    assert flags.layer_bytes(1024, 8, 8, 80, skv.DTYPE_BF16) > 2 * 64 * 8 * 128 * 16 * 2
    for bad in [(0, 16, 2, 256), (16, 0, 2, 256), (16, 16, 3, 256), (16, 16, 2, 513)]:
        with pytest.raises(skv.ConfigError):
            flags.layer_bytes(*bad, skv.DTYPE_BF16)
    with pytest.raises(skv.ConfigError):
        flags.layer_bytes(16, 16, 2, 256, 7)


def test_memory_guard_flags_follow_the_reference():
    # src/runtime_flags.rs:693-724, 773-792: the serve guard needs the shared guard; a cap of zero or
    # an unparsable one is no cap; headrooms default to 2 GiB and accept surrounding blanks
    d = _flags_in_subprocess({"RETI_MEMORY_GUARD": "0"})
    assert (d["guard"], d["oom"]) == (False, False)
    d = _flags_in_subprocess({"RETI_SERVE_OOM_GUARD": "off"})
    assert (d["guard"], d["oom"]) == (True, False)
    d = _flags_in_subprocess({"RETI_MEMORY_CAP_BYTES": " 1000000 ", "RETI_SERVE_MEMORY_CAP_BYTES": "0",
                              "RETI_MEMORY_HEADROOM_BYTES": "0", "RETI_SERVE_MEMORY_HEADROOM_BYTES": "12x"})
    assert (d["mcap"], d["scap"], d["mhead"], d["shead"]) == (1000000, None, 0, 2 << 30)
    d = _flags_in_subprocess({"RETI_MEMORY_CAP_BYTES": "-5", "RETI_SERVE_MEMORY_CAP_BYTES": "68719476736",
                              "RETI_SERVE_MEMORY_HEADROOM_BYTES": " 1073741824"})
    assert (d["mcap"], d["scap"], d["shead"]) == (None, 1 << 36, 1 << 30)
