"""The native host side (SHA-256 chain, prefix index) under AddressSanitizer + UBSan: a
g++ build of saragossa_amd/csrc/prefix.cpp and flags.cpp with tests/native/prefix_sanitize.cpp,
which replays 20000 random inserts, matches and evictions against a vector model of
BlockAwarePrefixCache (src/serve/cache.rs:72-219). Host code only; no GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "saragossa_amd", "csrc")


@pytest.mark.skipif(shutil.which("g++") is None, reason="g++ not available")
def test_prefix_index_under_sanitizers(tmp_path):
    exe = tmp_path / "prefix_sanitize"
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-omit-frame-pointer",
           "-fno-sanitize-recover=undefined", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + CSRC,
           "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "native", "prefix_sanitize.cpp"),
           os.path.join(CSRC, "prefix.cpp"), os.path.join(CSRC, "flags.cpp"), "-o", str(exe)]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0")
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0, (run.stdout[-1000:], run.stderr[-3000:])
    assert run.stdout.strip().endswith("ok")
