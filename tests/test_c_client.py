"""The boundary as a foreign-function binding sees it: include/saragossa_kv.h must be a
valid strict-C11 header, and a plain C program (tests/native/kv_c_client.c: no C++, no
Python, no torch) linked against libsaragossa_kv.so must seed, append, read back bit-exact
contents and get decode attention right. The program is compiled by
`__graft_entry__.build()`; the GPU test runs it."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "native", "kv_c_client.c")
EXE = os.path.join(ROOT, "tests", "native", "kv_c_client")
EXE_REMEMBER = os.path.join(ROOT, "tests", "native", "kv_c_remember")


def compile_c_client():
    import __graft_entry__ as entry
    entry.build_c_client()


@pytest.mark.skipif(shutil.which("gcc") is None, reason="gcc not available")
def test_header_is_strict_c11_and_cxx17():
    for cmd in (["gcc", "-std=c11", "-x", "c"], ["g++", "-std=c++17", "-x", "c++"]):
        run = subprocess.run(cmd + ["-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only",
                                    os.path.join(ROOT, "include", "saragossa_kv.h")],
                             capture_output=True, text=True, timeout=120)
        assert run.returncode == 0, run.stderr[-2000:]


@pytest.mark.skipif(shutil.which("gcc") is None, reason="gcc not available")
def test_c_client_compiles_and_links_against_the_library():
    compile_c_client()
    assert os.path.exists(EXE) and os.path.exists(EXE_REMEMBER)


@pytest.mark.gpu
def test_c_client_runs_on_the_gpu():
    if not os.path.exists(EXE):
        compile_c_client()
    run = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.stdout[-500:], run.stderr[-2000:])
    assert run.stdout.strip().endswith("ok")


@pytest.mark.gpu
def test_c_remember_client_caches_every_block_one_call_per_boundary():
    """256 block boundaries of a 4096-token prefix over 36 layers, one skv_hot_remember per
    boundary from plain C: every block is cached, and a call costs a native host a few
    microseconds (the bound here is loose: it catches a synchronisation or an allocation
    per call, not a slow machine)."""
    import json
    if not os.path.exists(EXE_REMEMBER):
        compile_c_client()
    run = subprocess.run([EXE_REMEMBER], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.stdout[-500:], run.stderr[-2000:])
    rep = json.loads(run.stdout.strip().splitlines()[-1])
    assert rep["calls"] == 256 and rep["cached"] == 256
    assert rep["host_us_per_call"] < 40.0, rep
