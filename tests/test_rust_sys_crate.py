"""The Rust -sys crate (rust/saragossa-kv-hip-sys) binds the whole header: its lib.rs is what
gen_bindings.py writes from include/saragossa_kv.h today, and, checked independently of the
generator, it declares every prototype of the header with the same number of arguments and every
#define as a constant. (No Rust toolchain exists in this image; the crate is not compiled here.)"""
import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CRATE = os.path.join(ROOT, "rust", "saragossa-kv-hip-sys")


def _generator():
    spec = importlib.util.spec_from_file_location("gen_bindings", os.path.join(CRATE, "gen_bindings.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _header_prototypes():
    """name -> argument count, parsed here with nothing shared with the generator."""
    text = open(os.path.join(ROOT, "include", "saragossa_kv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(skv_[a-z0-9_]+)\s*\(([^()]*)\)\s*;", text):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
    return out


def _rust_prototypes():
    text = open(os.path.join(CRATE, "src", "lib.rs")).read()
    out = {}
    for m in re.finditer(r"pub fn (skv_[a-z0-9_]+)\(([^()]*)\)", text):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if not args else args.count(",") + 1
    return out


def test_lib_rs_is_what_the_generator_writes_from_the_header():
    assert open(os.path.join(CRATE, "src", "lib.rs")).read() == _generator().generate()


def test_lib_rs_declares_every_prototype_with_the_same_argument_count():
    c, r = _header_prototypes(), _rust_prototypes()
    assert len(c) > 100
    assert sorted(c) == sorted(r)
    assert {n: k for n, k in c.items() if r[n] != k} == {}


def test_lib_rs_carries_the_constants_and_handle_types():
    text = open(os.path.join(CRATE, "src", "lib.rs")).read()
    header = open(os.path.join(ROOT, "include", "saragossa_kv.h")).read()
    for name, value in re.findall(r"^#define\s+(SKV_[A-Z0-9_]+)\s+(-?\d+)\b", header, flags=re.M):
        assert re.search(r"pub const %s: \w+ = %s;" % (name, value), text), name
    assert "pub const SKV_STATIC_SCRATCH_BYTES: usize = 8 << 20;" in text
    for handle in re.findall(r"typedef struct (skv_[a-z_]+) \1;", header):
        assert "pub struct %s " % handle in text, handle
    assert "pub struct skv_hit { pub tokens: usize, pub hash: [u8; 32], pub payload: u64, pub matched_blocks: usize }" in text


def test_pointer_mutability_follows_the_c_declarations():
    text = open(os.path.join(CRATE, "src", "lib.rs")).read()
    # T *const *  -> *const *mut T ; const T *const * -> *const *const T ; out parameters are *mut
    assert "seqs: *const *mut skv_layer" in text
    assert "k_dev: *const *const c_void" in text
    assert "out_dev: *const *mut f32" in text
    assert "pub fn skv_ctx_create(device: i32, out: *mut *mut skv_ctx) -> i32;" in text
    assert "pub fn skv_hash_root(out: *mut u8);" in text
    assert "pub fn skv_last_error() -> *const c_char;" in text
    assert "pub fn skv_len(layer: *const skv_layer) -> usize;" in text
