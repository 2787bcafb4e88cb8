import os
import sys

import numpy as np
import pytest

# torch ships its own copy of the HIP runtime. A process can initialise only one: whichever
# of torch and libsaragossa_kv.so is loaded first decides which copy both then use, and torch
# finds no GPU on a runtime that is not its own. The GPU tests use torch tensors as device
# memory, so torch goes first here.
try:
    import torch  # noqa: F401
except ImportError:
    pass

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pseudo(seed):
    """Deterministic data in [-0.1, 0.1], the generator of the reference's attention tests
    (src/decode_resident/tests.rs:544-547); `seed` may be an integer array."""
    s = np.asarray(seed, dtype=np.uint64)
    x = ((s * np.uint64(2654435761)) ^ np.uint64(0x9E3779B9)) % np.uint64(1000)
    return ((x.astype(np.float32) / np.float32(1000.0) - np.float32(0.5)) * np.float32(0.2)).astype(np.float32)


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


@pytest.fixture(scope="session")
def state():
    """try_state() of the reference tests (src/decode_resident/tests.rs:34-42), except that a
    missing device is a failure here: GPU tests must run on the GPU."""
    import saragossa_amd
    st = saragossa_amd.DecodeResidentState(0)
    yield st
    st.close()
