import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    return np.load(os.path.join(GOLDEN_DIR, "golden_small.npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def golden_cfg4():
    p = os.path.join(GOLDEN_DIR, "golden_cfg4.npz")
    if not os.path.exists(p):
        pytest.skip("golden_cfg4.npz not generated")
    return np.load(p, allow_pickle=False)


@pytest.fixture(scope="session")
def golden_sampling():
    """Tokens the compiled reference's sample_token drew for synth.SAMPLING_CASES, in order."""
    return np.load(os.path.join(GOLDEN_DIR, "golden_sampling.npz"), allow_pickle=False)["tokens"]


@pytest.fixture(scope="session")
def seeds():
    import json
    with open(os.path.join(GOLDEN_DIR, "golden_meta.json")) as f:
        return json.load(f)["seeds"]


@pytest.fixture(scope="session")
def po():
    """The CPU oracle (test infrastructure)."""
    from oracle import pyoracle
    pyoracle.lib()
    return pyoracle


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from prometorch_amd import _lib
    _lib.load()  # raises if the HIP library is not built: GPU tests must never run on a fallback
    torch.cuda.set_device(0)
    return torch.device("cuda:0")


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def sha(a):
    import hashlib
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def sha_of(golden, key):
    return bytes(golden[key]).decode()
