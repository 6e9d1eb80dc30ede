import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lm():
    """The luminal.jl_amd package (its directory name is not importable as a dotted module)."""
    import __graft_entry__
    return __graft_entry__.load_package()


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle
    _oracle.lib()
    return _oracle


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "attention_cases.npz")
    data = np.load(path)  # allow_pickle stays False
    names = sorted({k.rsplit(".", 1)[0] for k in data.files})
    cases = {}
    for n in names:
        c = {}
        for key in ("q", "k", "v"):
            c[key] = (data[n + "." + key].astype(np.uint32) << np.uint32(16)).view(np.float32)
        c["out"] = data[n + ".out"]
        c["causal"] = bool(data[n + ".meta"][0])
        c["scale"] = float(data[n + ".meta"][1])
        c["kv_len"] = data[n + ".kv_len"] if (n + ".kv_len") in data.files else None
        cases[n] = c
    return cases


@pytest.fixture(scope="session")
def hip(lm):
    """HIP device for the gpu-marked tests. No device (or no built library) is a failure, not a skip:
    a GPU run that silently tested nothing must not look green."""
    dev = lm.get_device()
    assert isinstance(dev, lm.HIPDevice), "no gfx950 device visible to libluminal_hip.so"
    return dev


def rel_err(got, want):
    """max |got - want| / max |want| — the parity metric of the benchmark contract."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.all(np.isfinite(got)), "non-finite values in result"
    return float(np.abs(got - want).max() / np.abs(want).max())


TOL = {"f32": 1e-5, "f16": 2e-3, "bf16": 2e-3}
