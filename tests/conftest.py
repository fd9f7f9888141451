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
def frontend():
    """Front end with the CPU oracle registered as backend 'c' (and 'openmp')."""
    from harp_amd import frontend as fe
    from oracle.c_backend import CBackend
    fe.register_backend(CBackend())
    fe.register_backend(CBackend(openmp=True))
    fe.register_backend(CBackend(exact_division=True))
    return fe


@pytest.fixture(scope="session")
def hip(frontend):
    """Front end with the HIP backend registered; skips when no GPU is present."""
    from harp_amd import backend as hb
    if hb.device_count() == 0:
        pytest.skip("no HIP device")
    hb.init()
    return hb


def realize_on(fe, kind, build, arrays, fuse=None):
    """Builds the graph on fresh input tensors bound to backend `kind`, realizes
    it and returns the flat result."""
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    fe.set_device_str(kind)
    old = os.environ.get("ECLAT_HIP_FUSE")
    if fuse is not None:
        os.environ["ECLAT_HIP_FUSE"] = "1" if fuse else "0"
    try:
        tensors = []
        for a in arrays:
            t = fe.Tensor.input(list(a.shape), fe.DType({np.dtype("float32"): "f32",
                                                         np.dtype("int32"): "i32",
                                                         np.dtype("int64"): "i64",
                                                         np.dtype("float64"): "f64"}[a.dtype]))
            t.set_data(a)
            tensors.append(t)
        y = build(*tensors)
        y.realize()
        return y.to_numpy()
    finally:
        _INPUT_BUFFER_CACHE.clear()
        if fuse is not None:
            if old is None:
                os.environ.pop("ECLAT_HIP_FUSE", None)
            else:
                os.environ["ECLAT_HIP_FUSE"] = old


def bits_equal_mod_zero(a: np.ndarray, b: np.ndarray) -> bool:
    """Bit-exact, except that +0/-0 (and flushed denormals) count as equal: the
    oracle is built with -ffast-math (no signed zeros, FTZ/DAZ)."""
    a = np.ascontiguousarray(a, dtype=np.float32).ravel()
    b = np.ascontiguousarray(b, dtype=np.float32).ravel()
    if a.shape != b.shape:
        return False
    same = a.view(np.uint32) == b.view(np.uint32)
    tiny = np.float32(1.1754944e-38)
    both_zero = (np.abs(a) < tiny) & (np.abs(b) < tiny)
    return bool(np.all(same | both_zero))
