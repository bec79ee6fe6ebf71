import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# The tests run in the library's default layout (slices packed, stride = heap
# size).  The spread layout (ROCSHMEM_EMU_SPREAD=1) only changes bandwidth, not
# results; the full-size tests, test_spread_layout_is_opt_in and bench.py run in it.
os.environ.pop("ROCSHMEM_EMU_SPREAD", None)
os.environ.pop("ROCSHMEM_EMU_PE_STRIDE", None)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    from oracle import pyoracle
    return pyoracle


@pytest.fixture(scope="session")
def L():
    """The product's ctypes module (enumerations + loader)."""
    from rocshmem_amd import lib
    return lib


class Runtime:
    """The library brought up with a given number of PEs and heap size;
    re-initialised on demand, since one process hosts one runtime at a time."""

    def __init__(self, L):
        self.L = L
        self.l = L.load()
        self.npes = 0
        self.heap = 0

    def up(self, npes, heap):
        if self.npes == npes and self.heap == heap:
            return self.l
        if self.npes:
            self.l.finalize()
        assert self.l.init(npes, heap) == 0
        self.npes, self.heap = npes, heap
        return self.l

    def down(self):
        if self.npes:
            self.l.finalize()
        self.npes = self.heap = 0

    # ---- helpers over the C entry points -----------------------------------
    def put_bytes(self, dev_ptr, array):
        a = np.ascontiguousarray(array)
        assert self.l.copy_in(dev_ptr, a.ctypes.data, a.nbytes) == 0

    def get_bytes(self, dev_ptr, nbytes, dtype=np.uint8):
        out = np.empty(nbytes // np.dtype(dtype).itemsize, dtype)
        assert self.l.copy_out(out.ctypes.data, dev_ptr, nbytes) == 0
        return out

    def dev_array(self, array):
        """Plain device copy of a host array; caller frees with dev_free."""
        a = np.ascontiguousarray(array)
        p = self.l.dev_alloc(max(a.nbytes, 1))
        if a.nbytes:
            self.l.copy_in(p, a.ctypes.data, a.nbytes)
        return p


@pytest.fixture(scope="session")
def rt(L):
    r = Runtime(L)
    yield r
    r.down()
