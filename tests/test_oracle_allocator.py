"""Pins the oracle's allocator restatement and the product's host allocator.

Three implementations are compared on the same request sequences:
  reference  the reference's own Pow2Bins/Binner/Bin/AddressRecord headers,
             compiled into oracle/_ref (skipped where that library is absent)
  oracle     oracle/oracle.cpp orc_heap_*
  product    rocshmem_amd/csrc/pow2_allocator.hpp through the
             rocshmem_amd_heap_model_* entry points (no GPU needed)
plus the known answers of the reference's unit tests.
"""
import numpy as np
import pytest

GiB = 1 << 30
BASE = 0x7F0000000000  # a 128-byte aligned pretend heap address


class ProductHeap:
    NONE = (1 << 64) - 1

    def __init__(self, L, base, size):
        self.l = L.load()
        self.base = base
        self.h = self.l.heap_model_create(base, size)
        self.size = size

    def alloc(self, n):
        off = self.l.heap_model_alloc(self.h, n)
        return 0 if off == self.NONE else self.base + off

    def free(self, addr):
        if addr:
            assert self.l.heap_model_free(self.h, addr - self.base) == 0

    def used(self):
        return self.l.heap_model_used(self.h)

    def num_bins(self):
        return self.l.heap_model_num_bins(self.h)

    def bin_population(self, b):
        return self.l.heap_model_bin_population(self.h, b)

    def close(self):
        self.l.heap_model_destroy(self.h)


def heaps(orc, L, base, size):
    hs = {"oracle": orc.Heap(base, size, "oracle"), "product": ProductHeap(L, base, size)}
    if orc.ref_allocator_available():
        hs["reference"] = orc.Heap(base, size, "reference")
    return hs


def test_reference_allocator_is_built_here(orc):
    import os
    if os.path.isdir("/root/reference"):
        assert orc.ref_allocator_available(), "run `make -C oracle` to build oracle/_ref"


# ---- known answers: tests/unit_tests/single_heap_gtest.cpp:27-141 -----------
@pytest.mark.parametrize("request_size,expected_used",
                         [(0, 0), (1, 128), (256, 256), (1024, 1024), (4097, 8192)])
def test_single_heap_known_answers(orc, L, request_size, expected_used):
    for name, h in heaps(orc, L, BASE, GiB).items():
        assert h.used() == 0
        p = h.alloc(request_size)
        assert (p == 0) == (request_size == 0), name
        assert h.used() == expected_used, name
        h.free(p)
        assert h.used() == 0, name
        h.close()


# ---- known answers: tests/unit_tests/pow2_bins_gtest.cpp:27-157 -------------
@pytest.mark.parametrize("size,bin_checked,population", [
    (1, 256, 1), (128, 256, 1), (256, 256, 1), (512, 512, 1), (513, 1024, 1),
    (4096, 4096, 1), (131072, 131072, 1), (GiB, GiB, 0)])
def test_pow2_bins_known_answers(orc, L, size, bin_checked, population):
    for name, h in heaps(orc, L, BASE, GiB).items():
        assert h.alloc(size) != 0, name
        assert h.bin_population(bin_checked) == population, name
        h.close()


def test_pow2_bins_free_returns_to_bin(orc, L):
    for name, h in heaps(orc, L, BASE, GiB).items():
        a, b = h.alloc(256), h.alloc(256)
        assert a and b and h.bin_population(256) == 0, name
        h.free(a)
        h.free(b)
        assert h.bin_population(256) == 2, name
        g = h.alloc(GiB)
        assert g == 0, name  # the 1 GiB record was split and is never merged back
        h.close()
    for name, h in heaps(orc, L, BASE, GiB).items():
        g = h.alloc(GiB)
        assert g and h.bin_population(GiB) == 0, name
        h.free(g)
        assert h.bin_population(GiB) == 1, name
        h.close()


# ---- known answers: tests/unit_tests/binner_gtest.cpp:111-136 ---------------
def test_bin_set_of_a_1gib_heap(orc, L):
    for name, h in heaps(orc, L, BASE, GiB).items():
        assert h.num_bins() == 24, name  # 2^7 .. 2^30
        assert h.bin_population(GiB) == 1, name
        for b in range(7, 30):
            assert h.bin_population(1 << b) == 0, name
        h.close()


def test_lowest_address_first_and_lifo_reuse(orc, L):
    for name, h in heaps(orc, L, BASE, GiB).items():
        a, b, c = h.alloc(128), h.alloc(128), h.alloc(300)
        assert (a, b) == (BASE, BASE + 128), name
        assert c == BASE + 512, name  # 256 was split into a,b; next 512 block
        h.free(a)
        h.free(b)
        assert h.alloc(100) == b, name  # last freed, first reused
        assert h.alloc(100) == a, name
        h.close()


def test_exhaustion_returns_null(orc, L):
    for name, h in heaps(orc, L, BASE, 1 << 20).items():
        blocks = [h.alloc(1 << 18) for _ in range(4)]
        assert all(blocks) and len(set(blocks)) == 4, name
        assert h.alloc(1) == 0, name
        assert h.alloc((1 << 20) + 1) == 0, name
        h.close()


# ---- random sequences against the reference's own code ----------------------
@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("base,size", [
    (BASE, 1 << 24), (BASE + 8, 1 << 24), (BASE + 120, (1 << 24) + 12345),
    (BASE, (1 << 22) * 3 + 640), (BASE + 64, 1000)])
def test_random_sequences_agree(orc, L, seed, base, size):
    hs = heaps(orc, L, base, size)
    if "reference" not in hs:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(seed)
    live = []
    names = list(hs)
    for step in range(600):
        if live and rng.random() < 0.45:
            i = int(rng.integers(len(live)))
            addr = live.pop(i)
            for h in hs.values():
                h.free(addr)
        else:
            kind = rng.random()
            if kind < 0.1:
                req = 0
            elif kind < 0.6:
                req = int(rng.integers(1, 5000))
            else:
                req = int(1 << rng.integers(0, 23)) + int(rng.integers(-1, 2))
            got = [h.alloc(max(req, 0)) for h in hs.values()]
            assert len(set(got)) == 1, (step, req, dict(zip(names, got)))
            if got[0]:
                live.append(got[0])
        used = [h.used() for h in hs.values()]
        assert len(set(used)) == 1, (step, dict(zip(names, used)))
    for b in range(7, 25):
        pops = [h.bin_population(1 << b) for h in hs.values()]
        assert len(set(pops)) == 1, (b, dict(zip(names, pops)))
    for h in hs.values():
        h.close()
