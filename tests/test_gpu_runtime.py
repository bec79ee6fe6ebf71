"""H1-H3, X2: bring-up, symmetric allocation on the device heap, PE
addressing and teams through the C entry points."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.gpu


def test_malloc_matches_the_oracle_allocator(rt, L, orc):
    rt.down()  # a fresh heap: freed blocks are never merged, so history matters
    l = rt.up(4, 1 << 26)
    base = l.malloc(1)
    l.free(base)
    model = orc.Heap(base, 1 << 26)
    assert model.alloc(1) == base  # replay what the device heap has seen so far
    model.free(base)
    rng = np.random.default_rng(0)
    live = []
    for _ in range(300):
        if live and rng.random() < 0.4:
            p = live.pop(int(rng.integers(len(live))))
            l.free(p)
            model.free(p)
        else:
            req = int(rng.integers(0, 1 << int(rng.integers(1, 25))))
            got = l.malloc(req) or 0
            assert got == model.alloc(req), req
            if got:
                live.append(got)
        assert l.heap_used() == model.used()
        assert l.heap_avail() == (1 << 26) - model.used()
    assert l.heap_size() == 1 << 26
    for p in live:
        l.free(p)
    assert l.heap_used() == 0
    assert l.malloc(0) is None and l.malloc((1 << 26) + 1) is None
    l.free(None)  # ignored


def test_same_offset_on_every_pe_and_slices_do_not_overlap(rt, L):
    l = rt.up(8, 1 << 24)
    stride = l.pe_stride()
    assert stride >= 1 << 24 and stride % (2 << 20) == 0
    a = l.malloc(1000)
    ptrs = [l.pe_ptr(a, p) for p in range(8)]
    assert ptrs == [a + p * stride for p in range(8)]
    for p in range(8):
        l.set_pe(p)
        b = l.malloc(64)
        assert b == l.pe_ptr(b, p) and (b - a) % stride == (l.pe_ptr(b, 0) - a)
        assert l.my_pe() == p
        l.free(b)
    l.set_pe(0)
    assert l.pe_ptr(a, 8) is None and l.pe_ptr(a + 8 * stride, 0) is None
    # a write through one PE's address is seen only there
    for p in range(8):
        l.fill(ptrs[p], p + 1, 1000)
    for p in range(8):
        buf = np.empty(1000, np.uint8)
        l.copy_out(buf.ctypes.data, ptrs[p], 1000)
        assert (buf == p + 1).all()
    l.free(a)


def test_fill_every_pe_touches_exactly_the_object(rt, L):
    l = rt.up(4, 1 << 26)
    for n in (1, 64, 1000, 300001):
        obj = l.malloc(n + 128)
        for pe in range(4):
            l.fill(l.pe_ptr(obj, pe), 0x11, n + 128)
        assert l.fill_every_pe(obj + 64, 0xC3, n, None) == 0
        l.stream_sync(None)
        for pe in range(4):
            got = rt.get_bytes(l.pe_ptr(obj, pe), n + 128)
            assert (got[:64] == 0x11).all() and (got[64 + n:] == 0x11).all(), (n, pe)
            assert (got[64:64 + n] == 0xC3).all(), (n, pe)
        l.free(obj)
    assert l.fill_every_pe(None, 0, 8, None) == -1
    assert l.fill_every_pe(l.pe_ptr(l.malloc(128), 1), 0, 8, None) == -1  # not PE 0's address


def test_teams(rt, L, orc):
    """src/rocshmem.cpp:193-319 and tests/sos_tests/shmem_team_translate.cpp."""
    l = rt.up(8, 1 << 24)
    world = l.team_world()
    assert l.team_n_pes(world) == 8 and l.team_my_pe(world) == 0
    assert l.team_n_pes(None) == -1 and l.team_my_pe(None) == -1
    t2, t3, bad = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    assert l.team_split_strided(world, 0, 2, 4, ctypes.byref(t2)) == 0
    assert l.team_split_strided(world, 0, 3, 3, ctypes.byref(t3)) == 0
    for args in [(-1, 1, 2), (8, 1, 1), (0, 0, 2), (0, 1, 0), (0, 1, 9), (2, 3, 3)]:
        assert l.team_split_strided(world, *args, ctypes.byref(bad)) == -1 and not bad.value
    for me in range(8):
        l.set_pe(me)
        a, b = l.team_on(t2, me), l.team_on(t3, me)
        assert (a is not None) == (me % 2 == 0) and (b is not None) == (me % 3 == 0)
        if a:
            assert l.team_my_pe(a) == me // 2 and l.team_n_pes(a) == 4
        if a and b:
            assert l.team_translate_pe(a, l.team_my_pe(a), b) == me // 3
        elif a:
            assert l.team_translate_pe(a, l.team_my_pe(a), t3) == -1
    l.set_pe(0)
    assert l.team_translate_pe(None, 0, t2) == -1
    # a split of a strided parent composes with it
    t22 = ctypes.c_void_p()
    assert l.team_split_strided(t2, 1, 2, 2, ctypes.byref(t22)) == 0   # world PEs 2, 6
    assert not t22.value  # PE 0 is not a member
    l.set_pe(6)
    assert l.team_split_strided(l.team_on(t2, 6), 1, 2, 2, ctypes.byref(t22)) == 0
    assert l.team_n_pes(t22) == 2 and l.team_my_pe(t22) == 1
    assert l.team_translate_pe(t22, 0, l.team_world()) == 2
    l.set_pe(0)
    for t in (t2, t3):
        l.team_destroy(t)


def test_team_pool_exhaustion(rt, L):
    """ROCSHMEM_MAX_NUM_TEAMS - 1 user teams (39 by default), then -1
    (tests/functional_tests/team_ctx_infra_tester.cpp:31-32, src/rocshmem.cpp:229-234)."""
    l = rt.up(2, 1 << 22)
    teams = []
    for _ in range(39):
        t = ctypes.c_void_p()
        assert l.team_split_strided(l.team_world(), 0, 1, 2, ctypes.byref(t)) == 0 and t.value
        teams.append(t)
    assert len({t.value for t in teams}) == 39
    t = ctypes.c_void_p()
    assert l.team_split_strided(l.team_world(), 0, 1, 2, ctypes.byref(t)) == -1 and not t.value
    l.team_destroy(teams.pop())
    assert l.team_split_strided(l.team_world(), 0, 1, 2, ctypes.byref(t)) == 0 and t.value
    for x in teams + [t]:
        l.team_destroy(x)


def test_default_layout_allocates_what_the_slices_need(rt, L, monkeypatch):
    """By default the slices are packed: stride = heap size rounded up to
    2 MiB, one allocation of P strides.  A default rocshmem_init with 8 PEs and
    the default 1 GiB per PE leaves the rest of the device memory to the user:
    free memory afterwards is within 1 GiB of what was free before minus the
    8 GiB of slices.  (In a process of its own: the heap is uncached memory,
    which a process keeps and reuses once it has it.)"""
    rt.down()
    code = (
        "import ctypes, sys\n"
        "sys.path.insert(0, %r)\n"
        "from rocshmem_amd import lib as L\n"
        "l = L.load()\n"
        "f0, f1, tot = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()\n"
        "assert l.dev_mem_info(ctypes.byref(f0), ctypes.byref(tot)) == 0\n"
        "assert l.init(8, 0) == 0\n"
        "assert l.heap_size() == 1 << 30 and l.pe_stride() == 1 << 30\n"
        "assert l.heap_alloc_bytes() == 8 << 30\n"
        "assert l.dev_mem_info(ctypes.byref(f1), ctypes.byref(tot)) == 0\n"
        "taken = f0.value - f1.value\n"
        "assert (8 << 30) - (64 << 20) <= taken <= (9 << 30), taken\n"
        "big = l.dev_alloc(f1.value // 2)\n"
        "assert big\n"
        "l.dev_free(big)\n"
        "l.finalize()\n"
        "for npes, heap in ((3, (1 << 24) + 5), (5, 3 << 20)):\n"
        "    assert l.init(npes, heap) == 0\n"
        "    want = (heap + (2 << 20) - 1) // (2 << 20) * (2 << 20)\n"
        "    assert l.pe_stride() == want\n"
        "    l.finalize()\n"
        "print('ok')\n" % ROOT)
    env = {k: v for k, v in os.environ.items()
           if k not in ("ROCSHMEM_EMU_PE_STRIDE", "ROCSHMEM_EMU_SPREAD", "ROCSHMEM_HEAP_SIZE")}
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "ok" in r.stdout, (r.stdout[-400:], r.stderr[-800:])


def test_spread_layout_is_opt_in(rt, L, monkeypatch):
    """ROCSHMEM_EMU_SPREAD=1 spreads the slices over half of the device
    memory on a 4 GiB grid (288 GB: 16 GiB for 8 PEs, 32 for 4, 44 for 3, 8
    for 16; two PEs keep 16 GiB), never closer than the heap size;
    ROCSHMEM_EMU_PE_STRIDE sets the stride directly.  Results do not depend on
    the layout: an all-reduce in the spread layout matches the packed one."""
    monkeypatch.delenv("ROCSHMEM_EMU_PE_STRIDE", raising=False)
    monkeypatch.setenv("ROCSHMEM_EMU_SPREAD", "1")
    rt.down()
    l = L.load()
    for npes, gib in ((2, 16), (3, 44), (4, 32), (5, 28), (8, 16), (16, 8)):
        assert l.init(npes, 1 << 24) == 0
        assert l.pe_stride() == gib << 30, npes
        a = l.malloc(64)
        assert l.pe_ptr(a, npes - 1) - a == (npes - 1) * (gib << 30)
        l.finalize()
    monkeypatch.setenv("ROCSHMEM_EMU_PE_STRIDE", str(6 << 20))
    assert l.init(4, 1 << 22) == 0
    assert l.pe_stride() == 6 << 20
    l.finalize()
    monkeypatch.delenv("ROCSHMEM_EMU_PE_STRIDE")
    results = []
    for spread in ("1", "0"):
        monkeypatch.setenv("ROCSHMEM_EMU_SPREAD", spread)
        assert l.init(8, 1 << 24) == 0
        n = 100003
        src, dst = l.malloc(n * 4), l.malloc(n * 4)
        for p in range(8):
            host = np.random.default_rng(p).standard_normal(n).astype(np.float32)
            l.copy_in(l.pe_ptr(src, p), host.ctypes.data, n * 4)
        assert l.wg_reduce(L.FLOAT, L.SUM, l.team_world(), dst, src, n, 256, None) == 0
        out = np.empty(n, np.float32)
        l.copy_out(out.ctypes.data, l.pe_ptr(dst, 5), n * 4)
        results.append(out)
        l.finalize()
    assert np.array_equal(results[0].view(np.uint32), results[1].view(np.uint32))


def test_reinit_and_environment_defaults(rt, L, monkeypatch):
    rt.down()
    l = L.load()
    monkeypatch.setenv("ROCSHMEM_EMU_NPES", "3")
    monkeypatch.setenv("ROCSHMEM_HEAP_SIZE", str(1 << 22))
    assert l.n_pes() == 3           # before init
    assert l.init(0, 0) == 0
    assert l.n_pes() == 3 and l.heap_size() == 1 << 22
    l.finalize()
    monkeypatch.delenv("ROCSHMEM_EMU_NPES")
    monkeypatch.delenv("ROCSHMEM_HEAP_SIZE")
