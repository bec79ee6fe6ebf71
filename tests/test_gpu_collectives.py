"""A2A, FC, BC, SY: alltoall / fcollect / broadcast through the device API (one
work-group per PE) and the host-called whole-GPU forms; barriers.  Byte-exact
against the oracle's index maps.  Through the C entry points."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P, HEAP = 8, 1 << 30


def fill_sources(rt, l, orc, src, pes, nbytes, seed):
    srcs = [orc.fill_u8(nbytes, seed, 100 + p) for p in pes]
    for k, p in enumerate(pes):
        rt.put_bytes(l.pe_ptr(src, p), srcs[k])
    return srcs


def run_move(rt, l, L, orc, kind, mode, elem, nelems, pes, team, root=0, wg=256, seed=0):
    n = elem * nelems
    T = len(pes)
    src_bytes = n * T if kind == "alltoall" else n
    dst_bytes = n if kind == "broadcast" else n * T
    src = l.malloc(max(src_bytes, 1) + 64)
    dst = l.malloc(max(dst_bytes, 1) + 64)
    srcs = fill_sources(rt, l, orc, src, pes, src_bytes, seed)
    for p in range(P):
        l.fill(l.pe_ptr(dst, p), 0xC3, dst_bytes + 64)
    me = l.my_pe()
    d, s = l.pe_ptr(dst, me), l.pe_ptr(src, me)
    if mode == "wg":
        if kind == "alltoall":
            rc = l.wg_alltoall(elem, team, d, s, nelems, wg, None)
        elif kind == "fcollect":
            rc = l.wg_fcollect(elem, team, d, s, nelems, wg, None)
        else:
            rc = l.wg_broadcast(elem, team, d, s, nelems, root, wg, None)
    else:
        if kind == "alltoall":
            rc = l.alltoallmem(team, d, s, n, None)
        elif kind == "fcollect":
            rc = l.fcollectmem(team, d, s, n, None)
        else:
            rc = l.broadcastmem(team, d, s, n, root, None)
    assert rc == 0, (kind, mode, elem, nelems)
    l.stream_sync(None)
    if kind == "alltoall":
        want = orc.alltoall(srcs, n)
    elif kind == "fcollect":
        want = orc.fcollect(srcs, n)
    else:
        want = [np.full(n, 0xC3, np.uint8) for _ in pes]
        orc.broadcast(srcs, want, n, root)
    for p in range(P):
        got = rt.get_bytes(l.pe_ptr(dst, p), dst_bytes + 64)
        if p in pes:
            k = pes.index(p)
            assert np.array_equal(got[:dst_bytes], want[k]), (kind, mode, elem, nelems, p)
            assert (got[dst_bytes:] == 0xC3).all()
        else:
            assert (got == 0xC3).all(), (kind, mode, p, "non-member touched")
    l.free(src)
    l.free(dst)


@pytest.mark.parametrize("mode", ["wg", "grid"])
@pytest.mark.parametrize("kind", ["alltoall", "fcollect", "broadcast"])
def test_world_team_sizes_and_types(rt, L, orc, kind, mode):
    l = rt.up(P, HEAP)
    pes = list(range(P))
    for elem in ((1, 2, 4, 8) if mode == "wg" else (1,)):
        for nelems in (1, 3, 17, 256, 1001, 65537):
            run_move(rt, l, L, orc, kind, mode, elem, nelems, pes, l.team_world(), root=nelems % P,
                     seed=nelems)


@pytest.mark.parametrize("mode", ["wg", "grid"])
def test_sub_teams(rt, L, orc, mode):
    l = rt.up(P, HEAP)
    for start, stride, size in [(0, 2, 4), (1, 2, 3), (3, 1, 4), (0, 7, 2)]:
        pes = [start + stride * k for k in range(size)]
        l.set_pe(pes[-1])
        team = ctypes.c_void_p()
        assert l.team_split_strided(l.team_world(), start, stride, size, ctypes.byref(team)) == 0
        for kind in ("alltoall", "fcollect", "broadcast"):
            run_move(rt, l, L, orc, kind, mode, 1 if mode == "grid" else 4, 999, pes, team,
                     root=size - 1, seed=start)
        l.team_destroy(team)
    l.set_pe(0)


def test_reference_alltoall_and_broadcast_vectors(rt, L, orc):
    """examples/rocshmem_alltoall_test.cc:49-75 (src[pe*n+i] = me+pe -> dst the
    same) and tests/functional_tests/team_broadcast_tester.cpp:176-243 (non-roots
    receive, the root's dest keeps its old contents)."""
    l = rt.up(P, HEAP)
    n = 256
    src, dst = l.malloc(P * n * 4), l.malloc(P * n * 4)
    for me in range(P):
        rt.put_bytes(l.pe_ptr(src, me), np.repeat(np.arange(P, dtype=np.int32) + me, n))
        l.fill(l.pe_ptr(dst, me), 0xFF, P * n * 4)
    assert l.wg_alltoall(4, l.team_world(), dst, src, n, 256, None) == 0
    l.stream_sync(None)
    for me in range(P):
        got = rt.get_bytes(l.pe_ptr(dst, me), P * n * 4, np.int32)
        assert np.array_equal(got, np.repeat(np.arange(P, dtype=np.int32) + me, n))
    for me in range(P):
        rt.put_bytes(l.pe_ptr(src, me), np.full(n, P + me, np.int32))
        rt.put_bytes(l.pe_ptr(dst, me), np.full(n, me, np.int32))
    assert l.wg_broadcast(4, l.team_world(), dst, src, n, 3, 128, None) == 0
    l.stream_sync(None)
    for me in range(P):
        got = rt.get_bytes(l.pe_ptr(dst, me), n * 4, np.int32)
        assert (got == (me if me == 3 else P + 3)).all()
    l.free(src)
    l.free(dst)


def test_moe_dispatch_shape_alltoall(rt, L, orc):
    """P=8, 512 tokens x 7168 bf16 per PE pair (7,340,032 bytes per block)."""
    l = rt.up(P, HEAP)
    blk = 512 * 7168 * 2
    src, dst = l.malloc(P * blk), l.malloc(P * blk)
    assert src and dst
    tile = 1 << 20
    srcs = []
    for p in range(P):  # a seeded 1 MiB tile repeated, rotated per block so blocks differ
        t = orc.fill_u8(tile, 4, p)
        full = np.concatenate([np.roll(np.resize(t, blk), j) for j in range(P)])
        srcs.append(full)
        rt.put_bytes(l.pe_ptr(src, p), full)
        l.fill(l.pe_ptr(dst, p), 0, P * blk)
    assert l.alltoallmem(l.team_world(), dst, src, blk, None) == 0
    l.stream_sync(None)
    want = orc.alltoall(srcs, blk, nthreads=4)
    for p in range(P):
        assert np.array_equal(rt.get_bytes(l.pe_ptr(dst, p), P * blk), want[p]), p
    l.free(src)
    l.free(dst)


@pytest.mark.parametrize("fn", ["BARRIER_ALL", "SYNC_ALL", "TEAM_SYNC"])
def test_barriers_order_puts(rt, L, fn):
    """A value put before the barrier is seen after it, for many rounds."""
    l = rt.up(P, HEAP)
    scratch = l.malloc(64)
    for p in range(P):
        l.fill(l.pe_ptr(scratch, p), 0, 64)
    team = l.team_world()
    sub = None
    if fn == "TEAM_SYNC":
        sub = ctypes.c_void_p()
        l.set_pe(1)
        assert l.team_split_strided(l.team_world(), 1, 2, 3, ctypes.byref(sub)) == 0
        team = sub
    for wg in (1, 64, 256):
        errors = l.wg_sync(getattr(L, fn), team, l.pe_ptr(scratch, l.my_pe()), 200, wg, None)
        assert errors == 0, (fn, wg)
        for p in range(P):
            l.fill(l.pe_ptr(scratch, p), 0, 64)
    if sub is not None:
        l.team_destroy(sub)
    l.set_pe(0)
    l.free(l.pe_ptr(scratch, 0))


def test_zero_length_collectives_do_nothing(rt, L):
    l = rt.up(P, HEAP)
    buf = l.malloc(4096)
    l.fill(buf, 0x77, 4096)
    assert l.wg_alltoall(4, l.team_world(), buf, buf, 0, 64, None) == 0
    assert l.wg_broadcast(4, l.team_world(), buf, buf, 0, 0, 64, None) == 0
    assert l.wg_fcollect(4, l.team_world(), buf, buf, 0, 64, None) == 0
    assert l.alltoallmem(l.team_world(), buf, buf, 0, None) == 0
    l.stream_sync(None)
    assert (rt.get_bytes(buf, 4096) == 0x77).all()
    assert l.wg_broadcast(4, l.team_world(), buf, buf, 8, P, 64, None) == -1  # bad root
    assert l.wg_alltoall(3, l.team_world(), buf, buf, 8, 64, None) == -1      # bad element size
    l.free(buf)


def test_the_largest_world(rt, L, orc):
    """256 PEs, the most one heap is divided into: whole-GPU and per-work-group
    block moves (65 536 sender-receiver pairs), an all-reduce over all of them
    and barrier rounds with one work-group per PE."""
    big = 256
    l = rt.up(big, 2 << 20)
    n = 48                                   # bytes per block
    src, dst = l.malloc(big * n), l.malloc(big * n)
    assert src and dst
    srcs = [orc.fill_u8(big * n, 9, p) for p in range(big)]
    for p in range(big):
        rt.put_bytes(l.pe_ptr(src, p), srcs[p])
    for mode in ("grid", "wg"):
        for kind in ("alltoall", "fcollect", "broadcast"):
            assert l.fill_every_pe(dst, 0xC3, big * n, None) == 0
            if kind == "alltoall":
                rc = (l.alltoallmem(l.team_world(), dst, src, n, None) if mode == "grid" else
                      l.wg_alltoall(1, l.team_world(), dst, src, n, 64, None))
                want = orc.alltoall(srcs, n)
            elif kind == "fcollect":
                rc = (l.fcollectmem(l.team_world(), dst, src, n, None) if mode == "grid" else
                      l.wg_fcollect(1, l.team_world(), dst, src, n, 64, None))
                want = orc.fcollect([s[:n] for s in srcs], n)
            else:
                rc = (l.broadcastmem(l.team_world(), dst, src, big * n, 200, None) if mode == "grid" else
                      l.wg_broadcast(1, l.team_world(), dst, src, big * n, 200, 64, None))
                want = [np.full(big * n, 0xC3, np.uint8) for _ in range(big)]
                orc.broadcast(srcs, want, big * n, 200)
            assert rc == 0, (mode, kind)
            l.stream_sync(None)
            for p in range(big):
                got = rt.get_bytes(l.pe_ptr(dst, p), big * n)
                assert np.array_equal(got, want[p]), (mode, kind, p)
    ints = [s.view(np.int32) for s in srcs]
    total = orc.to_all(L.INT, L.SUM, ints)
    assert l.to_all(L.INT, L.SUM, dst, src, big * n // 4, 0, 0, big, None) == 0
    l.stream_sync(None)
    for p in (0, 1, 100, 255):
        assert np.array_equal(rt.get_bytes(l.pe_ptr(dst, p), big * n, np.int32), total), p
    word = l.malloc(8)
    assert l.fill_every_pe(word, 0, 8, None) == 0
    for fn in (L.BARRIER_ALL, L.SYNC_ALL, L.TEAM_SYNC):
        assert l.wg_sync(fn, l.team_world(), word, 5, 64, None) == 0, fn
    for b in (src, dst, word):
        l.free(b)
    rt.up(P, HEAP)
