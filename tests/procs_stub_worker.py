"""Host logic of the runtime on a machine without a GPU: a child process of
tests/test_host_logic_without_gpu.py, run with tests/hip_stub's stand-in for
the HIP runtime in front of the real one.  Kernels do not run under it (only
the whole-GPU copy kernel is carried out, with bounds checks), so everything
here is about bring-up, bookkeeping, address resolution and host-initiated
copies.  One process (argv[1] == "one") or one PE of a job of processes."""
import ctypes as C
import os
import struct
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import pyoracle as orc  # noqa: E402  (the checker)
from rocshmem_amd import lib as L  # noqa: E402

HEAP = 8 << 20
TWO_MIB = 2 << 20
NOSTORE = 1


class CtxHandle(C.Structure):  # rocshmem_ctx_t (include/rocshmem/rocshmem_common.hpp)
    _fields_ = [("ctx_opaque", C.c_void_p), ("team_opaque", C.c_void_p)]


def get_bytes(l, dev, n, dtype=np.uint8):
    out = np.empty(n // np.dtype(dtype).itemsize, dtype)
    assert l.copy_out(out.ctypes.data, dev, n) == 0
    return out


def put_bytes(l, dev, a):
    a = np.ascontiguousarray(a)
    assert l.copy_in(dev, a.ctypes.data, a.nbytes) == 0


def context_fields(l, options):
    """The device-side context object that rocshmem_ctx_create hands out, field
    by field (detail/state.hpp: struct Context, 64 bytes)."""
    create = l.cdll._ZN8rocshmem19rocshmem_ctx_createElPNS_14rocshmem_ctx_tE
    create.restype, create.argtypes = C.c_int, [C.c_long, C.POINTER(CtxHandle)]
    destroy = l.cdll._ZN8rocshmem20rocshmem_ctx_destroyENS_14rocshmem_ctx_tE
    destroy.restype, destroy.argtypes = None, [CtxHandle]
    h = CtxHandle()
    assert create(options, C.byref(h)) == 0 and h.ctx_opaque
    raw = get_bytes(l, h.ctx_opaque, 64).tobytes()
    names = ("pe_stride", "my_pe", "options", "peer_delta", "heap_base", "ws_stride", "num_pes", "pool_slot",
             "tinfo", "world_sync")
    f = dict(zip(names, struct.unpack("<QiIQQQiiQQ", raw)))
    assert l.ctx_pe(h.ctx_opaque) == f["my_pe"]
    destroy(h)
    return f


def check_contexts(l, P, me, probe):
    """What device code would compute from a context of this PE: the address
    of `probe` on every PE, compared with the host's own resolution."""
    for options in (0, NOSTORE):
        f = context_fields(l, options)
        assert (f["my_pe"], f["num_pes"], f["options"] & NOSTORE) == (me, P, options)
        assert f["pe_stride"] == l.pe_stride()
        table = get_bytes(l, f["peer_delta"], 8 * P, np.int64)
        for p in range(P):
            by_table = probe + int(table[p])
            by_stride = probe + (p - me) * f["pe_stride"]
            assert by_table == l.pe_ptr(probe, p), (me, p, "table")
            if f["pe_stride"]:
                assert by_stride == l.pe_ptr(probe, p), (me, p, "stride")
        # the PE's own work/sync area starts where its slice ends
        slice_bytes = (l.heap_size() + TWO_MIB - 1) // TWO_MIB * TWO_MIB
        if f["pe_stride"] == 0:
            assert f["world_sync"] - f["heap_base"] == slice_bytes
            for p in range(P):  # and a peer's is readable through the same table entry
                get_bytes(l, f["world_sync"] + int(table[p]), 64)
    return True


def ring_copies(l, P, me, seed):
    """Host-called and whole-GPU-kernel copies to the next PE and from the
    previous one, ragged sizes and offsets; every PE checks its own slice."""
    nxt, prv = (me + 1) % P, (me - 1) % P
    n = 70001
    src, dst = l.malloc(n + 64), l.malloc(n + 64)
    assert src and dst
    for case, (off_s, off_d, size) in enumerate([(0, 0, n), (1, 3, 4099), (5, 2, 1), (16, 7, 65536), (3, 3, 0)]):
        for how in ("host_put", "host_get", "bulk_put", "bulk_get"):
            put_bytes(l, src, orc.fill_u8(n + 64, seed + case, me))
            assert l.fill(dst, 0xA5, n + 64) == 0
            assert l.barrier_all() == 0
            if how == "host_put":
                assert l.host_putmem(dst + off_d, src + off_s, size, me, nxt) == 0
            elif how == "host_get":
                assert l.host_getmem(dst + off_d, src + off_s, size, me, prv) == 0
            elif how == "bulk_put":
                assert l.putmem(dst + off_d, src + off_s, size, me, nxt, None) == 0
            else:
                assert l.getmem(dst + off_d, src + off_s, size, me, prv, None) == 0
            assert l.barrier_all() == 0
            want = np.full(n + 64, 0xA5, np.uint8)
            want[off_d:off_d + size] = orc.fill_u8(n + 64, seed + case, prv)[off_s:off_s + size]
            got = get_bytes(l, dst, n + 64)
            assert np.array_equal(got, want), (how, case, me)
    l.free(src)
    l.free(dst)


def one_process():
    l = L.load()
    for P in (8, 3):
        assert l.init(P, HEAP) == 0
        assert l.n_pes() == P and l.pe_stride() >= HEAP
        probe = l.malloc(4096)
        for me in range(P):
            l.set_pe(me)
            mine = l.pe_ptr(probe, me)
            check_contexts(l, P, me, mine)
            for p in range(P):
                assert l.pe_ptr(mine, p) - mine == (p - me) * l.pe_stride()
        l.set_pe(0)
        # copies between every pair of PEs through the whole-GPU kernel's driver
        n = 10007
        a, b = l.malloc(n), l.malloc(n)
        for me in range(P):
            put_bytes(l, l.pe_ptr(a, me), orc.fill_u8(n, 5, me))
        for me in range(P):
            for pe in range(P):
                assert l.putmem(l.pe_ptr(b, me), l.pe_ptr(a, me), n, me, pe, None) == 0
                assert np.array_equal(get_bytes(l, l.pe_ptr(b, pe), n), orc.fill_u8(n, 5, me))
                assert l.getmem(l.pe_ptr(b, me) + 1, l.pe_ptr(a, me) + 2, 333, me, pe, None) == 0
                assert np.array_equal(get_bytes(l, l.pe_ptr(b, me) + 1, 333), orc.fill_u8(n, 5, pe)[2:335])
        assert l.finalize() == 0
    print("one process ok")


def one_pe_of_a_job():
    P = int(os.environ["ROCSHMEM_EMU_PROCS"])
    me = int(os.environ["ROCSHMEM_EMU_RANK"])
    l = L.load()
    if sys.argv[1] == "unequal-heaps":
        l.init(0, (4 << 20) * (me + 1))
        print("init returned", me)
        return
    if sys.argv[1] == "one-dies":
        assert l.init(0, HEAP) == 0
        if me == 1:
            os._exit(3)          # without finalize, without a word to the others
        l.barrier_all()          # never completes: the wait runs out and ends this process too
        print("barrier returned", me)
        return
    if sys.argv[1] == "global-exit":
        assert l.init(0, HEAP) == 0
        if me == P - 1:
            l.cdll._ZN8rocshmem20rocshmem_global_exitEi(7)
        l.barrier_all()          # the others leave here, with the status asked for
        print("barrier returned", me)
        return
    for bring_up in range(2):  # the second rocshmem_init finds the block and the mappings of the first
        assert l.init(0, HEAP) == 0
        assert (l.n_pes(), l.my_pe(), l.pe_stride()) == (P, me, 0)
        probe = l.malloc(4096)
        assert l.pe_ptr(probe, me) == probe
        assert len({l.pe_ptr(probe, p) for p in range(P)}) == P
        check_contexts(l, P, me, probe)
        # every PE sees every PE's bytes at the address the table gives
        put_bytes(l, probe, orc.fill_u8(4096, 40 + bring_up, me))
        assert l.barrier_all() == 0
        for p in range(P):
            assert np.array_equal(get_bytes(l, l.pe_ptr(probe, p), 4096), orc.fill_u8(4096, 40 + bring_up, p))
        assert l.barrier_all() == 0
        ring_copies(l, P, me, 100 * bring_up)

        # block moves between the processes (they pull with the copy kernel)
        nb = 5003
        s, d = l.malloc(P * nb), l.malloc(P * nb)
        srcs = [orc.fill_u8(P * nb, 77, p) for p in range(P)]
        put_bytes(l, s, srcs[me])
        world = l.team_world()
        assert l.barrier_all() == 0
        assert l.alltoallmem(world, d, s, nb, None) == 0
        assert np.array_equal(get_bytes(l, d, P * nb), orc.alltoall(srcs, nb)[me])
        assert l.barrier_all() == 0
        assert l.fcollectmem(world, d, s, nb, None) == 0
        assert np.array_equal(get_bytes(l, d, P * nb), orc.fcollect([x[:nb] for x in srcs], nb)[me])
        assert l.barrier_all() == 0
        assert l.fill(d, 0x11, P * nb) == 0
        assert l.barrier_all() == 0
        assert l.broadcastmem(world, d, s, nb, P - 1, None) == 0
        want = [np.full(nb, 0x11, np.uint8) for _ in range(P)]
        orc.broadcast([x[:nb] for x in srcs], want, nb, P - 1)
        assert np.array_equal(get_bytes(l, d, nb), want[me])
        assert l.barrier_all() == 0

        # a team of the even PEs: made by its members, met by the whole parent team
        team = C.c_void_p()
        assert l.team_split_strided(world, 0, 2, (P + 1) // 2, C.byref(team)) == 0
        if me % 2 == 0:
            assert team.value and (l.team_n_pes(team), l.team_my_pe(team)) == ((P + 1) // 2, me // 2)
            assert l.broadcastmem(team, d, s, nb, 0, None) == 0
            if me:
                assert np.array_equal(get_bytes(l, d, nb), srcs[0][:nb])
        else:
            assert not team.value
        assert l.barrier_all() == 0

        # what belongs to the one-process harness is refused before anything is launched
        assert l.wg_reduce(L.INT, L.SUM, world, d, s, 4, 64, None) == -1
        assert l.rma(L.PUT, L.WG, d, s, 16, 0, (me + 1) % P, me, 1, 64, 1, None) == -1
        assert l.fill_every_pe(d, 0, 16, None) == -1
        for p in (s, d, probe):
            l.free(p)
        assert l.finalize() == 0
    print("ok", me)


def refusals():
    """Calls that must be refused on the host: each returns -1 and the stand-in
    sees no launch (what rocshmem_amd.h promises: pointers and sizes are
    checked against the heap before anything is enqueued)."""
    l = L.load()
    P, heap = 4, HEAP
    assert l.init(P, heap) == 0
    stub = C.CDLL("libamdhip64.so.7")
    stub.hip_stub_counts.argtypes = [C.POINTER(C.c_ulonglong), C.POINTER(C.c_ulonglong)]

    def launches():
        n = C.c_ulonglong()
        stub.hip_stub_counts(C.byref(n), None)
        return n.value

    a, b = l.malloc(4096), l.malloc(4096)
    last = l.malloc(heap // 4)        # some block; its PE-0 slice ends at base + heap
    base = a - (a - l.pe_ptr(a, 0))   # a is PE 0's
    end = base + l.heap_size()        # first byte past PE 0's usable slice
    local = l.dev_alloc(4096)
    world = l.team_world()
    outside = np.zeros(64, np.uint8).ctypes.data  # host memory, not in the heap
    calls = [
        # a PE that does not exist, either side
        lambda: l.rma(L.PUT, L.WG, a, b, 64, 0, 0, P, 1, 64, 1, None),
        lambda: l.rma(L.PUT, L.WG, a, b, 64, 0, -1, 1, 1, 64, 1, None),
        # launch shapes
        lambda: l.rma(L.PUT, L.WG, a, b, 64, 0, 0, 1, 0, 64, 1, None),
        lambda: l.rma(L.PUT, L.WG, a, b, 64, 0, 0, 1, 1, 2048, 1, None),
        lambda: l.rma(9, L.WG, a, b, 64, 0, 0, 1, 1, 64, 1, None),
        lambda: l.rma(L.PUT, 7, a, b, 64, 0, 0, 1, 1, 64, 1, None),
        # the symmetric side straddles the end of the slice, or is not symmetric at all
        lambda: l.rma(L.PUT, L.WG, end - 8, b, 16, 0, 0, 1, 1, 64, 1, None),
        lambda: l.rma(L.GET, L.WG, local, end - 8, 16, 0, 0, 1, 1, 64, 1, None),
        lambda: l.rma(L.PUT, L.WG, local, b, 16, 0, 0, 1, 1, 64, 1, None),
        lambda: l.rma(L.PUT, L.WG, l.pe_ptr(a, 1), b, 16, 0, 0, 1, 1, 64, 1, None),  # another PE's address
        lambda: l.putmem(end - 8, b, 16, 0, 1, None),
        lambda: l.getmem(local, end - 8, 16, 0, 1, None),
        lambda: l.putmem(a, b, 16, 0, P, None),
        lambda: l.host_putmem(end - 8, outside, 16, 0, 1),
        lambda: l.host_getmem(outside, end - 8, 16, 0, 1),
        lambda: l.host_putmem(a, outside, 16, P, 1),
        lambda: l.rma_staged(L.WG, a, local, local, 1 << 20, 0, 1, 64, None),
        lambda: l.rma_staged(L.WG, end - 8, local, local, 64, 0, 1, 64, None),
        lambda: l.put_signal(L.WG, end - 8, local, 64, b, 1, L.SIGNAL_SET, 0, 1, 1, 64, 1, None),
        lambda: l.put_signal(L.WG, a, local, 64, end - 4, 1, L.SIGNAL_SET, 0, 1, 1, 64, 1, None),
        lambda: l.amo(L.AMO_FETCH_ADD, L.LONG, end - 8, 4, local, None, None, None, 4, 0, 1, 64, None),
        lambda: l.amo(L.AMO_FETCH_ADD, L.LONG, a, 0, local, None, None, None, 4, 0, 1, 64, None),
        lambda: l.amo(L.AMO_FETCH_ADD, L.LONG, a, 4, None, None, None, None, 4, 0, 1, 64, None),
        # collectives: sets that leave the world, buffers that leave the slice, teams that are none
        lambda: l.to_all(L.INT, L.SUM, a, b, 4, 0, 0, P + 1, None),
        lambda: l.to_all(L.INT, L.SUM, a, b, 4, 2, 1, 2, None),
        lambda: l.to_all(L.INT, L.SUM, a, b, -1, 0, 0, P, None),
        lambda: l.to_all(L.INT, L.SUM, end - 8, b, 4, 0, 0, P, None),
        lambda: l.to_all(99, L.SUM, a, b, 4, 0, 0, P, None),
        lambda: l.reduce(L.INT, L.SUM, None, a, b, 4, None),
        lambda: l.alltoallmem(world, a, b, heap // 2, None),     # P blocks of that size leave the slice
        lambda: l.fcollectmem(world, a, b, heap // 2, None),
        lambda: l.broadcastmem(world, a, b, 64, P, None),
        lambda: l.broadcastmem(world, end - 8, b, 64, 0, None),
        lambda: l.broadcast_active_set(a, b, 64, 5, 0, 0, P, None),
        lambda: l.wg_reduce(L.INT, L.SUM, world, a, b, 4, 0, None),
        lambda: l.wg_reduce(L.INT, L.SUM, None, a, b, 4, 64, None),
        lambda: l.wg_alltoall(4, world, a, b, heap // 8, 64, None),
        lambda: l.wg_sync(L.BARRIER_ALL, world, end - 4, 1, 64, None),
        lambda: l.pingpong(a, b, 64, 1, 1, 0, 0, 64, None, None, None),
        lambda: l.pingpong(a, b, 64, 1, 500, 0, 1, 64, None, None, None),
    ]
    for i, call in enumerate(calls):
        before = launches()
        assert call() == -1, i
        assert launches() == before, (i, "launched something")
    # and a call that is accepted does launch
    before = launches()
    assert l.rma(L.PUT, L.WG, a, b, 64, 0, 0, 1, 1, 64, 1, None) == 0
    assert launches() == before + 1
    assert last
    l.finalize()
    print("refusals ok", len(calls))


def no_alloc():
    """rocshmem_amd_wg_reduce_teams_static must not allocate or free anything
    (it is the entry point for callers that cannot); its sibling does.  The
    stand-in counts every allocating and freeing call of the HIP runtime."""
    l = L.load()
    P = 8
    assert l.init(P, HEAP) == 0
    stub = C.CDLL("libamdhip64.so.7")
    stub.hip_stub_alloc_calls.restype = C.c_ulonglong
    n_teams = 5
    teams = (C.c_void_p * n_teams)()
    for t in range(n_teams):
        h = C.c_void_p()
        assert l.team_split_strided(l.team_world(), 0, 1, P, C.byref(h)) == 0 and h.value
        teams[t] = h.value
    n = 4099
    src, dst = l.malloc(n * 4), l.malloc(n * 4)
    l.wg_reduce_teams_static(L.INT, L.SUM, teams, n_teams, dst, src, n, 0, 64, 1, None)  # first call: set-up
    before = stub.hip_stub_alloc_calls()
    for _ in range(3):
        assert l.wg_reduce_teams_static(L.INT, L.SUM, teams, n_teams, dst, src, n, 0, 64, 1, None) == 0
        assert l.wg_reduce_teams_static(L.INT, L.SUM, teams, 300, dst, src, n, 0, 64, 1, None) == -1
    assert stub.hip_stub_alloc_calls() == before, "the static entry point allocated or freed"
    assert l.wg_reduce_teams(L.INT, L.SUM, teams, n_teams, dst, src, n, 0, 64, 1, None) == 0
    assert stub.hip_stub_alloc_calls() > before, "the counter does not see the allocating entry point"
    l.finalize()
    print("no alloc ok")


if __name__ == "__main__":
    if sys.argv[1] == "one":
        one_process()
    elif sys.argv[1] == "no-alloc":
        no_alloc()
    elif sys.argv[1] == "refusals":
        refusals()
    elif sys.argv[1] == "memset-outside":
        l = L.load()
        assert l.init(2, HEAP) == 0
        a = l.malloc(64)
        l.fill(a + (1 << 40), 0, 64)  # the stand-in ends the process: on a GPU this is a fault
        print("survived")
    else:
        one_pe_of_a_job()
