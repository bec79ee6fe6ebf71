"""One PE of the process-per-PE parity test: started P times by
tests/test_gpu_zy_processes.py through rocshmem_amd.launch.  Every process
calls the C entry points for its own PE and checks what lands in its own
slice against the CPU oracle (every process can compute every PE's seeded
input).  Prints "ok <pe>" at the end."""
import ctypes
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
from oracle import pyoracle as orc  # noqa: E402  (the checker)
from rocshmem_amd import lib as L  # noqa: E402
from test_gpu_reduce import TYPES, make_inputs  # noqa: E402

HEAP = 256 << 20


def put_bytes(l, dev, a):
    a = np.ascontiguousarray(a)
    assert l.copy_in(dev, a.ctypes.data, a.nbytes) == 0


def get_bytes(l, dev, nbytes, dtype=np.uint8):
    out = np.empty(nbytes // np.dtype(dtype).itemsize, dtype)
    assert l.copy_out(out.ctypes.data, dev, nbytes) == 0
    return out


def main():
    P = int(os.environ["ROCSHMEM_EMU_PROCS"])
    me = int(os.environ["ROCSHMEM_EMU_RANK"])
    l = L.load()
    if sys.argv[1:] == ["unequal-heaps"]:
        # every PE asks for another heap size: rocshmem_init ends the job with a message
        l.init(0, (64 << 20) * (me + 1))
        print("init returned", me)
        return
    assert l.init(0, HEAP) == 0
    assert (l.n_pes(), l.my_pe()) == (P, me)
    nxt, prv = (me + 1) % P, (me - 1) % P

    # ---- puts and gets, host-called and from kernels, ragged sizes and offsets
    n = 100003
    src, dst = l.malloc(n + 64), l.malloc(n + 64)
    assert src and dst
    for case, (off_s, off_d, size) in enumerate([(0, 0, n), (1, 3, 4099), (5, 2, 1), (16, 7, 65536), (3, 3, 0)]):
        for how in ("host_put", "host_get", "bulk_put", "bulk_get", "put_wg", "put_wave", "put_thread",
                    "get_wg", "put_nbi_wg"):
            mine = orc.fill_u8(n + 64, 100 + case, me)
            put_bytes(l, src, mine)
            assert l.fill(dst, 0xA5, n + 64) == 0
            assert l.barrier_all() == 0
            if how == "host_put":
                assert l.host_putmem(dst + off_d, src + off_s, size, me, nxt) == 0
            elif how == "host_get":
                assert l.host_getmem(dst + off_d, src + off_s, size, me, prv) == 0
            elif how == "bulk_put":  # the whole-GPU kernels behind the host's rocshmem_putmem / getmem
                assert l.putmem(dst + off_d, src + off_s, size, me, nxt, None) == 0
            elif how == "bulk_get":
                assert l.getmem(dst + off_d, src + off_s, size, me, prv, None) == 0
            elif how.startswith("put"):
                gran = {"wg": L.WG, "wave": L.WAVE, "thread": L.THREAD}[how.split("_")[-1]]
                op = L.PUT_NBI if "nbi" in how else L.PUT
                assert l.rma(op, gran, dst + off_d, src + off_s, size, 0, me, nxt, 4, 128, 1, None) == 0
            else:
                assert l.rma(L.GET, L.WG, dst + off_d, src + off_s, size, 0, me, prv, 4, 128, 1, None) == 0
            assert l.barrier_all() == 0
            # either way my destination now holds my predecessor's bytes
            want = np.full(n + 64, 0xA5, np.uint8)
            want[off_d:off_d + size] = orc.fill_u8(n + 64, 100 + case, prv)[off_s:off_s + size]
            got = get_bytes(l, dst, n + 64)
            assert np.array_equal(got, want), (how, case, me, int(np.flatnonzero(got != want)[0]))
    l.free(src)
    l.free(dst)

    # ---- atomics from kernels of every process on counters spread over all PEs
    slots, ops = 64, 20000
    counters = l.malloc(slots * 8)
    assert l.fill(counters, 0, slots * 8) == 0
    ids = [orc.fill_zipf_u32(ops, 7, p, P * slots, 0.9) for p in range(P)]
    vals = [(orc.fill_u64(ops, 8, p) % 1000).astype(np.int64) for p in range(P)]
    d_ids, d_vals, d_fetched = l.dev_alloc(ops * 4), l.dev_alloc(ops * 8), l.dev_alloc(ops * 8)
    put_bytes(l, d_ids, ids[me])
    put_bytes(l, d_vals, vals[me])
    assert l.barrier_all() == 0
    assert l.amo(L.AMO_FETCH_ADD, L.LONG, counters, slots, d_ids, d_vals, None, d_fetched, ops, me, 8, 128,
                 None) == 0
    assert l.barrier_all() == 0
    total = np.zeros(P * slots, np.int64)
    for p in range(P):
        np.add.at(total, ids[p], vals[p])
    got = get_bytes(l, counters, slots * 8, np.int64)
    assert np.array_equal(got, total[me * slots:(me + 1) * slots]), me
    # every fetched value is a partial sum of that counter that includes none of the op's own operand twice
    fetched = get_bytes(l, d_fetched, ops * 8, np.int64)
    assert ((fetched >= 0) & (fetched + vals[me] <= total[ids[me]])).all()
    # host-called atomics: P increments of PE 0's first counter, then a swap by the last PE
    one = np.array([1], np.int64)
    out = np.zeros(1, np.int64)
    assert l.barrier_all() == 0
    assert l.host_amo(L.AMO_FETCH_ADD, L.LONG, counters, one.ctypes.data, None, me, 0, out.ctypes.data) == 0
    assert total[0] <= out[0] < total[0] + P
    assert l.barrier_all() == 0
    if me == 0:
        assert get_bytes(l, counters, 8, np.int64)[0] == total[0] + P
    for d in (d_ids, d_vals, d_fetched):
        l.dev_free(d)
    l.free(counters)

    # ---- put with signal into the next PE, which waits for the signal on the host
    nbytes = 40000
    data, sig = l.malloc(nbytes), l.malloc(8)
    put_bytes(l, data, np.zeros(nbytes, np.uint8))
    put_bytes(l, sig, np.zeros(1, np.uint64))
    payload = l.dev_alloc(nbytes)
    put_bytes(l, payload, orc.fill_u8(nbytes, 55, me))
    assert l.barrier_all() == 0
    assert l.put_signal(L.WG, data, payload, nbytes, sig, 1000 + me, L.SIGNAL_SET, me, nxt, 1, 256, 1, None) == 0
    want_sig = np.array([1000 + prv], np.uint64)
    ret = ctypes.c_size_t(0)
    assert l.host_wait_test(L.WAIT_UNTIL, L.ULONG, sig, 1, None, L.CMP_EQ, want_sig.ctypes.data, 20000,
                            ctypes.byref(ret), None) == 0
    assert np.array_equal(get_bytes(l, data, nbytes), orc.fill_u8(nbytes, 55, prv))
    assert l.barrier_all() == 0
    l.dev_free(payload)
    l.free(data)
    l.free(sig)

    # ---- host-called all-reduce over the world and over an active set, in and out of place
    for dtype_name in TYPES:
        for op_name in TYPES[dtype_name]:
            for n in (1, 1000, 20001):
                dt, op = getattr(L, dtype_name), getattr(L, op_name)
                np_t = orc.NP_DTYPE[getattr(orc, dtype_name)]
                es = np.dtype(np_t).itemsize
                srcs = make_inputs(orc, dtype_name, P, n, n)
                s, d = l.malloc((n + 8) * es), l.malloc((n + 8) * es)
                put_bytes(l, s, srcs[me])
                assert l.fill(d, 0x5A, (n + 8) * es) == 0
                assert l.barrier_all() == 0
                assert l.to_all(dt, op, d, s, n, 0, 0, P, None) == 0
                want = orc.to_all(getattr(orc, dtype_name), getattr(orc, op_name), srcs)
                got = get_bytes(l, d, (n + 8) * es, np_t)
                assert np.array_equal(got[:n].view(np.uint8), want.view(np.uint8)), (dtype_name, op_name, n, me)
                assert (got[n:].view(np.uint8) == 0x5A).all()
                if P >= 4 and n == 1000:  # PEs 1 and 3, in place
                    assert l.barrier_all() == 0
                    if me in (1, 3):
                        assert l.to_all(dt, op, s, s, n, 1, 1, 2, None) == 0
                        want = orc.to_all(getattr(orc, dtype_name), getattr(orc, op_name), [srcs[1], srcs[3]])
                        got = get_bytes(l, s, n * es, np_t)
                        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (dtype_name, op_name, me)
                l.free(s)
                l.free(d)

    # ---- team collectives called from the host: alltoall, fcollect, broadcast
    nb = 7001
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
    root = P - 1
    assert l.broadcastmem(world, d, s, nb, root, None) == 0
    want = [np.full(nb, 0x11, np.uint8) for _ in range(P)]
    orc.broadcast([x[:nb] for x in srcs], want, nb, root)
    assert np.array_equal(get_bytes(l, d, nb), want[me])
    assert l.barrier_all() == 0

    # ---- what belongs to the one-process harness is refused, not misrun
    assert l.wg_reduce(L.INT, L.SUM, world, d, s, 4, 64, None) == -1
    assert l.rma(L.PUT, L.WG, d, s, 16, 0, nxt, me, 1, 64, 1, None) == -1  # cannot act for another PE
    l.free(s)
    l.free(d)
    assert l.finalize() == 0
    print("ok", me)


if __name__ == "__main__":
    main()
