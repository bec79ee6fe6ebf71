"""Host-side API on the emulated heap: put/get from host and device buffers,
atomics, test / wait_until families, active-set broadcast.  Through the C entry
points; results exact against the oracle."""
import ctypes
import os
import threading
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P, HEAP = 8, 1 << 30
GUARD = 64
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

NP = {"INT": np.int32, "LONG": np.int64, "LONGLONG": np.int64, "UINT": np.uint32,
      "ULONG": np.uint64, "ULONGLONG": np.uint64, "FLOAT": np.float32, "DOUBLE": np.float64,
      "SHORT": np.int16, "CHAR": np.int8, "SCHAR": np.int8, "UCHAR": np.uint8,
      "USHORT": np.uint16}


def one(np_t, v):
    return np.array([v], np_t)


# ---------------------------------------------------------------- put / get
@pytest.mark.parametrize("local", ["host", "device"])
def test_host_put_get_every_size_and_alignment(rt, L, orc, local):
    """src/host/host_helpers.hpp:52-88: put lands on `pe` at the same offset,
    get fetches from it; nothing outside [dest, dest+n) changes.  The local
    buffer is pageable host memory or plain device memory."""
    l = rt.up(P, HEAP)
    size = 1 << 20
    sym = l.malloc(size + 2 * GUARD + 32)
    host = orc.fill_u8(size + 32, 7, 1)
    dev = rt.dev_array(host) if local == "device" else None
    back_dev = l.dev_alloc(size + 32) if local == "device" else None
    cases = [(n, 3, 5) for n in list(range(0, 70)) + [255, 4099, 65536, 100001, size]]
    cases += [(777, s, d) for s in range(0, 16, 5) for d in range(16)]
    for n, soff, doff in cases:
        me, pe = (n % P), ((n * 3 + 1) % P)
        landing = l.pe_ptr(sym, pe) + GUARD + doff
        l.fill(landing - GUARD, 0xA5, n + 2 * GUARD)
        l.stream_sync(None)  # host put/get are not ordered with work queued on HIP streams
        src = (dev + soff) if dev else (host.ctypes.data + soff)
        assert l.host_putmem(l.pe_ptr(sym, me) + GUARD + doff, src, n, me, pe) == 0
        got = rt.get_bytes(landing - GUARD, n + 2 * GUARD)
        want = np.full(n + 2 * GUARD, 0xA5, np.uint8)
        want[GUARD:GUARD + n] = host[soff:soff + n]
        assert np.array_equal(got, want), ("put", n, soff, doff, me, pe)
        # and back through get, into a guarded local buffer
        if dev:
            l.fill(back_dev, 0x5A, size + 32)
            l.stream_sync(None)
            assert l.host_getmem(back_dev + 1, l.pe_ptr(sym, me) + GUARD + doff, n, me, pe) == 0
            back = rt.get_bytes(back_dev, n + 2)
        else:
            back = np.full(n + 2, 0x5A, np.uint8)
            assert l.host_getmem(back.ctypes.data + 1, l.pe_ptr(sym, me) + GUARD + doff, n, me, pe) == 0
        assert back[0] == 0x5A and back[n + 1] == 0x5A
        assert np.array_equal(back[1:1 + n], host[soff:soff + n]), ("get", n, soff, doff)
    if dev:
        l.dev_free(dev)
        l.dev_free(back_dev)
    l.free(sym)


def test_host_put_get_argument_errors(rt, L):
    l = rt.up(P, HEAP)
    sym = l.malloc(256)
    buf = np.zeros(256, np.uint8)
    assert l.host_putmem(sym, buf.ctypes.data, 16, 0, P) == -1            # bad PE
    assert l.host_putmem(sym, buf.ctypes.data, 16, -1, 0) == -1
    assert l.host_putmem(None, buf.ctypes.data, 16, 0, 1) == -1          # null symmetric side
    assert l.host_putmem(sym, None, 16, 0, 1) == -1
    assert l.host_putmem(l.pe_ptr(sym, 1), buf.ctypes.data, 16, 0, 1) == -1  # not my_pe's address
    assert l.host_putmem(sym, buf.ctypes.data, HEAP + 1, 0, 1) == -1     # beyond the slice
    assert l.host_getmem(buf.ctypes.data, buf.ctypes.data, 16, 0, 1) == -1  # source not symmetric
    assert l.host_putmem(sym, buf.ctypes.data, 0, 0, 1) == 0             # empty message
    l.free(sym)


def test_ctx_pe(rt, L):
    l = rt.up(P, HEAP)
    assert l.ctx_pe(None) == 0
    l.set_pe(5)
    assert l.ctx_pe(None) == 5
    l.set_pe(0)
    junk = np.zeros(8, np.uint8)
    assert l.ctx_pe(junk.ctypes.data) == -1


# ------------------------------------------------------------------ atomics
@pytest.mark.parametrize("dtype_name", ["INT", "LONG", "LONGLONG", "UINT", "ULONG", "ULONGLONG"])
def test_host_standard_atomics(rt, L, orc, dtype_name):
    """src/host/host_templates.hpp:254-330 and the known answers of
    tests/sos_tests/cxx_test_shmem_atomic_*.cpp: a chain of host atomics onto
    a word of another PE, every fetched value and the final word checked
    against the oracle's model of the same chain."""
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    dt = getattr(L, dtype_name)
    word = l.malloc(8)
    init = 1000
    for p in range(P):
        rt.put_bytes(l.pe_ptr(word, p), one(np_t, init))
    ops = [(L.AMO_FETCH_ADD, 5, 0), (L.AMO_ADD, 7, 0), (L.AMO_FETCH_INC, 0, 0), (L.AMO_INC, 0, 0),
           (L.AMO_COMPARE_SWAP, 99, 1014), (L.AMO_COMPARE_SWAP, 123, 1), (L.AMO_FETCH_ADD, -3, 0)]
    model = np.array([init], np.int64)
    for me, pe in ((0, 3), (6, 6), (2, 0)):
        rt.put_bytes(l.pe_ptr(word, pe), one(np_t, init))
        model[:] = init
        for op, v, c in ops:
            if v < 0 and np.dtype(np_t).kind == "u":
                v = 3
            val, cond, out = one(np_t, v), one(np_t, c), one(np_t, 0)
            assert l.host_amo(op, dt, l.pe_ptr(word, me), val.ctypes.data, cond.ctypes.data, me, pe,
                              out.ctypes.data) == 0
            model, fetched = orc.amo_i64(op, model, [0], [v], [c])
            if op not in (L.AMO_ADD, L.AMO_INC):
                assert int(out[0]) == int(fetched[0]), (dtype_name, op, v)
            assert int(rt.get_bytes(l.pe_ptr(word, pe), np.dtype(np_t).itemsize, np_t)[0]) == int(model[0])
    # the other PEs' words were never touched by the last chain
    assert int(rt.get_bytes(l.pe_ptr(word, 5), np.dtype(np_t).itemsize, np_t)[0]) == init
    l.free(word)


@pytest.mark.parametrize("dtype_name", ["INT", "LONG", "UINT", "ULONG", "FLOAT", "DOUBLE"])
def test_host_extended_atomics(rt, L, dtype_name):
    """fetch / set / swap (tests/sos_tests/cxx_test_shmem_atomic_fetch.cpp):
    set then fetch returns the value; swap returns the old one."""
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    dt = getattr(L, dtype_name)
    word = l.malloc(8)
    a, b = (1.5, -2.25) if np.dtype(np_t).kind == "f" else (41, 17)
    out, zero = one(np_t, 0), one(np_t, 0)
    assert l.host_amo(L.AMO_SET, dt, word, one(np_t, a).ctypes.data, None, 0, 4, None) == 0
    assert l.host_amo(L.AMO_FETCH, dt, word, zero.ctypes.data, None, 0, 4, out.ctypes.data) == 0
    assert out[0] == np_t(a)
    assert l.host_amo(L.AMO_SWAP, dt, word, one(np_t, b).ctypes.data, None, 0, 4, out.ctypes.data) == 0
    assert out[0] == np_t(a)
    assert rt.get_bytes(l.pe_ptr(word, 4), np.dtype(np_t).itemsize, np_t)[0] == np_t(b)
    l.free(word)


def test_host_bitwise_atomics_and_errors(rt, L):
    l = rt.up(P, HEAP)
    word = l.malloc(8)
    rt.put_bytes(l.pe_ptr(word, 2), one(np.uint64, 0b1100))
    out = one(np.uint64, 0)
    for op, v, old, new in ((L.AMO_FETCH_AND, 0b1010, 0b1100, 0b1000), (L.AMO_FETCH_OR, 0b0011, 0b1000, 0b1011),
                            (L.AMO_FETCH_XOR, 0b1111, 0b1011, 0b0100)):
        assert l.host_amo(op, L.ULONG, word, one(np.uint64, v).ctypes.data, None, 0, 2, out.ctypes.data) == 0
        assert int(out[0]) == old
        assert int(rt.get_bytes(l.pe_ptr(word, 2), 8, np.uint64)[0]) == new
    v = one(np.int64, 1)
    assert l.host_amo(L.AMO_FETCH_ADD, L.SHORT, word, v.ctypes.data, None, 0, 1, None) == -1  # no 2-byte atomics
    assert l.host_amo(L.AMO_FETCH_ADD, L.FLOAT, word, v.ctypes.data, None, 0, 1, None) == -1  # add is integer-only
    assert l.host_amo(L.AMO_COMPARE_SWAP, L.LONG, word, v.ctypes.data, None, 0, 1, None) == -1  # needs cond
    assert l.host_amo(L.AMO_FETCH_ADD, L.LONG, word, v.ctypes.data, None, 0, P, None) == -1
    l.free(word)


# ---------------------------------------------------------------- waits
@pytest.mark.parametrize("dtype_name", ["FLOAT", "DOUBLE", "CHAR", "SCHAR", "SHORT", "INT", "LONG",
                                        "LONGLONG", "UCHAR", "USHORT", "UINT", "ULONG", "ULONGLONG"])
def test_host_test_truth_table(rt, L, orc, dtype_name):
    """src/host/host_templates.hpp:395-424 for all 13 wait types and the six
    comparators, plus an unknown comparator (never holds)."""
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    k = np.dtype(np_t)
    if k.kind == "f":
        samples = [-1.5, 0.0, 2.25]
    elif k.kind == "u":
        samples = [0, 7, int(np.iinfo(np_t).max)]
    else:
        samples = [int(np.iinfo(np_t).min), 0, int(np.iinfo(np_t).max)]
    iv = l.malloc(8)
    dt = getattr(L, dtype_name)
    for x in samples:
        rt.put_bytes(iv, one(np_t, x))
        for v in samples:
            for cmp in range(7):
                ret = ctypes.c_size_t(99)
                assert l.host_wait_test(L.TEST, dt, iv, 1, None, cmp, one(np_t, v).ctypes.data, 0,
                                        ctypes.byref(ret), None) == 0
                assert ret.value == orc.test_value(getattr(orc, dtype_name), cmp, x, v), (dtype_name, x, cmp, v)
    l.free(iv)


def test_host_wait_any_all_some_on_settled_values(rt, L, orc):
    """src/host/host_templates.hpp:502-598 on values that no longer change:
    any -> first satisfied unmasked index, some -> all of them, all -> returns;
    empty and fully masked sets; sets nothing satisfies give up at the limit."""
    l = rt.up(P, HEAP)
    host = np.array([0, 5, 0, 5, 5, 1], np.int64)
    iv = rt.dev_array(host)
    five, nine = one(np.int64, 5), one(np.int64, 9)
    for status in (None, [0] * 6, [0, 1, 0, 0, 0, 0], [1, 1, 1, 0, 1, 0], [1, 1, 0, 0, 0, 0], [1] * 6):
        st = np.array(status, np.int32) if status is not None else None
        stp = st.ctypes.data if st is not None else None
        ret = ctypes.c_size_t()
        idx = np.full(6, orc.SIZE_MAX, np.uint64)
        want_any = orc.wait_until_any(orc.LONG, host, status, L.CMP_EQ, 5)
        rc = l.host_wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 6, stp, L.CMP_EQ, five.ctypes.data, 50,
                              ctypes.byref(ret), None)
        assert (rc, ret.value) == (0, want_any), status
        want_n, want_idx = orc.wait_until_some(orc.LONG, host, status, L.CMP_EQ, 5)
        rc = l.host_wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 6, stp, L.CMP_EQ, five.ctypes.data, 50,
                              ctypes.byref(ret), idx.ctypes.data)
        assert (rc, ret.value) == (0, want_n), status
        assert np.array_equal(idx[:want_n], want_idx[:want_n])
        # GE 0 holds everywhere: all returns at once whatever is masked
        assert l.host_wait_test(L.WAIT_UNTIL_ALL, L.LONG, iv, 6, stp, L.CMP_GE, one(np.int64, 0).ctypes.data,
                                50, ctypes.byref(ret), None) == 0
    ret = ctypes.c_size_t()
    # nothing equals 9: the oracle says these block; the bounded call reports the time-out
    assert orc.wait_until_any(orc.LONG, host, None, L.CMP_EQ, 9) == orc.WOULD_BLOCK
    t0 = time.time()
    assert l.host_wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 6, None, L.CMP_EQ, nine.ctypes.data, 30,
                            ctypes.byref(ret), None) == 1
    assert ret.value == orc.SIZE_MAX and time.time() - t0 < 5
    assert l.host_wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_EQ, nine.ctypes.data, 30,
                            ctypes.byref(ret), None) == 1
    assert l.host_wait_test(L.WAIT_UNTIL_ALL, L.LONG, iv, 6, None, L.CMP_EQ, five.ctypes.data, 30,
                            ctypes.byref(ret), None) == 1
    idx = np.zeros(6, np.uint64)
    assert l.host_wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 6, None, L.CMP_EQ, nine.ctypes.data, 30,
                            ctypes.byref(ret), idx.ctypes.data) == 1 and ret.value == 0
    # nelems == 0
    assert l.host_wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 0, None, L.CMP_EQ, five.ctypes.data, 30,
                            ctypes.byref(ret), None) == 0 and ret.value == orc.SIZE_MAX
    assert l.host_wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 0, None, L.CMP_EQ, five.ctypes.data, 30,
                            ctypes.byref(ret), None) == 0 and ret.value == 0
    l.dev_free(iv)


@pytest.mark.parametrize("fn", ["WAIT_UNTIL", "WAIT_UNTIL_ANY", "WAIT_UNTIL_ALL", "WAIT_UNTIL_SOME"])
def test_host_waits_are_released_by_a_later_put(rt, L, fn):
    """tests/sos_tests/waituntil.cpp / thread_wait.cpp: the waiter blocks until
    another party's put changes the word (here a second host thread acting for
    another PE, 50 ms later)."""
    l = rt.up(P, HEAP)
    sym = l.malloc(4 * 8)
    mine = l.pe_ptr(sym, 3)
    l.fill(mine, 0, 32)
    l.stream_sync(None)
    seven = one(np.int64, 7)

    def release():
        time.sleep(0.05)
        words = [2] if fn != "WAIT_UNTIL_ALL" else [0, 1, 2, 3]
        for w in words:
            assert l.host_putmem(l.pe_ptr(sym, 6) + 8 * w, seven.ctypes.data, 8, 6, 3) == 0

    t = threading.Thread(target=release)
    ret = ctypes.c_size_t(99)
    idx = np.full(4, 99, np.uint64)
    t0 = time.time()
    t.start()
    ivars = mine + (16 if fn == "WAIT_UNTIL" else 0)
    rc = l.host_wait_test(getattr(L, fn), L.LONG, ivars, 4, None, L.CMP_EQ, seven.ctypes.data, 20000,
                          ctypes.byref(ret), idx.ctypes.data)
    waited = time.time() - t0
    t.join()
    assert rc == 0 and waited >= 0.04
    if fn == "WAIT_UNTIL_ANY":
        assert ret.value == 2
    if fn == "WAIT_UNTIL_SOME":
        assert ret.value == 1 and idx[0] == 2
    l.free(sym)


@pytest.mark.parametrize("how", ["put", "atomic"])
def test_host_put_reaches_a_kernel_that_is_already_waiting(rt, L, how):
    """A kernel polls rocshmem_long_test on its PE's word (bounded: it gives up
    after a few seconds); while it runs, the host, acting for another PE, puts
    or atomically sets the value.  The host call must neither wait for the
    kernel nor be invisible to it: the kernel reports that it saw the value,
    after a number of polls that shows it was really waiting."""
    l = rt.up(P, HEAP)
    sym = l.malloc(8)
    l.fill(l.pe_ptr(sym, 2), 0, 8)
    res = l.dev_alloc(16)
    l.fill(res, 0xFF, 16)
    l.stream_sync(None)
    seven = one(np.int64, 7)
    assert l.poll_until(L.LONG, l.pe_ptr(sym, 2), L.CMP_EQ, seven.ctypes.data, 4_000_000, res, None) == 0
    time.sleep(0.05)
    t0 = time.time()
    if how == "put":
        assert l.host_putmem(l.pe_ptr(sym, 5), seven.ctypes.data, 8, 5, 2) == 0
    else:
        assert l.host_amo(L.AMO_SET, L.LONG, l.pe_ptr(sym, 5), seven.ctypes.data, None, 5, 2, None) == 0
    host_call_s = time.time() - t0
    l.stream_sync(None)
    seen, polls = (int(x) for x in rt.get_bytes(res, 16, np.uint64))
    assert seen == 1 and polls > 1000, (seen, polls)
    assert host_call_s < 2.0, host_call_s
    l.dev_free(res)
    l.free(sym)


def test_host_wait_argument_errors(rt, L):
    l = rt.up(P, HEAP)
    iv = l.malloc(64)
    v = one(np.int64, 0)
    ret = ctypes.c_size_t()
    assert l.host_wait_test(L.TEST, L.BF16, iv, 1, None, 0, v.ctypes.data, 0, ctypes.byref(ret), None) == -1
    assert l.host_wait_test(9, L.LONG, iv, 1, None, 0, v.ctypes.data, 0, ctypes.byref(ret), None) == -1
    assert l.host_wait_test(L.TEST, L.LONG, None, 1, None, 0, v.ctypes.data, 0, ctypes.byref(ret), None) == -1
    assert l.host_wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 4, None, 0, v.ctypes.data, 0, ctypes.byref(ret), None) == -1
    assert l.host_wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, HEAP, None, 0, v.ctypes.data, 0, ctypes.byref(ret), None) == -1
    l.free(iv)


# ------------------------------------------------------- active-set broadcast
@pytest.mark.parametrize("start,log_stride,size,root", [(0, 0, 8, 0), (0, 0, 8, 5), (1, 1, 3, 2),
                                                        (2, 0, 4, 1), (0, 2, 2, 1), (3, 0, 1, 0)])
def test_host_broadcast_over_an_active_set(rt, L, orc, start, log_stride, size, root):
    """src/host/host_templates.hpp:160-175 and
    tests/sos_tests/broadcast_active_set.cpp: members other than the root
    receive the root's source; the root's dest and non-members stay as they were."""
    l = rt.up(P, HEAP)
    n = 100003
    src, dst = l.malloc(n), l.malloc(n)
    members = [start + (i << log_stride) for i in range(size)]
    srcs = [orc.fill_u8(n, 9, p) for p in range(P)]
    for p in range(P):
        rt.put_bytes(l.pe_ptr(src, p), srcs[p])
        l.fill(l.pe_ptr(dst, p), 0x77, n)
    assert l.broadcast_active_set(l.pe_ptr(dst, start), l.pe_ptr(src, start), n, root, start, log_stride,
                                  size, None) == 0
    l.stream_sync(None)
    want = [np.full(n, 0x77, np.uint8) for _ in members]
    orc.broadcast([srcs[p] for p in members], want, n, root)
    for p in range(P):
        got = rt.get_bytes(l.pe_ptr(dst, p), n)
        if p in members:
            assert np.array_equal(got, want[members.index(p)]), p
        else:
            assert (got == 0x77).all(), p
    assert (want[root] == 0x77).all()
    assert l.broadcast_active_set(dst, src, n, size, start, log_stride, size, None) == -1   # root outside the set
    assert l.broadcast_active_set(dst, src, n, 0, 6, 1, 3, None) == -1                      # set runs past the last PE
    l.free(src)
    l.free(dst)
