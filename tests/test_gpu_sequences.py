"""Seeded random programs over the whole path: host-initiated copies, device
put/get and put-with-signal at every granularity, all-reduce over active sets
and teams (whole-GPU and one work-group per member), whole-GPU and
per-work-group alltoall / fcollect / broadcast on strided teams, host atomics —
one after another on the same three symmetric buffers, mirrored step by step
on numpy arrays with the oracle's folds and index maps.  After every step the
touched buffer, and at the end every buffer on every PE, must equal the mirror
byte for byte: what one call leaves behind (barrier epochs, team scratch,
write-through stores) must not disturb the next.  Through the C entry points."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HEAP = 64 << 20
SIZE = 1 << 20          # bytes per symmetric buffer
INT_TYPES = ("SHORT", "INT", "LONG", "LONGLONG")
OPS = ("SUM", "MAX", "MIN", "PROD", "AND", "OR", "XOR")


class Mirror:
    def __init__(self, rt, l, orc, npes, seed):
        self.rt, self.l, self.npes = rt, l, npes
        self.names = ("a", "b", "c")
        self.dev = {k: l.malloc(SIZE) for k in self.names}
        assert all(self.dev.values())
        self.host = {k: [orc.fill_u8(SIZE, seed, 16 * i + p) for p in range(npes)]
                     for i, k in enumerate(self.names)}
        for k in self.names:
            for p in range(npes):
                rt.put_bytes(l.pe_ptr(self.dev[k], p), self.host[k][p])

    def check(self, what, names=None):
        self.l.stream_sync(None)
        for k in names or self.names:
            for p in range(self.npes):
                got = self.rt.get_bytes(self.l.pe_ptr(self.dev[k], p), SIZE)
                if not np.array_equal(got, self.host[k][p]):
                    bad = np.flatnonzero(got != self.host[k][p])
                    raise AssertionError("%s: buffer %s on PE %d differs at %d bytes, first %d"
                                         % (what, k, p, bad.size, bad[0]))

    def close(self):
        for k in self.names:
            self.l.free(self.dev[k])


def random_team(rng, npes):
    """(start, stride, size) of a strided team inside the world."""
    size = int(rng.integers(1, npes + 1))
    stride = 1 if size == 1 else int(rng.integers(1, (npes - 1) // (size - 1) + 1))
    start = int(rng.integers(0, npes - (size - 1) * stride))
    return start, stride, size


def step_copy(rng, m, L):
    l = m.l
    s, d = rng.choice(m.names, 2, replace=False)
    me, pe = (int(x) for x in rng.integers(0, m.npes, 2))
    kind = rng.choice(["host_put", "host_get", "thread", "wave", "wg"])
    top = {"thread": 3000, "wave": 40000, "wg": 300000}.get(kind, 400000)
    n = int(rng.integers(0, top))
    so, do = (int(x) for x in rng.integers(0, SIZE - n + 1, 2))
    put = kind == "host_put" or (kind not in ("host_put", "host_get") and rng.integers(2) == 0)
    # every address is the one on `me`; the library resolves the remote side on `pe`
    if put:   # me's s[so:] -> pe's d[do:]
        dst_addr, src_addr = l.pe_ptr(m.dev[d], me) + do, l.pe_ptr(m.dev[s], me) + so
        src_pe, dst_pe = me, pe
    else:     # pe's s[so:] -> me's d[do:]
        dst_addr, src_addr = l.pe_ptr(m.dev[d], me) + do, l.pe_ptr(m.dev[s], me) + so
        src_pe, dst_pe = pe, me
    what = "%s %s n=%d %s[%d]@%d -> %s[%d]@%d" % (kind, "put" if put else "get", n, s, so, src_pe,
                                                 d, do, dst_pe)
    if kind == "host_put":
        assert l.putmem(dst_addr, src_addr, n, me, pe, None) == 0, what
    elif kind == "host_get":
        assert l.getmem(dst_addr, src_addr, n, me, pe, None) == 0, what
    else:
        gran = {"thread": L.THREAD, "wave": L.WAVE, "wg": L.WG}[kind]
        n_wgs = int(rng.integers(1, 5))
        wg = int(rng.choice([64, 128, 256, 1024])) if kind != "thread" else int(rng.choice([1, 7, 64]))
        assert l.rma(L.PUT if put else L.GET, gran, dst_addr, src_addr, n, 0, me, pe, n_wgs, wg, 1,
                     None) == 0, what
    m.host[d][dst_pe][do:do + n] = m.host[s][src_pe][so:so + n]
    return what, [d]


def step_reduce(rng, m, L, orc):
    """Active-set to_all, team reduce (both whole-GPU) or the device call
    wg_reduce with one work-group per member."""
    l = m.l
    tname = str(rng.choice(INT_TYPES))
    oname = str(rng.choice(OPS))
    dtype, op = getattr(L, tname), getattr(L, oname)
    npd = orc.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    mode = str(rng.choice(["to_all", "reduce", "wg_reduce"]))
    if mode == "to_all":
        size = int(rng.integers(1, m.npes + 1))
        log_stride = 0
        while size > 1 and rng.integers(2) and (size - 1) * (2 << log_stride) < m.npes:
            log_stride += 1
        stride = 1 << log_stride
        start = int(rng.integers(0, m.npes - (size - 1) * stride))
    else:
        start, stride, size = random_team(rng, m.npes)
    pes = [start + stride * k for k in range(size)]
    n = int(rng.integers(0, 20000))
    s, d = rng.choice(m.names, 2, replace=False)
    so = int(rng.integers(0, (SIZE - n * es) // es + 1)) * es
    do = int(rng.integers(0, (SIZE - n * es) // es + 1)) * es
    if rng.integers(4) == 0:
        d, do = s, so                       # in place
    what = "%s %s %s n=%d set=(%d,%d,%d) %s@%d -> %s@%d" % (mode, tname, oname, n, start, stride,
                                                            size, s, so, d, do)
    if mode == "to_all":
        assert l.to_all(dtype, op, l.pe_ptr(m.dev[d], start) + do, l.pe_ptr(m.dev[s], start) + so,
                        n, start, log_stride, size, None) == 0, what
    else:
        me = pes[int(rng.integers(0, size))]
        l.set_pe(me)
        team = ctypes.c_void_p()
        assert l.team_split_strided(l.team_world(), start, stride, size, ctypes.byref(team)) == 0
        da, sa = l.pe_ptr(m.dev[d], me) + do, l.pe_ptr(m.dev[s], me) + so
        if mode == "reduce":
            assert l.reduce(dtype, op, team, da, sa, n, None) == 0, what
        else:
            assert l.wg_reduce(dtype, op, team, da, sa, n, int(rng.choice([64, 256, 1024])),
                               None) == 0, what
        l.stream_sync(None)
        l.team_destroy(team)
        l.set_pe(0)
    if n:
        srcs = [m.host[s][p][so:so + n * es].view(npd).copy() for p in pes]
        out = orc.to_all(dtype, op, srcs)
        for p in pes:
            m.host[d][p][do:do + n * es] = out.view(np.uint8)
    return what, [d]


def step_put_signal(rng, m, L):
    """putmem_signal at thread / wavefront / work-group granularity: every group
    sends its tile and updates the signal word, `calls` times."""
    l = m.l
    s, d, g = rng.permutation(m.names)
    me, pe = (int(x) for x in rng.integers(0, m.npes, 2))
    gran = str(rng.choice(["THREAD", "WAVE", "WG"]))
    n_wgs = int(rng.integers(1, 4))
    wg = int(rng.choice([64, 128, 256]))
    groups = {"THREAD": n_wgs * wg, "WAVE": n_wgs * (wg // 64), "WG": n_wgs}[gran]
    n = groups * 16 * int(rng.integers(1, 9))     # whole 16-byte tiles: every group sends
    so, do = (int(x) for x in rng.integers(0, SIZE - n + 1, 2))
    slot = int(rng.integers(0, SIZE // 8))
    calls = int(rng.integers(1, 4))
    signal = int(rng.integers(1, 1 << 40))
    add = bool(rng.integers(2))
    what = "put_signal %s n=%d groups=%d calls=%d %s %s@%d[%d] -> %s@%d[%d] sig %s[%d]" % (
        gran, n, groups, calls, "ADD" if add else "SET", s, me, so, d, pe, do, g, slot)
    rc = l.put_signal(getattr(L, gran), l.pe_ptr(m.dev[d], me) + do, l.pe_ptr(m.dev[s], me) + so, n,
                      l.pe_ptr(m.dev[g], me) + slot * 8, signal,
                      L.SIGNAL_ADD if add else L.SIGNAL_SET, me, pe, n_wgs, wg, calls, None)
    assert rc == 0, what
    m.host[d][pe][do:do + n] = m.host[s][me][so:so + n]
    word = m.host[g][pe][slot * 8:slot * 8 + 8].view(np.uint64)
    word[0] = (int(word[0]) + calls * groups * signal) % (1 << 64) if add else signal
    return what, [d, g]


def step_move(rng, m, L, orc):
    l = m.l
    start, stride, size = random_team(rng, m.npes)
    pes = [start + stride * k for k in range(size)]
    kind = str(rng.choice(["alltoall", "fcollect", "broadcast"]))
    mode = str(rng.choice(["grid", "wg"]))
    elem = 1 if mode == "grid" else int(rng.choice([1, 2, 4, 8]))
    nelems = int(rng.integers(0, 60000 // (elem * size) + 1))
    n = elem * nelems
    root = int(rng.integers(0, size))
    s, d = rng.choice(m.names, 2, replace=False)
    src_bytes = n * size if kind == "alltoall" else n
    dst_bytes = n if kind == "broadcast" else n * size
    so = int(rng.integers(0, (SIZE - src_bytes) // elem + 1)) * elem
    do = int(rng.integers(0, (SIZE - dst_bytes) // elem + 1)) * elem
    what = "%s %s elem=%d nelems=%d team=(%d,%d,%d) root=%d %s@%d -> %s@%d" % (
        mode, kind, elem, nelems, start, stride, size, root, s, so, d, do)
    me = pes[int(rng.integers(0, size))]
    l.set_pe(me)
    team = ctypes.c_void_p()
    assert l.team_split_strided(l.team_world(), start, stride, size, ctypes.byref(team)) == 0, what
    da, sa = l.pe_ptr(m.dev[d], me) + do, l.pe_ptr(m.dev[s], me) + so
    if mode == "wg":
        wg = int(rng.choice([64, 256, 1024]))
        if kind == "alltoall":
            rc = l.wg_alltoall(elem, team, da, sa, nelems, wg, None)
        elif kind == "fcollect":
            rc = l.wg_fcollect(elem, team, da, sa, nelems, wg, None)
        else:
            rc = l.wg_broadcast(elem, team, da, sa, nelems, root, wg, None)
    else:
        if kind == "alltoall":
            rc = l.alltoallmem(team, da, sa, n, None)
        elif kind == "fcollect":
            rc = l.fcollectmem(team, da, sa, n, None)
        else:
            rc = l.broadcastmem(team, da, sa, n, root, None)
    assert rc == 0, what
    l.stream_sync(None)
    l.team_destroy(team)
    l.set_pe(0)
    if n:
        srcs = [m.host[s][p][so:so + src_bytes].copy() for p in pes]
        if kind == "alltoall":
            outs = orc.alltoall(srcs, n)
        elif kind == "fcollect":
            outs = orc.fcollect(srcs, n)
        else:
            outs = [m.host[d][p][do:do + n].copy() for p in pes]
            orc.broadcast(srcs, outs, n, root)
        for k, p in enumerate(pes):
            m.host[d][p][do:do + dst_bytes] = outs[k]
    return what, [d]


def step_amo(rng, m, L):
    l = m.l
    d = str(rng.choice(m.names))
    me, pe = (int(x) for x in rng.integers(0, m.npes, 2))
    slot = int(rng.integers(0, SIZE // 8))
    word = m.host[d][pe][slot * 8:slot * 8 + 8].view(np.int64)
    old = int(word[0])
    value = ctypes.c_int64(int(rng.integers(-1 << 62, 1 << 62)))
    hit = bool(rng.integers(2))
    cond = ctypes.c_int64(old if hit else old ^ 1)
    fetched = ctypes.c_int64(0x5A5A5A5A)
    opname = str(rng.choice(["FETCH_ADD", "ADD", "FETCH_INC", "INC", "COMPARE_SWAP", "FETCH", "SET",
                             "SWAP", "FETCH_AND", "FETCH_OR", "FETCH_XOR"]))
    what = "host_amo %s %s[%d] me=%d pe=%d" % (opname, d, slot, me, pe)
    # the bitwise operations exist for the unsigned types only (rocshmem_AMO.hpp)
    dtype = L.ULONG if opname in ("FETCH_AND", "FETCH_OR", "FETCH_XOR") else L.LONG
    rc = l.host_amo(getattr(L, "AMO_" + opname), dtype, l.pe_ptr(m.dev[d], me) + slot * 8,
                    ctypes.byref(value), ctypes.byref(cond), me, pe, ctypes.byref(fetched))
    assert rc == 0, what
    v = value.value
    new = {"FETCH_ADD": old + v, "ADD": old + v, "FETCH_INC": old + 1, "INC": old + 1,
           "COMPARE_SWAP": v if hit else old, "FETCH": old, "SET": v, "SWAP": v,
           "FETCH_AND": old & v, "FETCH_OR": old | v, "FETCH_XOR": old ^ v}[opname]
    new = (new + (1 << 63)) % (1 << 64) - (1 << 63)
    word[0] = new
    if opname not in ("ADD", "INC", "SET"):
        assert fetched.value == old, what
    return what, [d]


@pytest.mark.parametrize("npes,seed", [(8, 0), (8, 1), (5, 2), (3, 3), (2, 4), (1, 5), (8, 6), (7, 7),
                                       (4, 8), (6, 9)])
def test_random_program(rt, L, orc, npes, seed):
    l = rt.up(npes, HEAP)
    rng = np.random.default_rng(1000 + seed)
    m = Mirror(rt, l, orc, npes, seed)
    log = []
    # odd seeds drive the RMA and put-with-signal steps through NOSTORE contexts
    l.set_ctx_options(L.CTX_NOSTORE if seed % 2 else 0)
    try:
        for k in range(150):
            r = rng.integers(12)
            if r < 4:
                what, touched = step_copy(rng, m, L)
            elif r < 7:
                what, touched = step_reduce(rng, m, L, orc)
            elif r < 10:
                what, touched = step_move(rng, m, L, orc)
            elif r < 11:
                what, touched = step_put_signal(rng, m, L)
            else:
                what, touched = step_amo(rng, m, L)
            log.append(what)
            m.check("step %d of seed %d: %s" % (k, seed, what), touched)
        m.check("end of seed %d (after: %s)" % (seed, "; ".join(log[-3:])))
    finally:
        l.set_ctx_options(0)
        l.set_pe(0)
        m.close()
