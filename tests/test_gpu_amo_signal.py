"""A1, S1, W1, X1, C4: atomics, put-with-signal, signal_fetch, waits, the
ping-pong and dispatch patterns, context lifecycle and wavefront coalescing.
Integer results exact against the oracle.  Through the C entry points."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P, HEAP = 8, 1 << 30
NP = {"INT": np.int32, "LONG": np.int64, "LONGLONG": np.int64, "UINT": np.uint32,
      "ULONG": np.uint64, "ULONGLONG": np.uint64, "FLOAT": np.float32, "DOUBLE": np.float64,
      "SHORT": np.int16}


@pytest.fixture(autouse=True, params=[0, 1], ids=["default_ctx", "nostore_ctx"])
def ctx_options(request, rt):
    """Every case runs through default contexts and through contexts created
    with ROCSHMEM_CTX_NOSTORE (relaxed AMOs, no L2 write-back on completion):
    the values that land must not depend on it."""
    l = rt.up(P, HEAP)
    before = l.set_ctx_options(request.param)
    yield request.param
    l.set_ctx_options(max(before, 0))


class Counters:
    """n_slots symmetric counters per PE, viewed as one PE-major array."""

    def __init__(self, rt, l, n_slots, np_t, init=0):
        self.rt, self.l, self.n, self.t = rt, l, n_slots, np_t
        self.ptr = l.malloc(n_slots * np.dtype(np_t).itemsize)
        self.set_all(np.full(P * n_slots, init, np_t))

    def set_all(self, values):
        for p in range(P):
            self.rt.put_bytes(self.l.pe_ptr(self.ptr, p), values[p * self.n:(p + 1) * self.n])

    def read_all(self):
        es = np.dtype(self.t).itemsize
        return np.concatenate([self.rt.get_bytes(self.l.pe_ptr(self.ptr, p), self.n * es, self.t)
                               for p in range(P)])

    def free(self):
        self.l.free(self.ptr)


def run_amo(rt, l, L, op, dtype_name, ctr, ids, values=None, conds=None, fetch=True, n_wgs=64,
            wg=256, my_pe=0):
    np_t = NP[dtype_name]
    d_ids = rt.dev_array(np.ascontiguousarray(ids, np.uint32))
    d_val = rt.dev_array(np.ascontiguousarray(values, np_t)) if values is not None else None
    d_cond = rt.dev_array(np.ascontiguousarray(conds, np_t)) if conds is not None else None
    d_out = l.dev_alloc(max(len(ids), 1) * np.dtype(np_t).itemsize) if fetch else None
    rc = l.amo(op, getattr(L, dtype_name), l.pe_ptr(ctr.ptr, my_pe), ctr.n, d_ids, d_val, d_cond,
               d_out, len(ids), my_pe, n_wgs, wg, None)
    assert rc == 0
    l.stream_sync(None)
    out = rt.get_bytes(d_out, len(ids) * np.dtype(np_t).itemsize, np_t) if fetch else None
    for d in (d_ids, d_val, d_cond, d_out):
        if d:
            l.dev_free(d)
    return out


def check_fetch_chain(ids, fetched, values, init):
    """Per counter the fetched values must be the running sums of the addends
    in SOME order: sorted by fetched value, each equals its predecessor plus
    the predecessor's addend (addends > 0 make the order unique)."""
    order = np.lexsort((fetched, ids))
    i_s, f_s, v_s = ids[order], fetched[order], values[order]
    first = np.r_[True, i_s[1:] != i_s[:-1]]
    assert (f_s[first] == init).all()
    cont = ~first
    assert np.array_equal(f_s[cont], (f_s + v_s)[:-1][cont[1:]])


@pytest.mark.parametrize("dist", ["uniform", "zipf"])
def test_int64_fetch_add_histogram(rt, L, orc, dist):
    """The AMO workload at reduced count: fetch_add onto 4096 counters spread
    over 8 PEs, addresses uniform or Zipf(1.1); final histogram exact, fetched
    values a valid serialisation."""
    l = rt.up(P, HEAP)
    K, n = 4096, 1 << 20
    if dist == "uniform":
        ids = (orc.fill_u64(n, 0, 1) % K).astype(np.uint32)
    else:
        ids = orc.fill_zipf_u32(n, 0, 2, K, 1.1)
    vals = (orc.fill_u64(n, 0, 3) % 7 + 1).astype(np.int64)
    ctr = Counters(rt, l, K // P, np.int64)
    fetched = run_amo(rt, l, L, L.AMO_FETCH_ADD, "LONG", ctr, ids, values=vals)
    want, _ = orc.amo_i64(0, np.zeros(K, np.int64), ids, values=vals, want_fetched=False)
    assert np.array_equal(ctr.read_all(), want)
    check_fetch_chain(ids, fetched, vals, 0)
    # +1 form without a value array
    ctr.set_all(np.zeros(K, np.int64))
    fetched = run_amo(rt, l, L, L.AMO_FETCH_ADD, "LONG", ctr, ids)
    assert np.array_equal(ctr.read_all(), np.bincount(ids, minlength=K))
    check_fetch_chain(ids, fetched, np.ones(n, np.int64), 0)
    ctr.free()


@pytest.mark.parametrize("dtype_name", ["INT", "UINT", "LONG", "ULONGLONG"])
@pytest.mark.parametrize("K,n,wg", [(8, 64 * 257, 256), (3, 1000, 64), (64, 64 * 64 + 17, 192)])
def test_fetch_add_lanes_that_share_a_word_are_merged_correctly(rt, L, orc, dtype_name, K, n, wg):
    """Few counters, so most lanes of a wavefront share their word with many
    others: the merged add must hand every lane base + the sum of its group's
    lower lanes whether that sum comes from the lane count (equal addends), the
    DPP prefix sum (large groups in full wavefronts) or the walk (small groups,
    partly filled wavefronts: n is not a multiple of 64).  Final counters exact,
    fetched values a valid serialisation, for 32- and 64-bit types."""
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    ids = (orc.fill_u64(n, 7, K) % K).astype(np.uint32) * (P * 16 // K)  # spread over the PEs
    ctr = Counters(rt, l, 16, np_t)
    for vals in ((orc.fill_u64(n, 8, 1) % 5 + 1).astype(np_t), np.full(n, 3, np_t)):
        ctr.set_all(np.zeros(P * 16, np_t))
        fetched = run_amo(rt, l, L, L.AMO_FETCH_ADD, dtype_name, ctr, ids, values=vals, n_wgs=7, wg=wg)
        want = np.zeros(P * 16, np.int64)
        np.add.at(want, ids, vals.astype(np.int64))
        assert np.array_equal(ctr.read_all().astype(np.int64), want)
        check_fetch_chain(ids, fetched.astype(np.int64), vals.astype(np.int64), 0)
        # the non-fetching form lands the same totals
        ctr.set_all(np.zeros(P * 16, np_t))
        run_amo(rt, l, L, L.AMO_ADD, dtype_name, ctr, ids, values=vals, fetch=False, n_wgs=7, wg=wg)
        assert np.array_equal(ctr.read_all().astype(np.int64), want)
    ctr.free()


@pytest.mark.parametrize("dtype_name", ["INT", "LONG", "LONGLONG", "UINT", "ULONG", "ULONGLONG"])
def test_standard_amos_known_answers(rt, L, orc, dtype_name):
    """tests/functional_tests/amo_standard_tester.cpp:77-117,131-160: m calls on
    one remote counter: fetch_add(2) -> final 2m, largest fetched 2(m-1);
    fetch_inc -> m, m-1; add(2) -> 2m; inc -> m."""
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    m = 4096
    slot = 5 * 16 + 3  # PE 5, element 3
    ids = np.full(m, slot, np.uint32)
    ctr = Counters(rt, l, 16, np_t)
    f = run_amo(rt, l, L, L.AMO_FETCH_ADD, dtype_name, ctr, ids, values=np.full(m, 2))
    assert ctr.read_all()[slot] == 2 * m and f.max() == 2 * (m - 1)
    assert np.array_equal(np.sort(f), np.arange(0, 2 * m, 2, dtype=np_t))
    ctr.set_all(np.zeros(P * 16, np_t))
    f = run_amo(rt, l, L, L.AMO_FETCH_INC, dtype_name, ctr, ids)
    assert ctr.read_all()[slot] == m and f.max() == m - 1
    ctr.set_all(np.zeros(P * 16, np_t))
    run_amo(rt, l, L, L.AMO_ADD, dtype_name, ctr, ids, values=np.full(m, 2), fetch=False)
    assert ctr.read_all()[slot] == 2 * m
    ctr.set_all(np.zeros(P * 16, np_t))
    run_amo(rt, l, L, L.AMO_INC, dtype_name, ctr, ids, fetch=False)
    got = ctr.read_all()
    assert got[slot] == m and got.sum() == m  # nothing else touched
    ctr.free()


def test_compare_swap_hands_over_exactly_once(rt, L, orc):
    """Every thread tries cswap(k -> k+1) for its own k; exactly the chain
    0->1->...->m succeeds step by step when retried, and a single sweep leaves a
    value v such that fetched == cond holds for exactly v operations."""
    l = rt.up(P, HEAP)
    m = 2048
    ids = np.full(m, 2 * 4 + 1, np.uint32)
    ctr = Counters(rt, l, 4, np.int64)
    conds = np.arange(m, dtype=np.int64)
    f = run_amo(rt, l, L, L.AMO_COMPARE_SWAP, "LONG", ctr, ids, values=conds + 1, conds=conds)
    final = int(ctr.read_all()[2 * 4 + 1])
    assert final == int((f == conds).sum()) and final >= 1
    # serial: one thread, program order -> the oracle's serialisation exactly
    ctr.set_all(np.zeros(P * 4, np.int64))
    f = run_amo(rt, l, L, L.AMO_COMPARE_SWAP, "LONG", ctr, ids, values=conds + 1, conds=conds,
                n_wgs=1, wg=1)
    want_c, want_f = orc.amo_i64(4, np.zeros(P * 4, np.int64), ids, values=conds + 1, conds=conds)
    assert np.array_equal(ctr.read_all(), want_c) and np.array_equal(f, want_f)
    ctr.free()


@pytest.mark.parametrize("dtype_name", ["INT", "LONG", "UINT", "ULONG", "FLOAT", "DOUBLE"])
def test_extended_amos(rt, L, orc, dtype_name):
    """amo_extended_tester.cpp:77-110: set -> 44, fetch of a zero word -> 0;
    swap returns the old value.  Includes float/double."""
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    ctr = Counters(rt, l, 8, np_t)
    ids = np.array([3 * 8 + 2], np.uint32)
    assert run_amo(rt, l, L, L.AMO_FETCH, dtype_name, ctr, ids, n_wgs=1, wg=1)[0] == 0
    run_amo(rt, l, L, L.AMO_SET, dtype_name, ctr, ids, values=[44], fetch=False, n_wgs=1, wg=1)
    assert ctr.read_all()[3 * 8 + 2] == 44
    assert run_amo(rt, l, L, L.AMO_FETCH, dtype_name, ctr, ids, n_wgs=1, wg=1, my_pe=6)[0] == 44
    old = run_amo(rt, l, L, L.AMO_SWAP, dtype_name, ctr, ids, values=[7], n_wgs=1, wg=1)
    assert old[0] == 44 and ctr.read_all()[3 * 8 + 2] == 7
    # many swaps of distinct values: the fetched multiset plus the survivor is
    # the initial value plus all values written
    m = 1000
    vals = np.arange(100, 100 + m).astype(np_t)
    f = run_amo(rt, l, L, L.AMO_SWAP, dtype_name, ctr, np.full(m, 3 * 8 + 2, np.uint32), values=vals)
    survivor = ctr.read_all()[3 * 8 + 2]
    assert sorted(np.r_[f, survivor].tolist()) == sorted(np.r_[vals, np_t(7)].tolist())
    ctr.free()


@pytest.mark.parametrize("dtype_name", ["UINT", "ULONG", "ULONGLONG"])
def test_bitwise_amos(rt, L, orc, dtype_name):
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    bits = np.dtype(np_t).itemsize * 8
    ctr = Counters(rt, l, 4, np_t)
    slot = 7 * 4
    ids = np.full(bits, slot, np.uint32)
    one_hot = (np_t(1) << np.arange(bits).astype(np_t)).astype(np_t)
    f = run_amo(rt, l, L, L.AMO_FETCH_OR, dtype_name, ctr, ids, values=one_hot)
    assert ctr.read_all()[slot] == np_t(~np_t(0))
    assert len(set(f.tolist())) == bits  # each op saw a different partial mask
    f = run_amo(rt, l, L, L.AMO_FETCH_XOR, dtype_name, ctr, ids, values=one_hot)
    assert ctr.read_all()[slot] == 0
    ctr.set_all(np.full(P * 4, ~np_t(0), np_t))
    run_amo(rt, l, L, L.AMO_FETCH_AND, dtype_name, ctr, ids[:8], values=(~one_hot[:8]).astype(np_t))
    assert ctr.read_all()[slot] == np_t(~np_t(0)) & ~np_t(0xFF)
    # int types have no bitwise AMOs, float no arithmetic ones
    assert l.amo(L.AMO_FETCH_AND, L.INT, ctr.ptr, 4, 1, None, None, None, 0, 0, 1, 64, None) == -1
    assert l.amo(L.AMO_FETCH_ADD, L.FLOAT, ctr.ptr, 4, 1, None, None, None, 0, 0, 1, 64, None) == -1
    ctr.free()


# ------------------------------------------------------------------ signals
@pytest.mark.parametrize("gran,n_wgs,wg", [("THREAD", 2, 64), ("WAVE", 2, 256), ("WG", 4, 256)])
@pytest.mark.parametrize("sig_op", ["SET", "ADD"])
def test_put_signal_counts(rt, L, orc, gran, n_wgs, wg, sig_op):
    """tests/functional_tests/signaling_operations_tester.cpp:171-231: SET ->
    sig == signal; ADD -> init + calls * signal, calls counted per thread /
    wavefront / work-group.  The payload arrives intact."""
    l = rt.up(P, HEAP)
    groups = {"THREAD": n_wgs * wg, "WAVE": n_wgs * (wg // 64), "WG": n_wgs}[gran]
    n = groups * 48
    buf_s, buf_d, sig = l.malloc(n), l.malloc(n), l.malloc(8)
    host = orc.fill_u8(n, 1, 2)
    rt.put_bytes(l.pe_ptr(buf_s, 1), host)
    l.fill(l.pe_ptr(buf_d, 4), 0, n)
    rt.put_bytes(l.pe_ptr(sig, 4), np.array([1000], np.uint64))
    calls, signal = 3, 5
    rc = l.put_signal(getattr(L, gran), l.pe_ptr(buf_d, 1), l.pe_ptr(buf_s, 1), n, l.pe_ptr(sig, 1),
                      signal, getattr(L, "SIGNAL_" + sig_op), 1, 4, n_wgs, wg, calls, None)
    assert rc == 0
    l.stream_sync(None)
    assert np.array_equal(rt.get_bytes(l.pe_ptr(buf_d, 4), n), host)
    got = int(rt.get_bytes(l.pe_ptr(sig, 4), 8, np.uint64)[0])
    want = np.array([1000], np.uint64)  # the oracle's model applied once per call
    one = np.zeros(1, np.uint8)
    for _ in range(calls * groups):
        orc.lib.orc_put_signal(one.ctypes.data, one.ctypes.data, 1, want.ctypes.data, signal,
                               0 if sig_op == "SET" else 1)
    assert got == int(want[0])
    assert got == (signal if sig_op == "SET" else 1000 + calls * groups * signal)
    for b in (buf_s, buf_d, sig):
        l.free(b)


def test_put_signal_edge_cases(rt, L, orc):
    l = rt.up(P, HEAP)
    buf, sig = l.malloc(4096), l.malloc(8)
    rt.put_bytes(l.pe_ptr(sig, 2), np.array([9], np.uint64))
    # zero length: no signal update at all (src/context_device.cpp:251-262)
    assert l.put_signal(L.WG, buf, buf, 0, sig, 5, L.SIGNAL_ADD, 0, 2, 1, 64, 4, None) == 0
    l.stream_sync(None)
    assert int(rt.get_bytes(l.pe_ptr(sig, 2), 8, np.uint64)[0]) == 9
    # unknown signal op: payload only
    rt.put_bytes(buf, np.arange(256, dtype=np.uint8))
    l.fill(l.pe_ptr(buf, 2), 0, 256)
    assert l.put_signal(L.WG, buf, buf, 256, sig, 5, 7, 0, 2, 1, 64, 1, None) == 0
    l.stream_sync(None)
    assert int(rt.get_bytes(l.pe_ptr(sig, 2), 8, np.uint64)[0]) == 9
    assert np.array_equal(rt.get_bytes(l.pe_ptr(buf, 2), 256), np.arange(256, dtype=np.uint8))
    # groups beyond the end of the message send nothing and signal nothing
    rt.put_bytes(l.pe_ptr(sig, 2), np.array([0], np.uint64))
    assert l.put_signal(L.WG, buf, buf, 32, sig, 1, L.SIGNAL_ADD, 0, 2, 8, 64, 1, None) == 0
    l.stream_sync(None)
    assert int(rt.get_bytes(l.pe_ptr(sig, 2), 8, np.uint64)[0]) == 2  # 32 bytes = two 16-byte tiles
    l.free(buf)
    l.free(sig)


@pytest.mark.parametrize("gran", ["THREAD", "WAVE", "WG"])
def test_signal_fetch(rt, L, gran):
    """signaling_operations_tester: signal_fetch returns the local word (myid+123)."""
    l = rt.up(P, HEAP)
    sig = l.malloc(8)
    for p in range(P):
        rt.put_bytes(l.pe_ptr(sig, p), np.array([p + 123], np.uint64))
    for p in (0, 3, 7):
        out = ctypes.c_uint64()
        assert l.signal_fetch(getattr(L, gran), l.pe_ptr(sig, p), p, ctypes.byref(out)) == 0
        assert out.value == p + 123
    l.free(sig)


@pytest.mark.parametrize("pairs", [1, 8, 32])
@pytest.mark.parametrize("nbytes", [8, 64, 1024, 65536])
def test_pingpong(rt, L, orc, nbytes, pairs):
    """ping_pong_tester.cpp:43-61, run with 1, 8 and 32 work-groups as
    scripts/functional_tests/driver.sh:313-315 does: after `iters` round trips
    both signal words of every pair hold `iters` and both buffers hold the
    payload that bounced."""
    l = rt.up(P, HEAP)
    slot = (nbytes + 255) // 256 * 256
    buf, sig = l.malloc(slot * pairs), l.malloc(8 * pairs)
    host = orc.fill_u8(slot * pairs, 2, 3)
    rt.put_bytes(l.pe_ptr(buf, 2), host)
    l.fill(l.pe_ptr(buf, 6), 0, slot * pairs)
    for p in (2, 6):
        l.fill(l.pe_ptr(sig, p), 0, 8 * pairs)
    ticks, hz = ctypes.c_uint64(), ctypes.c_double()
    iters = 300
    assert l.pingpong(l.pe_ptr(buf, 2), l.pe_ptr(sig, 2), nbytes, iters, pairs, 2, 6, 256,
                      ctypes.byref(ticks), ctypes.byref(hz), None) == 0
    want = host.copy().reshape(pairs, slot)
    want_b = np.zeros_like(want)
    want_b[:, :nbytes] = want[:, :nbytes]  # only the payload crosses; slot padding stays
    for p, w in ((2, want), (6, want_b)):
        assert (rt.get_bytes(l.pe_ptr(sig, p), 8 * pairs, np.uint64) == iters).all()
        assert np.array_equal(rt.get_bytes(l.pe_ptr(buf, p), slot * pairs).reshape(pairs, slot), w)
    assert ticks.value > 0 and hz.value > 1e6
    assert l.pingpong(l.pe_ptr(buf, 2), l.pe_ptr(sig, 2), nbytes, 1, 129, 2, 6, 256, None, None, None) == -1
    l.free(buf)
    l.free(sig)


def zipf_routing(orc, P, tokens, experts, topk, seed):
    """Per source PE: for every token draw topk distinct experts from
    Zipf(1.1) (redraw duplicates); expert e lives on PE e // (experts / P)."""
    per_pe = experts // P
    counts = np.zeros((P, P), np.uint32)
    dest_of = []
    for s in range(P):
        draws = orc.fill_zipf_u32(tokens * topk * 4, seed, 50 + s, experts, 1.1).reshape(tokens, -1)
        chosen = np.zeros((tokens, topk), np.int64)
        for t in range(tokens):
            seen = []
            for e in draws[t]:
                if e not in seen:
                    seen.append(int(e))
                    if len(seen) == topk:
                        break
            k = 0
            while len(seen) < topk:  # deterministic completion if the draws ran out
                if k not in seen:
                    seen.append(k)
                k += 1
            chosen[t] = seen
        d = (chosen // per_pe).ravel()
        dest_of.append(d)
        counts[s] = np.bincount(d, minlength=P)
    return counts, dest_of


@pytest.mark.parametrize("rows_per_call", [1, 7, 64, 100000])
def test_dispatch_put_signal(rt, L, orc, rows_per_call):
    """MoE-dispatch pattern at reduced size: per-pair row counts from top-8 of
    256 Zipf(1.1) routing; rows packed per destination; receivers wait on the
    per-source signal.  Rows byte-exact, signals equal the counts."""
    l = rt.up(P, HEAP)
    tokens, row = 256, 1024
    counts, dest_of = zipf_routing(orc, P, tokens, 256, 8, 0)
    send_row = np.zeros((P, P), np.uint32)
    recv_row = np.zeros((P, P), np.uint32)
    for s in range(P):
        send_row[s] = np.r_[0, np.cumsum(counts[s])[:-1]]
    for d in range(P):
        recv_row[:, d] = np.r_[0, np.cumsum(counts[:, d])[:-1]]
    max_rows = int(max(counts.sum(1).max(), counts.sum(0).max()))
    send, recv, sig = l.malloc(max_rows * row), l.malloc(max_rows * row), l.malloc(8 * P)
    packed = []
    for s in range(P):
        rows = orc.fill_u8(int(counts[s].sum()) * row, 3, s)  # rows already grouped by destination
        packed.append(rows)
        rt.put_bytes(l.pe_ptr(send, s), rows)
        l.fill(l.pe_ptr(recv, s), 0, max_rows * row)
        l.fill(l.pe_ptr(sig, s), 0xFF, 8 * P)
    assert l.fill_every_pe(sig, 0, 8 * P, None) == 0
    counts, send_row, recv_row = (np.ascontiguousarray(a, np.uint32) for a in (counts, send_row, recv_row))
    assert l.dispatch_put_signal(recv, send, sig, counts.ctypes.data, send_row.ctypes.data,
                                 recv_row.ctypes.data, row, rows_per_call, 256, None, None) == 0
    l.stream_sync(None)
    # ... and twice more with running totals instead of cleared signal words
    expect = l.dev_alloc(8 * P * P)
    l.fill(expect, 0, 8 * P * P)
    assert l.fill_every_pe(sig, 0, 8 * P, None) == 0
    rounds = 3 if rows_per_call != 1 else 1
    for _ in range(rounds):
        assert l.dispatch_put_signal(recv, send, sig, counts.ctypes.data, send_row.ctypes.data,
                                     recv_row.ctypes.data, row, rows_per_call, 256, expect, None) == 0
    l.stream_sync(None)
    totals = rt.get_bytes(expect, 8 * P * P, np.uint64).reshape(P, P)  # [d][s]
    assert np.array_equal(totals, rounds * counts.T.astype(np.uint64))
    l.dev_free(expect)
    for d in range(P):
        sigs = rt.get_bytes(l.pe_ptr(sig, d), 8 * P, np.uint64)
        assert np.array_equal(sigs, rounds * counts[:, d].astype(np.uint64))
        got = rt.get_bytes(l.pe_ptr(recv, d), max_rows * row)
        for s in range(P):
            c = int(counts[s, d])
            a = int(send_row[s, d]) * row
            b = int(recv_row[s, d]) * row
            assert np.array_equal(got[b:b + c * row], packed[s][a:a + c * row]), (s, d)
    for x in (send, recv, sig):
        l.free(x)


# -------------------------------------------------------------------- waits
def one_value(np_t, v):
    return np.array([v], np_t)


@pytest.mark.parametrize("dtype_name", ["SHORT", "INT", "LONG", "UINT", "ULONG", "FLOAT", "DOUBLE"])
def test_test_comparators(rt, L, orc, dtype_name):
    """Context::test truth table (src/context_tmpl_device.hpp:337-377),
    including an unknown comparator, which never holds."""
    l = rt.up(P, HEAP)
    np_t = NP[dtype_name]
    samples = {"SHORT": [-7, 0, 9], "INT": [-5, 0, 3], "LONG": [-2**40, 0, 2**40],
               "UINT": [0, 7, 2**32 - 1], "ULONG": [0, 2**63, 2**64 - 1],
               "FLOAT": [-1.5, 0.0, 2.25], "DOUBLE": [-1e300, 0.5, 3.0]}[dtype_name]
    iv = l.dev_alloc(8)
    for x in samples:
        rt.put_bytes(iv, one_value(np_t, x))
        for v in samples:
            for cmp in range(7):
                ret = ctypes.c_size_t()
                val = one_value(np_t, v)
                assert l.wait_test(L.TEST, getattr(L, dtype_name), iv, 1, None, cmp, val.ctypes.data,
                                   ctypes.byref(ret), None) == 0
                assert ret.value == orc.test_value(getattr(orc, dtype_name), cmp, x, v), \
                    (dtype_name, x, cmp, v)
    l.dev_free(iv)


def test_wait_until_any_all_some_on_settled_values(rt, L, orc):
    l = rt.up(P, HEAP)
    host = np.array([0, 5, 0, 5, 5, 1], np.int64)
    iv = rt.dev_array(host)
    val = one_value(np.int64, 5)
    cases = [None, [0, 1, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1] * 6, [0, 0, 0, 1, 0, 0]]
    for status in cases:
        st = np.array(status, np.int32) if status is not None else None
        stp = st.ctypes.data if st is not None else None
        ret = ctypes.c_size_t()
        want_any = orc.wait_until_any(orc.LONG, host, status, 0, 5)
        if want_any != orc.WOULD_BLOCK:
            assert l.wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 6, stp, L.CMP_EQ, val.ctypes.data,
                               ctypes.byref(ret), None) == 0
            assert ret.value == want_any, status
        want_n, want_idx = orc.wait_until_some(orc.LONG, host, status, 0, 5)
        if want_n != orc.WOULD_BLOCK:
            idx = np.zeros(6, np.uint64)
            assert l.wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 6, stp, L.CMP_EQ, val.ctypes.data,
                               ctypes.byref(ret), idx.ctypes.data) == 0
            assert ret.value == want_n and np.array_equal(idx[:want_n], want_idx[:want_n]), status
    # nelems == 0
    ret = ctypes.c_size_t(7)
    assert l.wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 0, None, 0, val.ctypes.data, ctypes.byref(ret), None) == 0
    assert ret.value == L.SIZE_MAX
    assert l.wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 0, None, 0, val.ctypes.data, ctypes.byref(ret), None) == 0
    assert ret.value == 0
    # wait_until_all over entries that all hold (>= 0), masked or not
    zero = one_value(np.int64, 0)
    assert l.wait_test(L.WAIT_UNTIL_ALL, L.LONG, iv, 6, None, L.CMP_GE, zero.ctypes.data,
                       ctypes.byref(ret), None) == 0
    assert l.wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_LE, val.ctypes.data,
                       ctypes.byref(ret), None) == 0
    l.dev_free(iv)


@pytest.mark.parametrize("fn", ["WAIT_UNTIL", "WAIT_UNTIL_ANY", "WAIT_UNTIL_ALL", "WAIT_UNTIL_SOME"])
def test_blocking_waits_are_released_by_a_later_store(rt, L, fn):
    """The waiter starts on a value that does not hold; another work-group
    stores the awaited value some time later."""
    l = rt.up(P, HEAP)
    host = np.array([5, 5, 0, 5], np.uint64)
    if fn in ("WAIT_UNTIL_ANY", "WAIT_UNTIL_SOME"):
        host[:] = 0
    iv = rt.dev_array(host)
    val, wake = one_value(np.uint64, 5), one_value(np.uint64, 5)
    ret = ctypes.c_size_t()
    idx = np.zeros(4, np.uint64)
    ivp, n = (iv + 16, 1) if fn == "WAIT_UNTIL" else (iv, 4)
    wi = 0 if fn == "WAIT_UNTIL" else 2
    assert l.wait_test_woken(getattr(L, fn), L.ULONG, ivp, n, None, L.CMP_EQ, val.ctypes.data, wi,
                             wake.ctypes.data, 200000, ctypes.byref(ret), idx.ctypes.data) == 0
    if fn == "WAIT_UNTIL_ANY":
        assert ret.value == 2
    if fn == "WAIT_UNTIL_SOME":
        assert ret.value == 1 and idx[0] == 2
    assert rt.get_bytes(iv, 32, np.uint64)[2] == 5
    l.dev_free(iv)


# ---------------------------------------------------------------- contexts
def test_ctx_create_reports_pe_and_team(rt, L):
    """rocshmem_wg_ctx_create binds the world team of the acting PE; a team
    context reports the team-relative PE and the team size
    (src/rocshmem_gpu.cpp:286-325,606-635)."""
    l = rt.up(P, HEAP)
    n_wgs, per = 16, 3
    st, pe, npes = (np.zeros(n_wgs * per, np.int32) for _ in range(3))
    for acting in (0, 5):
        l.set_pe(acting)
        assert l.ctx_cycle(None, n_wgs, 64, per, st.ctypes.data, pe.ctypes.data, npes.ctypes.data) == 0
        assert not st.any() and (pe == acting).all() and (npes == P).all()
    # PE taken from blockIdx.x
    l.set_pe_rule(1)
    assert l.ctx_cycle(None, n_wgs, 64, 1, st.ctypes.data, pe.ctypes.data, npes.ctypes.data) == 0
    assert np.array_equal(pe[:n_wgs], np.arange(n_wgs) % P)
    l.set_pe_rule(0)
    l.set_pe(3)
    team = ctypes.c_void_p()
    assert l.team_split_strided(l.team_world(), 1, 2, 4, ctypes.byref(team)) == 0  # PEs 1,3,5,7
    assert l.ctx_cycle(team, 4, 64, 2, st.ctypes.data, pe.ctypes.data, npes.ctypes.data) == 0
    assert not st[:8].any() and (pe[:8] == 1).all() and (npes[:8] == 4).all()
    l.team_destroy(team)
    l.set_pe(0)


def test_ctx_pool_exhaustion_and_reuse(rt, L, monkeypatch):
    """ROCSHMEM_MAX_NUM_CONTEXTS contexts per PE; one more -> -1; destroyed
    contexts are reusable (src/ipc/backend_ipc.cpp:123-140)."""
    monkeypatch.setenv("ROCSHMEM_MAX_NUM_CONTEXTS", "5")
    rt.down()
    l = rt.up(2, 8 << 20)
    st, pe, npes = (np.zeros(8, np.int32) for _ in range(3))
    for _ in range(3):  # repeated: everything is returned each time
        assert l.ctx_cycle(None, 1, 64, 8, st.ctypes.data, pe.ctypes.data, npes.ctypes.data) == 0
        assert st.tolist() == [0] * 5 + [-1] * 3
        assert pe.tolist() == [0] * 5 + [-2] * 3
    monkeypatch.delenv("ROCSHMEM_MAX_NUM_CONTEXTS")
    rt.down()


# ---------------------------------------------------------------- coalesce
@pytest.mark.parametrize("seed", range(12))
def test_wf_coalesce_matches_oracle(rt, L, orc, seed):
    l = rt.up(P, HEAP)
    rng = np.random.default_rng(seed)
    size = rng.choice([4, 8, 8, 8, 16], 64).astype(np.uint64)
    pe = rng.choice([0, 1, 1, 1], 64).astype(np.int32)
    src = np.zeros(64, np.uint64)
    dst = np.zeros(64, np.uint64)
    s, d = 0x10000, 0x80000
    for k in range(64):
        if rng.random() < 0.2:
            s += 64
        if rng.random() < 0.1:
            d += 128
        src[k], dst[k] = s, d
        s += int(size[k])
        d += int(size[k])
    mask = (1 << 64) - 1 if seed % 3 == 0 else int(rng.integers(1, 1 << 63, dtype=np.uint64)) | 1
    if seed == 1:  # the worked example of src/wf_coal_policy.cpp:41-53
        size[:] = 8
        pe[:] = 1
        src = 0x1000 + 8 * np.arange(64, dtype=np.uint64)
        dst = 0x9000 + 8 * np.arange(64, dtype=np.uint64)
        src[9] += 4096
        mask = (1 << 64) - 1
    sends = np.zeros(64, np.int32)
    out = np.zeros(64, np.uint64)
    assert l.wf_coalesce(pe.ctypes.data, src.ctypes.data, dst.ctypes.data, size.ctypes.data, mask,
                         sends.ctypes.data, out.ctypes.data) == 0
    wsends, wout = orc.wf_coalesce(pe, src, dst, size, mask)
    act = np.array([(mask >> k) & 1 for k in range(64)], bool)
    assert np.array_equal(sends[act], wsends[act])
    assert np.array_equal(out[act], wout[act])
    if seed == 1:
        assert sends.sum() == 3 and (out[0], out[9], out[10]) == (72, 8, 432)


@pytest.mark.parametrize("coalesce", [0, 1])
@pytest.mark.parametrize("seed", range(10))
def test_per_lane_puts_with_and_without_coalescing(rt, L, orc, seed, coalesce):
    """Every active lane of one wavefront makes its own rocshmem_putmem call
    (src/ipc/context_ipc_device.cpp:62-69): mixed runs, lone lanes, inactive
    lanes, several target PEs, sizes that are no multiple of anything, and —
    seeds 0 to 2 — one run across the whole wavefront, which the coalescing
    front end moves as a single message (src/wf_coal_policy.cpp:57-172).  With
    the front end off and on, the destination on every PE must be what the
    oracle's plain copies of the sending lanes give; where the oracle's
    coalescing finds exactly one sender, its merged size is the whole run."""
    l = rt.up(P, HEAP)
    rng = np.random.default_rng(100 + seed)
    span = 1 << 16
    src_sym, dst_sym = l.malloc(span), l.malloc(span)
    payload = orc.fill_u8(span, 9, seed)
    rt.put_bytes(l.pe_ptr(src_sym, 2), payload)
    for p in range(P):
        l.fill(l.pe_ptr(dst_sym, p), 0xEE, span)
    if seed < 3:
        unit = [8, 64, 12][seed]
        size = np.full(64, unit, np.uint64)
        pe = np.full(64, 5, np.int32)
        src = 40 + unit * np.arange(64, dtype=np.uint64)
        dst = 24 + unit * np.arange(64, dtype=np.uint64)
        mask = (1 << 64) - 1 if seed != 2 else ((1 << 64) - 1) & ~((1 << 7) - 1)  # lanes 7..63
    else:
        size = rng.choice([1, 3, 4, 8, 8, 8, 16, 100], 64).astype(np.uint64)
        pe = rng.choice([0, 5, 5, 5], 64).astype(np.int32)
        src = np.zeros(64, np.uint64)
        dst = np.zeros(64, np.uint64)
        so, do = 16, 48
        for k in range(64):
            if rng.random() < 0.2:
                so += 64
            if rng.random() < 0.1:
                do += 128
            src[k], dst[k] = so, do
            so += int(size[k])
            do += int(size[k])
        mask = int(rng.integers(1, 1 << 63, dtype=np.uint64)) | 1
    before = l.set_coalesce_puts(coalesce)
    rc = l.lane_puts(l.pe_ptr(dst_sym, 2), l.pe_ptr(src_sym, 2), pe.ctypes.data, src.ctypes.data,
                     dst.ctypes.data, size.ctypes.data, mask, 2, None)
    l.set_coalesce_puts(before)
    assert rc == 0
    want = {p: np.full(span, 0xEE, np.uint8) for p in range(P)}
    for k in range(64):
        if (mask >> k) & 1:
            n = int(size[k])
            piece = np.empty(n, np.uint8)
            orc.lib.orc_copy(piece.ctypes.data, payload[int(src[k]):int(src[k]) + n].ctypes.data, n)
            want[int(pe[k])][int(dst[k]):int(dst[k]) + n] = piece
    for p in range(P):
        assert np.array_equal(rt.get_bytes(l.pe_ptr(dst_sym, p), span), want[p]), (seed, coalesce, p)
    sends, merged = orc.wf_coalesce(pe, src, dst, size, mask)
    act = np.array([(mask >> k) & 1 for k in range(64)], bool)
    if seed < 3:
        assert sends[act].sum() == 1 and merged[act][0] == size[act].sum()
    l.free(src_sym)
    l.free(dst_sym)
