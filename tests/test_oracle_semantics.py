"""Pins the oracle's restatements of PE/team arithmetic, reductions, block
moves, coalescing, atomics, waits and bf16 against the reference's own test
vectors, closed forms and independent formulations (numpy / torch on CPU)."""
import itertools
import math

import numpy as np
import pytest


# ------------------------------------------------------------------ H2 teams
def test_pe_maps_closed_form(orc):
    l = orc.lib
    for start, stride, size in itertools.product(range(4), range(1, 5), range(1, 6)):
        members = [start + stride * k for k in range(size)]
        for k, w in enumerate(members):
            assert l.orc_pe_in_world(start, stride, k) == w
            assert l.orc_pe_in_team(start, stride, size, w) == k
        for w in range(0, start + stride * size + 3):
            expect = members.index(w) if w in members else -1
            assert l.orc_pe_in_team(start, stride, size, w) == expect


@pytest.mark.parametrize("npes", range(1, 13))
def test_team_translate_sos_vectors(orc, npes):
    """tests/sos_tests/shmem_team_translate.cpp:46-92: stride-2 and stride-3
    teams over the world; a PE translates between them iff it is in both."""
    l = orc.lib
    t2 = (0, 2, (npes - 1) // 2 + 1)
    t3 = (0, 3, (npes - 1) // 3 + 1)
    for me in range(npes):
        p2 = l.orc_pe_in_team(*t2, me)
        p3 = l.orc_pe_in_team(*t3, me)
        assert (p2 != -1) == (me % 2 == 0)
        assert (p3 != -1) == (me % 3 == 0)
        # translating "-1" is meaningless in the test; it only checks members
        if p3 != -1:
            t = l.orc_team_translate_pe(*t3, p3, *t2)
            assert (t != -1) == (me % 2 == 0)
            if t != -1:
                assert t == me // 2
        if p2 != -1:
            t = l.orc_team_translate_pe(*t2, p2, *t3)
            assert (t != -1) == (me % 3 == 0)
    assert l.orc_team_translate_pe(0, 1, 0, 0, 0, 1, npes) == -1  # invalid team


def test_split_strided_checks(orc):
    l = orc.lib
    out = np.zeros(3, np.int32)
    # src/rocshmem.cpp:243-256: bad arguments
    for args in [(-1, 1, 2), (8, 1, 1), (0, 0, 2), (0, 1, 0), (0, 1, 9)]:
        assert l.orc_split_strided(0, 1, 8, 8, *args, 0, out.ctypes.data) == -1
    assert l.orc_split_strided(0, 1, 8, 8, 1, 2, 3, 0, out.ctypes.data) == 0
    assert out.tolist() == [1, 2, 3]
    # a split of a strided parent composes strides and starts
    assert l.orc_split_strided(1, 2, 4, 8, 1, 2, 2, 0, out.ctypes.data) == 0
    assert out.tolist() == [3, 4, 2]
    # the reference lets a team end exactly one past the last PE; strict mode does not
    assert l.orc_split_strided(0, 1, 8, 8, 2, 3, 3, 0, out.ctypes.data) == 0  # ends at PE 8
    assert l.orc_split_strided(0, 1, 8, 8, 2, 3, 3, 1, out.ctypes.data) == -1
    assert l.orc_split_strided(0, 1, 8, 8, 3, 3, 3, 0, out.ctypes.data) == -1  # ends at PE 9


def test_address_translation(orc):
    bases = np.array([0x1000, 0x9000, 0x5000], np.uint64)
    for me, pe in itertools.product(range(3), range(3)):
        dest = int(bases[me]) + 0x123
        assert orc.lib.orc_translate(bases.ctypes.data, dest, me, pe) == int(bases[pe]) + 0x123


# -------------------------------------------------------------- R reductions
def test_allreduce_example_closed_form(orc):
    """examples/rocshmem_allreduce_test.cc:49-70: src[i] = pe + i%9."""
    for P in (2, 3, 8):
        n = 256
        srcs = [np.array([pe + i % 9 for i in range(n)], np.int32) for pe in range(P)]
        out = orc.to_all(orc.INT, orc.SUM, srcs)
        expect = np.array([P * (P - 1) // 2 + P * (i % 9) for i in range(n)], np.int32)
        assert np.array_equal(out, expect)


@pytest.mark.parametrize("P", [1, 2, 4, 7])
def test_sos_to_all_closed_forms(orc, P):
    """tests/sos_tests/to_all.cpp:118-153,208-250,305-346,402-428,466-546,
    626-657,696-724 and big_reduction.cpp:77,90-105."""
    n = 10
    for dt, np_t in ((orc.SHORT, np.int16), (orc.INT, np.int32), (orc.LONG, np.int64)):
        me = [np.full(n, p, np_t) for p in range(P)]
        mei = [np.arange(n, dtype=np_t) + p for p in range(P)]
        assert np.all(orc.to_all(dt, orc.SUM, me) == P * (P - 1) // 2)
        assert np.array_equal(orc.to_all(dt, orc.MAX, mei), np.arange(n, dtype=np_t) + P - 1)
        assert np.array_equal(orc.to_all(dt, orc.MIN, mei), np.arange(n, dtype=np_t))
        assert np.all(orc.to_all(dt, orc.AND, me) == (0 if P > 1 else 0))
        ors = [np.full(n, (p + 1) % 4, np_t) for p in range(P)]
        assert np.all(orc.to_all(dt, orc.OR, ors) == (1 if P == 1 else 3))
        xors = [np.full(n, p % 2, np_t) for p in range(P)]
        assert np.all(orc.to_all(dt, orc.XOR, xors) == (P // 2) % 2)
        prod = [np.full(n, p + 1, np_t) for p in range(P)]
        assert np.all(orc.to_all(dt, orc.PROD, prod) == math.factorial(P))
    for dt, np_t in ((orc.FLOAT, np.float32), (orc.DOUBLE, np.float64)):
        me = [np.full(n, p, np_t) for p in range(P)]
        assert np.all(orc.to_all(dt, orc.SUM, me) == P * (P - 1) // 2)
        assert np.all(orc.to_all(dt, orc.PROD, [m + 1 for m in me]) == math.factorial(P))
    # tests/functional_tests/tester.cpp:147-159: all ones -> P
    assert np.all(orc.to_all(orc.FLOAT, orc.SUM, [np.ones(n, np.float32)] * P) == P)


@pytest.mark.parametrize("dt,np_t", [(0, np.int16), (1, np.int32), (2, np.int64)])
def test_integer_ops_match_numpy_with_wraparound(orc, dt, np_t):
    rng = np.random.default_rng(dt)
    info = np.iinfo(np_t)
    P, n = 5, 1000
    srcs = [rng.integers(info.min, info.max, n, dtype=np_t, endpoint=True) for _ in range(P)]
    stack = np.stack(srcs)
    with np.errstate(over="ignore"):
        expect = {
            orc.SUM: np.add.reduce(stack, axis=0, dtype=np_t),
            orc.PROD: np.multiply.reduce(stack, axis=0, dtype=np_t),
            orc.MAX: stack.max(0), orc.MIN: stack.min(0),
            orc.AND: np.bitwise_and.reduce(stack, axis=0),
            orc.OR: np.bitwise_or.reduce(stack, axis=0),
            orc.XOR: np.bitwise_xor.reduce(stack, axis=0),
        }
    for op, e in expect.items():
        assert np.array_equal(orc.to_all(dt, op, srcs), e), op


def test_float_sum_is_the_ascending_left_fold(orc):
    """Brute force in numpy float32 scalar arithmetic, and a case where the
    order matters so that a wrong order fails."""
    rng = np.random.default_rng(3)
    P, n = 8, 2000
    srcs = [rng.standard_normal(n).astype(np.float32) * np.float32(10.0 ** rng.integers(-3, 4))
            for _ in range(P)]
    acc = srcs[0].copy()
    for p in range(1, P):
        acc = (acc + srcs[p]).astype(np.float32)
    out = orc.to_all(orc.FLOAT, orc.SUM, srcs)
    assert np.array_equal(out.view(np.uint32), acc.view(np.uint32))
    # order-sensitive triple: (1e8 + -1e8) + 1 = 1 but 1e8 + (-1e8 + 1) = 0
    t = [np.array([1e8], np.float32), np.array([-1e8], np.float32), np.array([1.0], np.float32)]
    assert orc.to_all(orc.FLOAT, orc.SUM, t)[0] == 1.0
    assert orc.to_all(orc.FLOAT, orc.SUM, t[::-1])[0] == 0.0
    # max / min are order independent
    assert np.array_equal(orc.to_all(orc.FLOAT, orc.MAX, srcs), np.stack(srcs).max(0))
    assert np.array_equal(orc.to_all(orc.DOUBLE, orc.MIN, [s.astype(np.float64) for s in srcs]),
                          np.stack(srcs).astype(np.float64).min(0))


def test_multiple_destinations_and_threads_agree(orc):
    rng = np.random.default_rng(4)
    srcs = [rng.standard_normal(10007).astype(np.float32) for _ in range(4)]
    one = orc.to_all(orc.FLOAT, orc.SUM, srcs)
    many = orc.to_all(orc.FLOAT, orc.SUM, srcs, ndst=4, nthreads=5)
    for d in many:
        assert np.array_equal(d.view(np.uint32), one.view(np.uint32))


def test_reduce_plan_thresholds(orc):
    """src/ipc/context_ipc_tmpl_device.hpp:361-418."""
    # direct iff max(n/2+1, 1024) >= P*n
    for P in (2, 4, 8):
        edge = 1024 // P
        assert orc.reduce_plan(P, edge)["algo"] == 0
        assert orc.reduce_plan(P, edge + 1)["algo"] == 1
    # the two benchmark configurations: 1 Mi ints on 2 PEs, 64 Mi on 8 PEs
    p = orc.reduce_plan(2, 1 << 20)
    assert (p["algo"], p["chunk_size"], p["seg_size"], p["n_seg"]) == (1, 512, 1024, 1024)
    p = orc.reduce_plan(8, 1 << 26)
    assert (p["algo"], p["chunk_size"], p["n_seg"]) == (1, 128, 65536)
    # remainder ring + direct tail
    p = orc.reduce_plan(8, 1024 * 3 + 8 * 5 + 3)
    assert (p["n_seg"], p["has_remainder_ring"], p["p_count"], p["p_chunk"],
            p["tail_direct_count"]) == (3, 1, 43, 5, 3)
    # 2P > 256 -> ROCSHMEM_ERROR (only reachable when the direct test fails)
    assert orc.reduce_plan(129, 100)["status"] == 1
    assert orc.reduce_plan(128, 100)["status"] == 0


@pytest.mark.parametrize("P,n", [(2, 1500), (4, 300), (8, 5000), (8, 100), (3, 1024 + 7)])
def test_reference_order_differs_by_rounding_only(orc, P, n):
    """The ascending order (this build) vs the reference's direct/ring orders:
    equal for integer-valued data, within (P-1) ulp-scale roundings otherwise."""
    rng = np.random.default_rng(P * 1000 + n)
    ints = [rng.integers(-1000, 1001, n).astype(np.float32) for _ in range(P)]
    asc = orc.to_all(orc.FLOAT, orc.SUM, ints)
    for pe in range(P):
        ref = orc.reduce_f32_sum_reference_order(ints, pe)
        assert np.array_equal(ref, asc)
    srcs = [rng.standard_normal(n).astype(np.float32) for _ in range(P)]
    asc = orc.to_all(orc.FLOAT, orc.SUM, srcs)
    exact = np.sum(np.stack(srcs).astype(np.float64), axis=0)
    bound = (P - 1) * np.spacing(np.abs(np.stack(srcs)).sum(0).astype(np.float32))
    for pe in range(P):
        ref = orc.reduce_f32_sum_reference_order(srcs, pe)
        assert np.all(np.abs(ref.astype(np.float64) - asc.astype(np.float64)) <= bound)
        assert np.all(np.abs(ref.astype(np.float64) - exact) <= bound)


# ------------------------------------------------------------------- bf16
def test_bf16_conversions_against_torch(orc):
    torch = pytest.importorskip("torch")
    # every bf16 bit pattern widens exactly
    allb = np.arange(65536, dtype=np.uint16)
    mine = orc.bf16_to_f32(allb)
    theirs = torch.from_numpy(allb.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(mine.view(np.uint32), theirs.view(np.uint32))
    # round to nearest even on random bit patterns, ties, boundaries
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 1 << 32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 1 << 16, 4096, dtype=np.uint32) << 16) | np.uint32(0x8000)
    near = np.concatenate([ties, ties + 1, ties - 1, np.array([0x7F7FFFFF, 0x7F800000, 0xFF800000,
                           0x00000001, 0x80000000, 0x3F800000, 0x7F7F8000], np.uint32)])
    x = np.concatenate([bits, near]).view(np.float32)
    finite = ~np.isnan(x)
    got = orc.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[finite], want[finite])
    assert np.all((got[~finite] & 0x7FC0) == 0x7FC0)  # NaN stays a quiet NaN


def test_bf16_sum_definition(orc):
    rng = np.random.default_rng(1)
    P, n = 8, 4096
    srcs = [orc.f32_to_bf16(rng.standard_normal(n).astype(np.float32)) for _ in range(P)]
    acc = orc.bf16_to_f32(srcs[0])
    for p in range(1, P):
        acc = (acc + orc.bf16_to_f32(srcs[p])).astype(np.float32)
    assert np.array_equal(orc.to_all(orc.BF16, orc.SUM, srcs), orc.f32_to_bf16(acc))


# --------------------------------------------------------- A2A / FC / BC
def test_alltoall_example_vectors(orc):
    """examples/rocshmem_alltoall_test.cc:49-75: src_me[pe*n+i] = me + pe and
    the received block from pe must also read me + pe."""
    P, n = 4, 16
    srcs = [np.array([me + pe for pe in range(P) for _ in range(n)], np.int32) for me in range(P)]
    dsts = orc.alltoall(srcs, n * 4)
    for me in range(P):
        got = dsts[me].view(np.int32)
        assert np.array_equal(got, srcs[me])  # symmetric pattern: dst equals own src
    # asymmetric data: the index identity dst_j[i*n+k] = src_i[j*n+k]
    rng = np.random.default_rng(2)
    srcs = [rng.integers(0, 256, P * 40, dtype=np.uint8) for _ in range(P)]
    dsts = orc.alltoall(srcs, 40, nthreads=3)
    for i, j, k in itertools.product(range(P), range(P), range(40)):
        assert dsts[j][i * 40 + k] == srcs[i][j * 40 + k]


def test_fcollect_and_broadcast(orc):
    P, n = 5, 24
    rng = np.random.default_rng(3)
    srcs = [rng.integers(0, 256, n, dtype=np.uint8) for _ in range(P)]
    dsts = orc.fcollect(srcs, n)
    for j in range(P):
        assert np.array_equal(dsts[j], np.concatenate(srcs))
    # broadcast: non-roots get the root's source, the root's dest is untouched
    # (tests/functional_tests/team_broadcast_tester.cpp:210-243)
    for root in range(P):
        d = [np.full(n, 0xEE, np.uint8) for _ in range(P)]
        orc.broadcast(srcs, d, n, root)
        for j in range(P):
            assert np.array_equal(d[j], srcs[root] if j != root else np.full(n, 0xEE, np.uint8))


# ----------------------------------------------------------------- C1 copy
def test_reference_lane_loop_model_and_its_tail_defect(orc):
    """The lane model of src/util.hpp:188-262 copies every byte for even sizes
    and for size 1, and drops the last byte of odd sizes >= 3 (stale pointer in
    the one-byte tail).  The contract this build implements is the full copy."""
    rng = np.random.default_rng(5)
    for lanes in (1, 3, 64, 256):
        for n in list(range(0, 70)) + [255, 256, 257, 1000, 1001]:
            src = rng.integers(1, 256, n, dtype=np.uint8)
            dst = np.zeros(n + 2, np.uint8)
            if n:
                orc.lib.orc_ref_memcpy_lanes_model(dst.ctypes.data, src.ctypes.data, n, lanes)
            if n % 2 == 0 or n == 1:
                assert np.array_equal(dst[:n], src), (lanes, n)
            else:
                assert np.array_equal(dst[:n - 1], src[:n - 1]) and dst[n - 1] == 0, (lanes, n)
            assert dst[n] == 0 and dst[n + 1] == 0


# -------------------------------------------------------------- C4 coalesce
def _independent_coalesce(pe, src, dst, size, mask):
    """Run-length formulation: walk lanes upward, extending the current run
    while each next lane is active and continues its lower neighbour."""
    sends = np.full(64, -1, np.int32)
    out = np.zeros(64, np.uint64)
    l = 0
    while l < 64:
        if not (mask >> l) & 1:
            l += 1
            continue
        run = 0
        k = l + 1
        while (k < 64 and (mask >> k) & 1 and pe[k] == pe[k - 1] and
               (int(size[k - 1]) & 0xFFFFFFFF) == int(size[k]) and
               int(src[k - 1]) + int(size[k]) == int(src[k]) and
               int(dst[k - 1]) + int(size[k]) == int(dst[k])):
            run += 1
            k += 1
        sends[l] = 1
        out[l] = int(size[l]) * (1 + run)
        for a in range(l + 1, k):
            sends[a] = 0
            out[a] = size[a]
        l = k
    return sends, out


def test_coalesce_worked_example(orc):
    """src/wf_coal_policy.cpp:41-53: lanes 0-8 and 10-63 contiguous, lane 9 not
    -> three messages."""
    size = np.full(64, 8, np.uint64)
    src = 0x1000 + 8 * np.arange(64, dtype=np.uint64)
    dst = 0x9000 + 8 * np.arange(64, dtype=np.uint64)
    src[9] += 4096  # lane 9 breaks the run on both sides
    pe = np.ones(64, np.int32)
    sends, out = orc.wf_coalesce(pe, src, dst, size, (1 << 64) - 1)
    assert sends.sum() == 3 and list(np.nonzero(sends)[0]) == [0, 9, 10]
    assert (out[0], out[9], out[10]) == (72, 8, 54 * 8)


@pytest.mark.parametrize("seed", range(20))
def test_coalesce_brute_force(orc, seed):
    rng = np.random.default_rng(seed)
    size = rng.choice([4, 8, 8, 8, 16], 64).astype(np.uint64)
    src = np.zeros(64, np.uint64)
    dst = np.zeros(64, np.uint64)
    pe = rng.choice([0, 1, 1, 1], 64).astype(np.int32)
    s, d = 0x10000, 0x80000
    for l in range(64):
        if rng.random() < 0.2:
            s += int(rng.integers(1, 5)) * 64
        if rng.random() < 0.1:
            d += 128
        src[l], dst[l] = s, d
        s += int(size[l])
        d += int(size[l])
    mask = int(rng.integers(0, 1 << 63, dtype=np.uint64)) | (int(rng.integers(0, 2)) << 63)
    if seed % 4 == 0:
        mask = (1 << 64) - 1
    sends, out = orc.wf_coalesce(pe, src, dst, size, mask)
    esends, eout = _independent_coalesce(pe, src, dst, size, mask)
    act = np.array([(mask >> l) & 1 for l in range(64)], bool)
    assert np.array_equal(sends[act], esends[act])
    assert np.array_equal(out[act], eout[act])
    # every byte of every active lane is sent exactly once
    assert out[act & (sends == 1)].sum() == size[act].sum()


# -------------------------------------------------------------- A1 atomics
def test_amo_known_answers(orc):
    """tests/functional_tests/amo_standard_tester.cpp:77-117,131-160 and
    amo_extended_tester.cpp:77-110 with m operations on one counter."""
    m = 50
    ids = np.zeros(m, np.uint32)
    c, f = orc.amo_i64(0, [0], ids, values=np.full(m, 2))      # fetch_add(2) x m
    assert c[0] == 2 * m and f.max() == 2 * (m - 1) and sorted(f) == list(range(0, 2 * m, 2))
    c, f = orc.amo_i64(2, [0], ids)                            # fetch_inc x m
    assert c[0] == m and f.max() == m - 1
    assert orc.amo_i64(1, [0], ids, values=np.full(m, 2))[0][0] == 2 * m   # add
    assert orc.amo_i64(3, [0], ids)[0][0] == m                              # inc
    # compare_swap chain: op i swaps i -> i+1
    c, f = orc.amo_i64(4, [0], ids, values=np.arange(1, m + 1), conds=np.arange(m))
    assert c[0] == m and np.array_equal(f, np.arange(m))
    assert orc.amo_i64(6, [7], ids[:1], values=[44])[0][0] == 44             # set -> 44
    c, f = orc.amo_i64(5, [0], ids[:3])                                      # fetch -> 0
    assert c[0] == 0 and not f.any()
    c, f = orc.amo_i64(7, [5], ids[:2], values=[9, 11])                      # swap
    assert c[0] == 11 and list(f) == [5, 9]
    assert orc.amo_i64(8, [0b1100], ids[:1], values=[0b1010])[0][0] == 0b1000
    assert orc.amo_i64(9, [0b1100], ids[:1], values=[0b1010])[0][0] == 0b1110
    assert orc.amo_i64(10, [0b1100], ids[:1], values=[0b1010])[0][0] == 0b0110


def test_amo_histogram_invariant(orc):
    rng = np.random.default_rng(7)
    K, n = 64, 20000
    ids = rng.integers(0, K, n).astype(np.uint32)
    vals = rng.integers(1, 10, n)
    c, f = orc.amo_i64(0, np.zeros(K, np.int64), ids, values=vals)
    assert np.array_equal(c, np.bincount(ids, weights=vals, minlength=K).astype(np.int64))
    t0 = orc.lib.orc_amo_fetch_add_threaded  # threaded baseline gives the same totals
    counters = np.zeros(K, np.int64)
    fetched = np.zeros(n, np.int64)
    v = np.ascontiguousarray(vals, np.int64)
    t0(counters.ctypes.data, ids.ctypes.data, v.ctypes.data, fetched.ctypes.data, n, 4)
    assert np.array_equal(counters, c)
    for k in range(K):  # fetched values of a counter chain through its addends
        sel = np.nonzero(ids == k)[0]
        order = sel[np.argsort(fetched[sel])]
        assert fetched[order[0]] == 0
        assert np.array_equal(fetched[order[1:]], (fetched[order] + v[order])[:-1])


# ---------------------------------------------------------- S1 / W1 signals
def test_put_signal_model(orc):
    src = np.arange(16, dtype=np.uint8)
    dst = np.zeros(16, np.uint8)
    sig = np.array([5], np.uint64)
    orc.lib.orc_put_signal(dst.ctypes.data, src.ctypes.data, 16, sig.ctypes.data, 9, 0)
    assert sig[0] == 9 and np.array_equal(dst, src)
    orc.lib.orc_put_signal(dst.ctypes.data, src.ctypes.data, 16, sig.ctypes.data, 9, 1)
    assert sig[0] == 18
    orc.lib.orc_put_signal(dst.ctypes.data, src.ctypes.data, 0, sig.ctypes.data, 1, 1)
    assert sig[0] == 18  # zero length: nothing at all
    orc.lib.orc_put_signal(dst.ctypes.data, src.ctypes.data, 16, sig.ctypes.data, 1, 7)
    assert sig[0] == 18  # unknown op: payload only


def test_comparators_truth_table(orc):
    import operator
    ops = [operator.eq, operator.ne, operator.gt, operator.ge, operator.lt, operator.le]
    samples = {orc.INT: [-5, 0, 3, 2**31 - 1], orc.LONG: [-2**40, -1, 0, 2**40],
               orc.ULONG: [0, 1, 2**63, 2**64 - 1], orc.FLOAT: [-1.5, 0.0, 2.25, 1e30],
               orc.DOUBLE: [-1e300, 0.5, 3.0], orc.SHORT: [-32768, -1, 7, 32767],
               orc.UINT: [0, 7, 2**32 - 1]}
    for dt, vals in samples.items():
        for x, v in itertools.product(vals, vals):
            for cmp, op in enumerate(ops):
                assert orc.test_value(dt, cmp, x, v) == int(op(x, v)), (dt, cmp, x, v)
            assert orc.test_value(dt, 6, x, v) == 0  # unknown comparator never holds
            assert orc.test_value(dt, -1, x, v) == 0


def test_wait_until_any_some_models(orc):
    iv = [0, 5, 0, 5, 5]
    assert orc.wait_until_any(orc.INT, iv, None, 0, 5) == 1
    assert orc.wait_until_any(orc.INT, iv, [0, 1, 0, 0, 0], 0, 5) == 3
    assert orc.wait_until_any(orc.INT, [], None, 0, 5) == orc.SIZE_MAX
    assert orc.wait_until_any(orc.INT, iv, [1] * 5, 0, 5) == orc.SIZE_MAX
    assert orc.wait_until_any(orc.INT, iv, None, 0, 9) == orc.WOULD_BLOCK
    n, idx = orc.wait_until_some(orc.INT, iv, [0, 0, 0, 1, 0], 0, 5)
    assert n == 2 and list(idx[:2]) == [1, 4]
    assert orc.wait_until_some(orc.INT, [], None, 0, 5)[0] == 0
    assert orc.wait_until_some(orc.INT, iv, [1] * 5, 0, 5)[0] == 0
    # status entries before the first zero are skipped as a prefix; later
    # non-zero entries are skipped one by one (src/context_tmpl_device.hpp:208-218)
    assert orc.wait_until_any(orc.INT, [5, 5, 0, 5], [1, 1, 0, 0], 0, 5) == 3


# ------------------------------------------------------------------ inputs
def test_seeded_inputs_are_reproducible_and_in_range(orc):
    a = orc.fill_i32_pm1000(10000, 0, 1)
    assert a.min() >= -1000 and a.max() <= 1000 and np.array_equal(a, orc.fill_i32_pm1000(10000, 0, 1))
    assert not np.array_equal(a, orc.fill_i32_pm1000(10000, 0, 2))
    g = orc.fill_normal_f32(200000, 0, 0)
    assert np.isfinite(g).all() and abs(g.mean()) < 0.02 and abs(g.std() - 1) < 0.02
    assert not (g == 0).any()  # no +-0 so fp32 max is order independent
    z = orc.fill_zipf_u32(200000, 0, 0, 4096, 1.1)
    assert z.max() < 4096 and np.bincount(z)[0] > np.bincount(z)[1] > np.bincount(z)[10]
    u = orc.fill_u8(4096, 0, 3)
    assert len(np.unique(u)) == 256
