"""R1-R6, R-CPU: all-reduce through the device API (one work-group per PE) and
through the host-called whole-GPU form, bit-exact against the oracle's
ascending-PE fold.  Through the C entry points."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HEAP = 1 << 30
INT_OPS = ["SUM", "MAX", "MIN", "PROD", "AND", "OR", "XOR"]
FLT_OPS = ["SUM", "MAX", "MIN", "PROD"]
TYPES = {"SHORT": INT_OPS, "INT": INT_OPS, "LONG": INT_OPS, "LONGLONG": INT_OPS,
         "FLOAT": FLT_OPS, "DOUBLE": FLT_OPS, "BF16": ["SUM"]}


def make_inputs(orc, dtype_name, P, n, seed):
    rng = np.random.default_rng(seed)
    np_t = orc.NP_DTYPE[getattr(orc, dtype_name)]
    if dtype_name == "BF16":
        return [orc.f32_to_bf16(orc.fill_normal_f32(n, seed, p)) for p in range(P)]
    if dtype_name in ("FLOAT", "DOUBLE"):
        return [orc.fill_normal_f32(n, seed, p).astype(np_t) for p in range(P)]
    info = np.iinfo(np_t)
    return [rng.integers(info.min, info.max, n, dtype=np_t, endpoint=True) for _ in range(P)]


class Buffers:
    def __init__(self, rt, l, nbytes):
        self.rt, self.l = rt, l
        self.src = l.malloc(nbytes)
        self.dst = l.malloc(nbytes)
        assert self.src and self.dst

    def free(self):
        self.l.free(self.src)
        self.l.free(self.dst)


def check_all(rt, l, orc, L, P, dtype_name, op_name, n, mode, seed=0, off=0, wg=256, pes=None,
              team=None):
    """pes: world PEs taking part (default all); off: element offset into the
    buffers (exercises unaligned starts)."""
    pes = list(range(P)) if pes is None else pes
    dt, op = getattr(L, dtype_name), getattr(L, op_name)
    np_t = orc.NP_DTYPE[getattr(orc, dtype_name)]
    es = np.dtype(np_t).itemsize
    b = Buffers(rt, l, (n + off + 8) * es)
    srcs = make_inputs(orc, dtype_name, len(pes), n, seed)
    for p in range(P):
        l.fill(l.pe_ptr(b.dst, p), 0x5A, (n + off + 8) * es)
    for k, p in enumerate(pes):
        rt.put_bytes(l.pe_ptr(b.src, p) + off * es, srcs[k])
    me = l.my_pe()
    d = l.pe_ptr(b.dst, me) + off * es
    s = l.pe_ptr(b.src, me) + off * es
    if mode == "wg":
        rc = l.wg_reduce(dt, op, team if team else l.team_world(), d, s, n, wg, None)
    elif mode == "to_all":
        stride = pes[1] - pes[0] if len(pes) > 1 else 1
        log = int(np.log2(stride))
        rc = l.to_all(dt, op, l.pe_ptr(b.dst, pes[0]) + off * es, l.pe_ptr(b.src, pes[0]) + off * es,
                      n, pes[0], log, len(pes), None)
    else:
        rc = l.reduce(dt, op, team if team else l.team_world(), d, s, n, None)
    assert rc == 0, (dtype_name, op_name, n, mode)
    l.stream_sync(None)
    want = orc.to_all(getattr(orc, dtype_name), getattr(orc, op_name), srcs)
    for p in range(P):
        got = rt.get_bytes(l.pe_ptr(b.dst, p), (n + off + 8) * es, np_t)
        if p in pes:
            assert np.array_equal(got[off:off + n].view(np.uint8), want.view(np.uint8)), \
                (dtype_name, op_name, n, mode, p)
            rest = np.concatenate([got[:off], got[off + n:]]).view(np.uint8)
        else:
            rest = got.view(np.uint8)
        assert (rest == 0x5A).all(), (dtype_name, op_name, n, mode, p, "guard")
    b.free()


@pytest.mark.parametrize("mode", ["wg", "to_all"])
@pytest.mark.parametrize("dtype_name", list(TYPES))
def test_every_type_and_op(rt, L, orc, dtype_name, mode):
    l = rt.up(8, HEAP)
    for op_name in TYPES[dtype_name]:
        for n in (1, 37, 1000, 4099):
            check_all(rt, l, orc, L, 8, dtype_name, op_name, n, mode, seed=n)


@pytest.mark.parametrize("mode", ["wg", "to_all"])
@pytest.mark.parametrize("P", [1, 2, 3, 4, 5, 8])
def test_pe_counts_and_ragged_sizes(rt, L, orc, P, mode):
    l = rt.up(P, 64 << 20)
    for n in (1, 2, 3, 5, 7, 8, 9, 63, 64, 65, 127, 1025, 20001):
        check_all(rt, l, orc, L, P, "FLOAT", "SUM", n, mode, seed=n)
        check_all(rt, l, orc, L, P, "LONG", "XOR", n, mode, seed=n)
        check_all(rt, l, orc, L, P, "BF16", "SUM", n, mode, seed=n)
    rt.up(8, HEAP)


@pytest.mark.parametrize("mode", ["wg", "to_all"])
def test_unaligned_starts(rt, L, orc, mode):
    l = rt.up(8, HEAP)
    for off in (1, 2, 3, 5):
        for dtype_name in ("SHORT", "INT", "FLOAT", "LONG", "BF16"):
            check_all(rt, l, orc, L, 8, dtype_name, "SUM", 3001, mode, seed=off, off=off)


@pytest.mark.parametrize("wg", [1, 64, 100, 1024])
def test_work_group_sizes(rt, L, orc, wg):
    l = rt.up(8, HEAP)
    check_all(rt, l, orc, L, 8, "FLOAT", "SUM", 5003, "wg", wg=wg)
    check_all(rt, l, orc, L, 8, "INT", "MAX", 333, "wg", wg=wg)


def test_zero_elements_is_a_no_op(rt, L, orc):
    l = rt.up(8, HEAP)
    b = Buffers(rt, l, 256)
    l.fill(b.dst, 0x11, 256)
    assert l.wg_reduce(L.INT, L.SUM, l.team_world(), b.dst, b.src, 0, 64, None) == 0
    assert l.to_all(L.INT, L.SUM, b.dst, b.src, 0, 0, 0, 8, None) == 0
    l.stream_sync(None)
    assert (rt.get_bytes(b.dst, 256) == 0x11).all()
    b.free()


def test_in_place(rt, L, orc):
    """dest == source is allowed on the host path (src/host/host_templates.hpp:353)."""
    l = rt.up(8, HEAP)
    n = 70001
    srcs = make_inputs(orc, "FLOAT", 8, n, 9)
    want = orc.to_all(orc.FLOAT, orc.SUM, srcs)
    for mode in ("to_all", "wg"):
        buf = l.malloc(n * 4)
        for p in range(8):
            rt.put_bytes(l.pe_ptr(buf, p), srcs[p])
        if mode == "to_all":
            assert l.to_all(L.FLOAT, L.SUM, buf, buf, n, 0, 0, 8, None) == 0
        else:
            assert l.wg_reduce(L.FLOAT, L.SUM, l.team_world(), buf, buf, n, 256, None) == 0
        l.stream_sync(None)
        for p in range(8):
            got = rt.get_bytes(l.pe_ptr(buf, p), n * 4, np.float32)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (mode, p)
        l.free(buf)


def test_active_sets_and_teams(rt, L, orc):
    l = rt.up(8, HEAP)
    import ctypes
    # host to_all over (PE_start, logPE_stride, PE_size)
    for pes in ([0, 2, 4, 6], [1, 3, 5, 7], [2, 3, 4], [4], [0, 4]):
        check_all(rt, l, orc, L, 8, "INT", "SUM", 2049, "to_all", seed=len(pes), pes=pes)
    # strided team through the device API and the host team form
    for start, stride, size in [(0, 2, 4), (1, 3, 2), (2, 1, 5)]:
        team = ctypes.c_void_p()
        pes = [start + stride * k for k in range(size)]
        l.set_pe(pes[0])
        assert l.team_split_strided(l.team_world(), start, stride, size, ctypes.byref(team)) == 0
        assert team.value and l.team_n_pes(team) == size
        for mode in ("wg", "reduce"):
            check_all(rt, l, orc, L, 8, "FLOAT", "SUM", 1234, mode, seed=start, pes=pes, team=team)
            check_all(rt, l, orc, L, 8, "LONGLONG", "MIN", 77, mode, seed=start, pes=pes, team=team)
        l.team_destroy(team)
    l.set_pe(0)


@pytest.mark.parametrize("n_teams", [1, 3, 16, 39])
def test_many_teams_reduce_their_slices_at_once(rt, L, orc, n_teams):
    """tests/functional_tests/team_reduction_tester.cpp: one team per
    work-group.  n_teams duplicates of a team each reduce their slice of one
    array in the same launch; the whole array must equal the oracle's fold,
    for the world team and for a strided one, with ragged sizes."""
    import ctypes
    l = rt.up(8, HEAP)
    for start, stride, size in [(0, 1, 8), (1, 2, 3)]:
        pes = [start + stride * k for k in range(size)]
        l.set_pe(pes[0])
        teams = (ctypes.c_void_p * n_teams)()
        for t in range(n_teams):
            h = ctypes.c_void_p()
            assert l.team_split_strided(l.team_world(), start, stride, size, ctypes.byref(h)) == 0 and h.value
            teams[t] = h.value
        for dtype_name, op_name, n in [("FLOAT", "SUM", 100003), ("INT", "XOR", 7), ("BF16", "SUM", 4099),
                                       ("DOUBLE", "MAX", 1 << 16)]:
            np_t = orc.NP_DTYPE[getattr(orc, dtype_name)]
            es = np.dtype(np_t).itemsize
            b = Buffers(rt, l, (n + 8) * es)
            srcs = make_inputs(orc, dtype_name, size, n, n_teams)
            for p in range(8):
                l.fill(l.pe_ptr(b.dst, p), 0x5A, (n + 8) * es)
            for k, p in enumerate(pes):
                rt.put_bytes(l.pe_ptr(b.src, p), srcs[k])
            want = orc.to_all(getattr(orc, dtype_name), getattr(orc, op_name), srcs)
            # one slice per team, then slices of `chunk` elements dealt out in turn
            # (a chunk that is no whole number of vectors, one larger than the array)
            for chunk in (0, 1000, 4 * n):
                assert l.wg_reduce_teams(getattr(L, dtype_name), getattr(L, op_name), teams, n_teams,
                                         l.pe_ptr(b.dst, pes[0]), l.pe_ptr(b.src, pes[0]), n, chunk, 256, 1,
                                         None) == 0
                for p in range(8):
                    got = rt.get_bytes(l.pe_ptr(b.dst, p), (n + 8) * es, np_t)
                    if p in pes:
                        assert np.array_equal(got[:n].view(np.uint8), want.view(np.uint8)), (dtype_name, n, p, chunk)
                        assert (got[n:].view(np.uint8) == 0x5A).all()
                    else:
                        assert (got.view(np.uint8) == 0x5A).all()
                    l.fill(l.pe_ptr(b.dst, p), 0x5A, (n + 8) * es)
            b.free()
        # the same team twice, or teams over different PEs, are refused
        if n_teams >= 2:
            twice = (ctypes.c_void_p * 2)(teams[0], teams[0])
            assert l.wg_reduce_teams(L.INT, L.SUM, twice, 2, l.pe_ptr(b.src, pes[0]), l.pe_ptr(b.src, pes[0]),
                                     0, 0, 64, 1, None) == -1
        for t in range(n_teams):
            l.team_destroy(teams[t])
    l.set_pe(0)


def test_closed_forms_of_the_reference_tests(rt, L, orc):
    """examples/rocshmem_allreduce_test.cc:49-70 (src[i] = pe + i%9) and
    tests/functional_tests/tester.cpp:147-159 (all ones -> P)."""
    l = rt.up(8, HEAP)
    P, n = 8, 256
    b = Buffers(rt, l, n * 4)
    for p in range(P):
        rt.put_bytes(l.pe_ptr(b.src, p), np.array([p + i % 9 for i in range(n)], np.int32))
    assert l.wg_reduce(L.INT, L.SUM, l.team_world(), b.dst, b.src, n, 256, None) == 0
    expect = np.array([P * (P - 1) // 2 + P * (i % 9) for i in range(n)], np.int32)
    for p in range(P):
        assert np.array_equal(rt.get_bytes(l.pe_ptr(b.dst, p), n * 4, np.int32), expect)
    for p in range(P):
        rt.put_bytes(l.pe_ptr(b.src, p), np.ones(n, np.float32))
    assert l.wg_reduce(L.FLOAT, L.SUM, l.team_world(), b.dst, b.src, n, 64, None) == 0
    for p in range(P):
        assert (rt.get_bytes(l.pe_ptr(b.dst, p), n * 4, np.float32) == P).all()
    b.free()


def test_config1_int32_sum_two_pes_one_mi(rt, L, orc):
    """int32 sum, P=2, 1,048,576 elements per PE, uniform in [-1000,1000], seed 0."""
    l = rt.up(2, 64 << 20)
    n = 1 << 20
    srcs = [orc.fill_i32_pm1000(n, 0, p) for p in range(2)]
    want = orc.to_all(orc.INT, orc.SUM, srcs, nthreads=4)
    assert np.array_equal(want, srcs[0] + srcs[1])
    b = Buffers(rt, l, n * 4)
    for p in range(2):
        rt.put_bytes(l.pe_ptr(b.src, p), srcs[p])
    for mode in ("wg", "to_all"):
        for p in range(2):
            l.fill(l.pe_ptr(b.dst, p), 0, n * 4)
        if mode == "wg":
            assert l.wg_reduce(L.INT, L.SUM, l.team_world(), b.dst, b.src, n, 1024, None) == 0
        else:
            assert l.to_all(L.INT, L.SUM, b.dst, b.src, n, 0, 0, 2, None) == 0
        l.stream_sync(None)
        for p in range(2):
            assert np.array_equal(rt.get_bytes(l.pe_ptr(b.dst, p), n * 4, np.int32), want), (mode, p)
    b.free()
    rt.up(8, HEAP)


@pytest.mark.parametrize("P,nreduce", [(130, 4), (130, 7), (130, 8), (130, 16), (256, 4), (256, 5),
                                       (128, 16), (128, 20000)])
def test_team_too_large_for_reduce_follows_the_reference_selector(rt, L, orc, P, nreduce):
    """A team with 2*P > ROCSHMEM_REDUCE_SYNC_SIZE is refused only when the
    reference's direct path does not fit either (P * nreduce elements against
    max(nreduce/2 + 1, 1024)): src/ipc/context_ipc_tmpl_device.hpp:361-418.
    Status against the oracle's restatement of that selector; data, where the
    call is accepted, against the ascending fold; a refused call leaves the
    destination alone."""
    l = rt.up(P, 2 << 20)
    plan = orc.reduce_plan(P, nreduce)
    b = Buffers(rt, l, nreduce * 4)
    srcs = make_inputs(orc, "INT", P, nreduce, 11)
    for p in range(P):
        rt.put_bytes(l.pe_ptr(b.src, p), srcs[p])
        l.fill(l.pe_ptr(b.dst, p), 0x5A, nreduce * 4)
    rc = l.wg_reduce(L.INT, L.SUM, l.team_world(), b.dst, b.src, nreduce, 64, None)
    assert rc == plan["status"], (P, nreduce, plan)
    want = orc.to_all(orc.INT, orc.SUM, srcs)
    for p in (0, 1, P // 2, P - 1):
        got = rt.get_bytes(l.pe_ptr(b.dst, p), nreduce * 4, np.int32)
        if rc == 0:
            assert np.array_equal(got, want), (P, nreduce, p)
        else:
            assert (got.view(np.uint8) == 0x5A).all(), (P, nreduce, p)
    b.free()
    rt.up(8, HEAP)


@pytest.mark.parametrize("P,lanes", [(3, [64, 192, 1024]), (8, [1024, 64, 256, 192, 1, 640, 128, 65]),
                                     (2, [100, 1000]), (5, [7, 1024, 64, 64, 333])])
@pytest.mark.parametrize("n", [5, 4099, 300007])
def test_member_shares_do_not_depend_on_work_group_sizes(rt, L, orc, P, lanes, n):
    """Team members may run work-groups of different sizes (they are separate
    work-groups, possibly separate kernels): the split of the index range among
    them must tile it all the same.  Each member's share computed with its own
    lane count; every element of every destination against the oracle."""
    import ctypes
    l = rt.up(P, 64 << 20)
    b = Buffers(rt, l, (n + 8) * 4)
    srcs = make_inputs(orc, "INT", P, n, 5)
    for p in range(P):
        rt.put_bytes(l.pe_ptr(b.src, p), srcs[p])
        l.fill(l.pe_ptr(b.dst, p), 0x5A, (n + 8) * 4)
    arr = (ctypes.c_int * P)(*lanes)
    assert l.fold_shares(l.pe_ptr(b.dst, 0), l.pe_ptr(b.src, 0), n, arr, None) == 0
    l.stream_sync(None)
    want = orc.to_all(orc.INT, orc.SUM, srcs)
    for p in range(P):
        got = rt.get_bytes(l.pe_ptr(b.dst, p), (n + 8) * 4, np.int32)
        assert np.array_equal(got[:n], want), (P, lanes, n, p)
        assert (got[n:].view(np.uint8) == 0x5A).all()
    b.free()
    rt.up(8, HEAP)


def test_unsupported_combinations_are_rejected(rt, L):
    l = rt.up(8, HEAP)
    buf = l.malloc(1024)
    assert l.to_all(L.FLOAT, L.XOR, buf, buf, 4, 0, 0, 8, None) == -1
    assert l.to_all(L.BF16, L.MAX, buf, buf, 4, 0, 0, 8, None) == -1
    assert l.to_all(L.INT, L.SUM, buf, buf, 4, 0, 1, 8, None) == -1   # active set leaves the world
    assert l.to_all(L.INT, L.SUM, buf, buf, 1 << 30, 0, 0, 8, None) == -1
    assert l.wg_reduce(L.INT, 9, l.team_world(), buf, buf, 4, 64, None) == -1
    l.free(buf)


@pytest.mark.parametrize("dtype_name,op_name", [("FLOAT", "SUM"), ("BF16", "SUM"), ("FLOAT", "MAX"),
                                                ("LONG", "XOR")])
def test_full_size_64mi_properties(rt, L, orc, dtype_name, op_name, monkeypatch):
    """P=8 x 64 Mi elements, slices in the spread layout (ROCSHMEM_EMU_SPREAD=1,
    as bench.py runs).  Inputs are made on the CPU for windows only; the
    bulk is checked through size-independent properties: all P destinations are
    identical, the windows match the oracle, and for xor reducing the result
    with itself gives zero / reducing twice with P even returns to zero."""
    monkeypatch.setenv("ROCSHMEM_EMU_SPREAD", "1")
    rt.down()
    l = rt.up(8, 2 << 30)
    assert l.pe_stride() >= 16 << 30
    n = 1 << 26
    np_t = orc.NP_DTYPE[getattr(orc, dtype_name)]
    es = np.dtype(np_t).itemsize
    b = Buffers(rt, l, n * es)
    # fill sources on the device by replicating a seeded 4 Mi-element tile
    tile = 1 << 22
    tiles = make_inputs(orc, dtype_name, 8, tile, 123)
    for p in range(8):
        base = l.pe_ptr(b.src, p)
        rt.put_bytes(base, tiles[p])
        done = tile
        while done < n:  # doubling copy inside the slice
            step = min(done, n - done)
            assert l.putmem(base + done * es, base, step * es, p, p, None) == 0
            done += step
    l.stream_sync(None)
    dt, op = getattr(L, dtype_name), getattr(L, op_name)
    assert l.to_all(dt, op, b.dst, b.src, n, 0, 0, 8, None) == 0
    l.stream_sync(None)
    want_tile = orc.to_all(getattr(orc, dtype_name), getattr(orc, op_name), tiles, nthreads=4)
    first = rt.get_bytes(l.pe_ptr(b.dst, 0), n * es, np_t)
    assert np.array_equal(first.reshape(-1, tile).view(np.uint8),
                          np.broadcast_to(want_tile, (n // tile, tile)).copy().view(np.uint8))
    for p in range(1, 8):
        other = rt.get_bytes(l.pe_ptr(b.dst, p), n * es, np_t)
        assert np.array_equal(other.view(np.uint8), first.view(np.uint8)), p
    b.free()
    rt.down()
