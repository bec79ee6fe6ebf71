"""The entry point that allocates nothing: rocshmem_amd_wg_reduce_teams_static
against rocshmem_amd_wg_reduce_teams, through the C entry points."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HEAP = 64 << 20
P = 8


def _teams(l, n_teams):
    teams = (ctypes.c_void_p * n_teams)()
    for t in range(n_teams):
        h = ctypes.c_void_p()
        assert l.team_split_strided(l.team_world(), 0, 1, P, ctypes.byref(h)) == 0 and h.value
        teams[t] = h.value
    return teams


def _run(rt, l, L, entry, dtype, op, np_t, teams, n_teams, n, srcs, wg, chunk=0):
    """One call of `entry` on fresh destination arrays; returns (status, the
    destination array of every PE with 8 guard elements behind it)."""
    es = np.dtype(np_t).itemsize
    src, dst = l.malloc((n + 8) * es), l.malloc((n + 8) * es)
    assert src and dst
    for p in range(P):
        rt.put_bytes(l.pe_ptr(src, p), srcs[p])
        l.fill(l.pe_ptr(dst, p), 0x5A, (n + 8) * es)
    rc = entry(dtype, op, teams, n_teams, dst, src, n, chunk, wg, 1, None)
    out = [rt.get_bytes(l.pe_ptr(dst, p), (n + 8) * es, np.uint8) for p in range(P)]
    l.free(src)
    l.free(dst)
    return rc, out


def test_static_entry_point_matches_the_allocating_one_twice_in_a_row(rt, L, orc):
    """Calls in a row, each with fewer teams and a smaller array than the one
    before: the static status words keep the earlier call's contents, so a
    later call only passes if it clears what it uses.  Bit-exact against the
    allocating entry point and against the oracle's ascending fold."""
    l = rt.up(P, HEAP)
    l.set_pe(0)
    teams = _teams(l, 24)
    cases = [(24, 200003, L.FLOAT, L.SUM, orc.FLOAT, orc.SUM, np.float32, 256, 0),
             (5, 4099, L.LONG, L.XOR, orc.LONG, orc.XOR, np.int64, 64, 0),
             (3, 1001, L.LONG, L.XOR, orc.LONG, orc.XOR, np.int64, 128, 64)]
    for n_teams, n, dt, op, odt, oop, np_t, wg, chunk in cases:
        rng = np.random.default_rng(n)
        if np_t is np.float32:
            srcs = [rng.standard_normal(n).astype(np.float32) for _ in range(P)]
        else:
            srcs = [rng.integers(-2**62, 2**62, n, dtype=np.int64) for _ in range(P)]
        rc_a, out_a = _run(rt, l, L, l.wg_reduce_teams, dt, op, np_t, teams, n_teams, n, srcs, wg, chunk)
        rc_s, out_s = _run(rt, l, L, l.wg_reduce_teams_static, dt, op, np_t, teams, n_teams, n, srcs, wg, chunk)
        assert rc_a == 0 and rc_s == 0
        want = orc.to_all(odt, oop, srcs).view(np.uint8)
        for p in range(P):
            assert np.array_equal(out_s[p], out_a[p]), (n_teams, n, p)
            assert np.array_equal(out_s[p][:want.size], want), (n_teams, n, p)
            assert (out_s[p][want.size:] == 0x5A).all()
    for t in range(24):
        l.team_destroy(teams[t])


def test_static_entry_point_reports_the_device_status_and_its_limit(rt, L):
    """A team too large for the reduce (2 P > ROCSHMEM_REDUCE_SYNC_SIZE cannot be
    built with 8 PEs), so the error path taken here is the launch refusal; a
    clean call after it still returns 0 (stale status words are cleared).  More
    than 256 teams are refused before anything is launched."""
    l = rt.up(P, HEAP)
    l.set_pe(0)
    teams = _teams(l, 2)
    n = 1000
    src, dst = l.malloc(n * 4), l.malloc(n * 4)
    for p in range(P):
        l.fill(l.pe_ptr(src, p), 0, n * 4)
    # the same team twice is refused, by both entry points alike
    twice = (ctypes.c_void_p * 2)(teams[0], teams[0])
    assert l.wg_reduce_teams_static(L.INT, L.SUM, twice, 2, dst, src, n, 0, 64, 1, None) == -1
    assert l.wg_reduce_teams(L.INT, L.SUM, twice, 2, dst, src, n, 0, 64, 1, None) == -1
    assert l.wg_reduce_teams_static(L.INT, L.SUM, teams, 2, dst, src, n, 0, 64, 1, None) == 0
    many = (ctypes.c_void_p * 300)(*([teams[0]] * 300))
    assert l.wg_reduce_teams_static(L.INT, L.SUM, many, 300, dst, src, n, 0, 64, 1, None) == -1
    # a refused call puts nothing on the stream, not even the clearing of the
    # status words: the destination is as it was
    for p in range(P):
        l.fill(l.pe_ptr(dst, p), 0x5A, n * 4)
    assert l.wg_reduce_teams_static(L.INT, L.SUM, teams, 2, dst, src, -1, 0, 64, 1, None) == -1
    assert l.wg_reduce_teams_static(L.INT, L.SUM, teams, 2, dst, src, n, -5, 64, 1, None) == -1
    l.stream_sync(None)
    for p in range(P):
        assert (rt.get_bytes(l.pe_ptr(dst, p), n * 4) == 0x5A).all()
    l.free(src)
    l.free(dst)
    for t in range(2):
        l.team_destroy(teams[t])


def test_static_entry_point_allocates_no_device_memory(rt, L):
    """Free device memory is the same before and after repeated calls, and does
    not dip during them as far as the host can see between calls."""
    l = rt.up(P, HEAP)
    l.set_pe(0)
    teams = _teams(l, 8)
    n = 50000
    src, dst = l.malloc(n * 4), l.malloc(n * 4)
    for p in range(P):
        l.fill(l.pe_ptr(src, p), 1, n * 4)
    assert l.wg_reduce_teams_static(L.INT, L.SUM, teams, 8, dst, src, n, 0, 128, 1, None) == 0
    free0, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert l.dev_mem_info(ctypes.byref(free0), ctypes.byref(total)) == 0
    seen = set()
    for k in range(20):
        assert l.wg_reduce_teams_static(L.INT, L.SUM, teams, 1 + k % 8, dst, src, n, 0, 128, 1, None) == 0
        free1 = ctypes.c_size_t()
        assert l.dev_mem_info(ctypes.byref(free1), ctypes.byref(total)) == 0
        seen.add(free1.value)
    assert seen == {free0.value}, (free0.value, sorted(seen))
    l.free(src)
    l.free(dst)
    for t in range(8):
        l.team_destroy(teams[t])
