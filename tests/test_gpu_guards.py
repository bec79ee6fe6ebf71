"""Refusals on the GPU: a grid of work-groups that wait for each other and
cannot all be resident, a blocking wait that nobody will satisfy, and team
creation from several host threads at once."""
import ctypes
import os
import subprocess
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HEAP = 32 << 20
P = 8
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXAMPLE = os.path.join(ROOT, "oracle", "_ref", "examples", "rocshmem_allreduce_test")


def test_reduce_grid_that_cannot_be_resident_is_refused_and_launches_nothing(rt, L, monkeypatch):
    """256 teams x 8 PEs x 1024 lanes is eight times what 256 CUs hold: every
    work-group would wait for a member that is never scheduled.  The driver
    returns -1, the destination keeps its fill, and the same call at a size that
    fits works right after."""
    monkeypatch.setenv("ROCSHMEM_MAX_NUM_TEAMS", "264")
    rt.down()
    l = rt.up(P, HEAP)
    l.set_pe(0)
    n_teams = 256
    teams = (ctypes.c_void_p * n_teams)()
    for t in range(n_teams):
        h = ctypes.c_void_p()
        assert l.team_split_strided(l.team_world(), 0, 1, P, ctypes.byref(h)) == 0 and h.value
        teams[t] = h.value
    n = 1 << 16
    src, dst = l.malloc(n * 4), l.malloc(n * 4)
    ones = np.ones(n, np.int32)
    for p in range(P):
        rt.put_bytes(l.pe_ptr(src, p), ones)
        l.fill(l.pe_ptr(dst, p), 0x5A, n * 4)
    for entry in (l.wg_reduce_teams, l.wg_reduce_teams_static):
        assert entry(L.INT, L.SUM, teams, n_teams, dst, src, n, 0, 1024, 1, None) == -1
    l.stream_sync(None)
    for p in range(P):
        assert (rt.get_bytes(l.pe_ptr(dst, p), n * 4) == 0x5A).all()
    assert l.wg_reduce_teams(L.INT, L.SUM, teams, 16, dst, src, n, 0, 256, 1, None) == 0
    for p in range(P):
        assert (rt.get_bytes(l.pe_ptr(dst, p), n * 4, np.int32) == P).all()
    # the other drivers whose work-groups wait for each other share the rule
    buf, sig = l.malloc(1 << 20), l.malloc(8 * 128)
    ticks, hz = ctypes.c_uint64(), ctypes.c_double()
    assert l.pingpong(buf, sig, 64, 10, 128, 0, 1, 1024, ctypes.byref(ticks), ctypes.byref(hz), None) == 0
    for x in (src, dst, buf, sig):
        l.free(x)
    for t in range(n_teams):
        l.team_destroy(teams[t])
    rt.down()


def test_waits_give_up_after_the_spin_limit(rt, L):
    """With a spin limit the runtime's waits stop after that many polls, count
    themselves and return, so a wait that nobody will satisfy ends its kernel
    normally (the reference's would spin for ever,
    src/context_tmpl_device.hpp:201-218).  Without a limit nothing changes: the
    same call is refused before launch, satisfied waits count nothing."""
    l = rt.up(P, HEAP)
    vals = np.array([5, 0, 5, 0, 0, 0], np.int64)
    iv = rt.dev_array(vals)
    five, nine = np.array([5], np.int64), np.array([9], np.int64)
    ret = ctypes.c_size_t(77)
    idx = (ctypes.c_size_t * 6)()
    assert l.waits_given_up(1) == 0
    assert l.wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret), None) == -2
    assert l.set_spin_limit(2000) == 0
    try:
        assert l.wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret),
                           None) == 0
        assert l.waits_given_up(0) == 1
        assert l.wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 6, None, L.CMP_EQ, nine.ctypes.data,
                           ctypes.byref(ret), None) == 0
        assert ret.value == L.SIZE_MAX          # nothing was satisfied
        assert l.wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 6, None, L.CMP_EQ, nine.ctypes.data,
                           ctypes.byref(ret), idx) == 0
        assert ret.value == 0
        assert l.waits_given_up(1) == 3 and l.waits_given_up(0) == 0
        # a wait whose condition holds does not count
        assert l.wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_EQ, five.ctypes.data, ctypes.byref(ret),
                           None) == 0
        assert l.waits_given_up(0) == 0
    finally:
        assert l.set_spin_limit(0) == 0
    assert l.wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret), None) == -2
    l.dev_free(iv)


def test_blocking_wait_that_nobody_will_satisfy_is_refused(rt, L):
    """rocshmem_amd_wait_test launches a wait with no waker: if the condition
    does not hold already the kernel would spin for ever, so the call returns
    -2 and launches nothing; satisfied conditions and empty vectors still run."""
    l = rt.up(P, HEAP)
    vals = np.array([5, 0, 5, 0, 0, 0], np.int64)
    iv = rt.dev_array(vals)
    five, nine = np.array([5], np.int64), np.array([9], np.int64)
    ret = ctypes.c_size_t()
    assert l.wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret), None) == -2
    assert l.wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 6, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret), None) == -2
    assert l.wait_test(L.WAIT_UNTIL_SOME, L.LONG, iv, 6, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret), None) == -2
    assert l.wait_test(L.WAIT_UNTIL_ALL, L.LONG, iv, 6, None, L.CMP_EQ, five.ctypes.data, ctypes.byref(ret), None) == -2
    # masked entries do not count: only entries 0 and 2 are looked at
    status = (ctypes.c_int * 6)(0, 1, 0, 1, 1, 1)
    assert l.wait_test(L.WAIT_UNTIL_ALL, L.LONG, iv, 6, status, L.CMP_EQ, five.ctypes.data, ctypes.byref(ret), None) == 0
    assert l.wait_test(L.WAIT_UNTIL, L.LONG, iv, 1, None, L.CMP_EQ, five.ctypes.data, ctypes.byref(ret), None) == 0
    assert l.wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 6, None, L.CMP_EQ, five.ctypes.data, ctypes.byref(ret), None) == 0
    assert ret.value == 0
    assert l.wait_test(L.TEST, L.LONG, iv, 1, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret), None) == 0
    assert ret.value == 0
    assert l.wait_test(L.WAIT_UNTIL_ANY, L.LONG, iv, 0, None, L.CMP_EQ, nine.ctypes.data, ctypes.byref(ret), None) == 0
    # a null or out-of-slice array is an argument error
    assert l.wait_test(L.TEST, L.LONG, None, 1, None, L.CMP_EQ, five.ctypes.data, ctypes.byref(ret), None) == -1
    l.dev_free(iv)


def test_teams_created_and_destroyed_from_two_host_threads_at_once(rt, L):
    """Two host threads split and destroy sub-teams of different parents at the
    same time, as PE threads of disjoint teams do.  Every handle must be valid,
    distinct from the handles that are live at that moment, and describe the
    team that was asked for."""
    l = rt.up(P, HEAP)
    l.set_pe(0)
    parents = []
    for stride, size in ((2, 4), (1, 4)):
        h = ctypes.c_void_p()
        assert l.team_split_strided(l.team_world(), 0, stride, size, ctypes.byref(h)) == 0 and h.value
        parents.append((h.value, stride))
    errors = []

    def worker(parent, parent_stride):
        try:
            for it in range(150):
                made = []
                for size in (2, 3):
                    h = ctypes.c_void_p()
                    rc = l.team_split_strided(parent, 0, 1, size, ctypes.byref(h))
                    if rc != 0 or not h.value:
                        errors.append(("split", rc))
                        return
                    s, st, sz = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
                    if l.team_active_set(h.value, ctypes.byref(s), ctypes.byref(st), ctypes.byref(sz)) != 0 or \
                            (s.value, st.value, sz.value) != (0, parent_stride, size):
                        errors.append(("shape", s.value, st.value, sz.value, parent_stride, size))
                        return
                    made.append(h.value)
                if len(set(made)) != len(made):
                    errors.append(("duplicate", made))
                    return
                for h in made:
                    l.team_destroy(h)
        except Exception as e:  # pragma: no cover
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=p) for p in parents]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:3]
    # the pool is back to the two parents: 37 more teams can be made
    spare = []
    for _ in range(37):
        h = ctypes.c_void_p()
        assert l.team_split_strided(l.team_world(), 0, 1, 2, ctypes.byref(h)) == 0 and h.value
        spare.append(h.value)
    for h in spare + [p[0] for p in parents]:
        l.team_destroy(h)


@pytest.mark.skipif(not os.path.exists(EXAMPLE),
                    reason="oracle/_ref/examples is built where the reference tree exists")
@pytest.mark.parametrize("npes,queues", [(4, 2), (4, 4), (8, 8)])
def test_too_few_hardware_queues_end_the_program_before_anything_is_launched(rt, npes, queues):
    """One host thread per PE, each launching kernels on a stream of its own
    (the reference's all-reduce example, built with a per-thread default
    stream), with fewer hardware queues than PEs + 1: the set-up in which a
    kernel can queue behind the kernel that waits for it.  rocshmem_init refuses
    it before the runtime allocates or enqueues anything: message, exit status
    1 (with ROCSHMEM_EMU_VERBOSE the layout line of a completed init never
    appears)."""
    rt.down()
    env = dict(os.environ, ROCSHMEM_EMU_NPES=str(npes), GPU_MAX_HW_QUEUES=str(queues),
               ROCSHMEM_EMU_VERBOSE="1")
    r = subprocess.run([EXAMPLE], env=env, capture_output=True, text=True, timeout=60)
    assert r.returncode == 1, (r.returncode, r.stderr[-400:])
    assert "GPU_MAX_HW_QUEUES=%d" % queues in r.stderr and "Nothing was launched" in r.stderr
    assert "slices" not in r.stderr  # the runtime never came up
