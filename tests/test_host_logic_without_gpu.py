"""The runtime's host logic without a GPU: rocshmem_init in one process and
between the processes of a job (handle exchange, layout check, peer table,
contexts), address resolution, the allocator's symmetry, team bookkeeping and
host-initiated copies, with tests/hip_stub's stand-in for the HIP runtime in
front of the real one for the child processes that load the product library.
Kernels do not run there — launches are counted and dropped, except the
whole-GPU copy kernel, which the stand-in carries out after checking both
ranges against the memory the process has allocated or mapped — so nothing
here is a parity result of device code; those are the -m gpu tests.

What these tests pin is what a kernel would be GIVEN: the context fields and
the table from which device code forms a peer's address
(detail/state.hpp::remote_addr; the reference's ipc_bases[pe] + offset,
src/ipc/context_ipc_device.cpp:62-69) must give the address the host resolves,
in one process and across processes, and a host-computed address that leaves
the mapped memory ends the test instead of faulting a GPU."""
import os
import subprocess
import sys

import pytest

from rocshmem_amd import launch
from rocshmem_amd import lib as L

HERE = os.path.dirname(os.path.abspath(__file__))
STUB_DIR = os.path.join(HERE, "hip_stub")
STUB = os.path.join(STUB_DIR, "_build", "libamdhip64.so.7")
WORKER = [sys.executable, os.path.join(HERE, "procs_stub_worker.py")]


@pytest.fixture(scope="module")
def stub_env():
    if not os.path.exists(L.LIB_PATH):
        pytest.skip("library not built")
    r = subprocess.run(["make", "-C", STUB_DIR], capture_output=True, text=True)
    if r.returncode != 0 or not os.path.exists(STUB):
        pytest.skip("the HIP stand-in does not build here: " + r.stderr[-300:])
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = os.path.dirname(STUB) + os.pathsep + env.get("LD_LIBRARY_PATH", "")
    for name in ("ROCSHMEM_EMU_NPES", "ROCSHMEM_EMU_SPREAD", "ROCSHMEM_EMU_HEAP_CACHED", "ROCSHMEM_HEAP_SIZE"):
        env.pop(name, None)
    return env


def test_one_process_contexts_and_copies(stub_env):
    r = subprocess.run(WORKER + ["one"], env=stub_env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.stdout[-800:], r.stderr[-1500:])
    assert "one process ok" in r.stdout


def test_refused_calls_launch_nothing(stub_env):
    """include/rocshmem_amd.h: every driver validates pointers and sizes against
    the heap on the host before launching.  Forty calls that must be refused,
    with the stand-in counting the launches in between."""
    r = subprocess.run(WORKER + ["refusals"], env=stub_env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.stdout[-800:], r.stderr[-1500:])
    assert "refusals ok" in r.stdout


def test_the_entry_point_for_callers_that_cannot_allocate_allocates_nothing(stub_env):
    r = subprocess.run(WORKER + ["no-alloc"], env=stub_env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.stdout[-800:], r.stderr[-1500:])
    assert "no alloc ok" in r.stdout


@pytest.mark.parametrize("nprocs", [2, 5])
def test_a_job_of_processes_brings_up_and_moves_data(stub_env, nprocs):
    status, outs = launch.run(nprocs, WORKER + ["job"], timeout=120, env=stub_env, capture=True)
    assert status == 0, [o[-1500:] for o in outs]
    for pe, o in enumerate(outs):
        assert "ok %d" % pe in o, o[-1500:]


def test_processes_that_disagree_about_the_heap_are_stopped_at_init(stub_env):
    status, outs = launch.run(2, WORKER + ["unequal-heaps"], timeout=60, env=stub_env, capture=True)
    text = "".join(outs)
    assert status != 0 and "disagree about the job" in text, text[-800:]
    assert "init returned" not in text


def test_a_process_that_dies_does_not_leave_the_others_waiting_for_ever(stub_env):
    """Failure handling between processes, on the CPU: the survivors' meeting
    runs out (ROCSHMEM_EMU_RDV_TIMEOUT_S) and they end; the launcher reports
    the first failure."""
    import time
    env = dict(stub_env, ROCSHMEM_EMU_RDV_TIMEOUT_S="2")
    t0 = time.monotonic()
    status, outs = launch.run(3, WORKER + ["one-dies"], timeout=60, env=env, capture=True)
    assert status == 3, outs
    assert time.monotonic() - t0 < 30
    assert "barrier returned" not in "".join(outs)


def test_global_exit_ends_every_process_with_its_status(stub_env):
    """rocshmem_global_exit(status) (the reference: MPI_Abort): the caller ends
    at once and the others at their next meeting, all with that status."""
    status, outs = launch.run(3, WORKER + ["global-exit"], timeout=60, env=stub_env, capture=True)
    assert status == 7, outs
    assert "barrier returned" not in "".join(outs)


def test_the_stand_in_ends_a_process_that_leaves_its_memory(stub_env):
    r = subprocess.run(WORKER + ["memset-outside"], env=stub_env, capture_output=True, text=True, timeout=60)
    assert r.returncode == 97, (r.returncode, r.stderr[-500:])
    assert "not inside memory this process has allocated or mapped" in r.stderr
    assert "survived" not in r.stdout


# The reference's host programs (tests/sos_tests, built unchanged by
# oracle/Makefile) that get by without any kernel of the library — puts, gets,
# barriers, broadcasts, allocation, teams, global_exit — and that do not race
# by construction: as 2 and 4 processes under the stand-in they exercise the
# host API between processes end to end, each program checking its own data.
SOS_DIR = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "sos")
SOS_WITHOUT_KERNELS = ["hello", "barrier", "put1", "get1", "bigget", "circular_shift", "shmalloc",
                       "asym_alloc", "bcast", "bcast_flood", "broadcast_active_set", "global_exit",
                       "get_nbi", "shmem_team_translate", "shmem_team_reuse_teams", "cxx_test_shmem_p",
                       "cxx_test_shmem_g"]


@pytest.mark.skipif(not os.path.isdir(SOS_DIR), reason="oracle/_ref/sos is built where the reference tree exists")
@pytest.mark.parametrize("nprocs", [2, 4])
@pytest.mark.parametrize("name", SOS_WITHOUT_KERNELS)
def test_reference_host_programs_as_processes(stub_env, name, nprocs):
    prog = os.path.join(SOS_DIR, name)
    if not os.access(prog, os.X_OK):
        pytest.skip("not built")
    env = dict(stub_env, ROCSHMEM_HEAP_SIZE=str(64 << 20))
    status, outs = launch.run(nprocs, [prog], timeout=60, env=env, capture=True)
    assert status == 0, (name, nprocs, [o[-600:] for o in outs])


# The same with a host thread per PE (the builds with their main() run once per
# PE): there the host broadcast is a kernel of its own, which the stand-in
# drops, so the broadcast programs are left to the GPU tests.
SOS_THREADS_DIR = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "sos_threads")
SOS_THREADS_WITHOUT_KERNELS = [n for n in SOS_WITHOUT_KERNELS
                               if n not in ("bcast", "bcast_flood", "broadcast_active_set")]


@pytest.mark.skipif(not os.path.isdir(SOS_THREADS_DIR),
                    reason="oracle/_ref/sos_threads is built where the reference tree exists")
@pytest.mark.parametrize("npes", [2, 8])
@pytest.mark.parametrize("name", SOS_THREADS_WITHOUT_KERNELS)
def test_reference_host_programs_with_a_thread_per_pe(stub_env, name, npes):
    prog = os.path.join(SOS_THREADS_DIR, name)
    if not os.access(prog, os.X_OK):
        pytest.skip("not built")
    env = dict(stub_env, ROCSHMEM_EMU_NPES=str(npes), ROCSHMEM_HEAP_SIZE=str(64 << 20))
    r = subprocess.run([prog], env=env, capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, (name, npes, r.stdout[-600:], r.stderr[-600:])


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits."""
    r = subprocess.run([sys.executable, os.path.join(os.path.dirname(HERE), "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_bench_two_process_leg_runs_to_completion(stub_env):
    """The plumbing of bench.py's optional leg between two processes (bring-up
    with a 1.9 GiB heap per process, three rotating 256 MiB buffer pairs, the
    order of the meetings between the timing PE and the checking PE, the
    record it prints).  Under the stand-in no kernel runs, so the figures mean
    nothing and the check passes vacuously; what is tested is that both
    processes get through and that the record parses."""
    import json
    bench = os.path.join(os.path.dirname(HERE), "bench.py")
    status, outs = launch.run(2, [sys.executable, bench, "--process-leg", "--steps", "2", "--warmup", "1"],
                              timeout=240, env=stub_env, capture=True)
    assert status == 0, [o[-800:] for o in outs]
    text = "\n".join(outs)
    rec = [ln for ln in text.splitlines() if ln.startswith("PROCESS_LEG ")]
    assert len(rec) == 1 and "PROCESS_LEG_VERIFIED 1" in text
    fields = json.loads(rec[0][len("PROCESS_LEG "):])
    assert set(fields) == {"putmem_wg_nostore_gbs", "getmem_wg_nostore_gbs", "putmem_wg_default_ctx_gbs",
                           "host_putmem_gbs"}
