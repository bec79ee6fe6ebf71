"""The reference's own programs against this library: its host-API tests
(tests/sos_tests), its device-API functional test driver
(tests/functional_tests with the matrix of scripts/functional_tests/driver.sh)
and its examples, compiled unchanged by oracle/Makefile where the reference
tree lies, run here as separate processes.  Collected last: a program that
fails must not hide the library's own parity tests."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOS_DIR = os.path.join(ROOT, "oracle", "_ref", "sos")
SOS_THREADS_DIR = os.path.join(ROOT, "oracle", "_ref", "sos_threads")


# ---------------------------------------------- the reference's host test programs
# Programs of tests/sos_tests that cannot pass here for reasons of their own:
SOS_EXPECTED_FAILURES = {
    "bigput": "hands addresses of static variables to a reduction; only heap objects are symmetric",
    "put_ctx_mbw_mr": "needs exactly two processes and carries on after finalize otherwise",
    "query_thread": "branches on a variable it never initialises",
}


def sos_programs():
    if not os.path.isdir(SOS_DIR):
        return []
    return sorted(f for f in os.listdir(SOS_DIR) if os.access(os.path.join(SOS_DIR, f), os.X_OK))


@pytest.mark.skipif(not sos_programs(), reason="oracle/_ref/sos is built where the reference tree exists")
@pytest.mark.parametrize("name", sos_programs())
def test_reference_host_programs_run_against_this_library(rt, name):
    """The reference's host-API tests (tests/sos_tests/*.cpp), compiled unchanged
    against these headers and linked with this library by oracle/Makefile, run
    as one PE (they are one-process-per-PE programs; with one PE every transfer
    targets the caller itself) and must report success themselves."""
    rt.down()  # the program brings up its own runtime on the same GPU
    env = dict(os.environ, ROCSHMEM_EMU_NPES="1", ROCSHMEM_HEAP_SIZE=str(1 << 30))
    r = subprocess.run([os.path.join(SOS_DIR, name)], env=env, capture_output=True, text=True, timeout=100)
    if name in SOS_EXPECTED_FAILURES:
        assert r.returncode != 0, "now passes: drop it from the exceptions"
        return
    assert r.returncode == 0, (name, r.stdout[-800:], r.stderr[-800:])


# Run with one thread per PE (rocshmem_emu_run_pes), all PEs share the
# program's file-scope variables and only the PE threads themselves carry a PE
# identity; programs that cannot live with that, or that race by construction,
# are left out:
SOS_NOT_AS_PE_THREADS = {
    "to_all": "keeps its symmetric pointers in file-scope variables",
    "micro_unit_shmem": "keeps its symmetric pointers in file-scope variables",
    "bigput": "hands addresses of static variables to a reduction",
    "put_ctx_mbw_mr": "needs exactly two processes and carries on after finalize otherwise",
    "query_thread": "branches on a variable it never initialises",
    "mt_a2a": "starts threads of its own inside each PE",
    "threading": "starts threads of its own inside each PE",
    "cxx_test_shmem_test": "zeroes its own word with no barrier before the neighbour's put to it",
    "cxx_test_shmem_wait_until": "zeroes its own word with no barrier before the neighbour's put to it",
    "shmem_test": "zeroes its own word with no barrier before the neighbour's put to it",
    "sping": "zeroes its own word with no barrier before the neighbour's put to it",
}


def sos_thread_programs():
    if not os.path.isdir(SOS_THREADS_DIR):
        return []
    return sorted(f for f in os.listdir(SOS_THREADS_DIR)
                  if os.access(os.path.join(SOS_THREADS_DIR, f), os.X_OK) and f not in SOS_NOT_AS_PE_THREADS)


@pytest.mark.skipif(not sos_thread_programs(), reason="oracle/_ref/sos_threads is built where the reference tree exists")
@pytest.mark.parametrize("npes", [2, 8])
@pytest.mark.parametrize("name", sos_thread_programs())
def test_reference_host_programs_run_with_a_thread_per_pe(rt, name, npes):
    """The same programs with their main() run once per PE, every PE a host
    thread of one process (-DROCSHMEM_EMU_PE_THREADS_MAIN): puts, gets,
    atomics, waits, barriers, team splits, broadcasts and reductions between 2
    and 8 PEs, checked by the programs themselves."""
    rt.down()
    env = dict(os.environ, ROCSHMEM_EMU_NPES=str(npes), ROCSHMEM_HEAP_SIZE=str(1 << 30))
    r = subprocess.run([os.path.join(SOS_THREADS_DIR, name)], env=env, capture_output=True, text=True,
                       timeout=100)
    assert r.returncode == 0, (name, npes, r.stdout[-800:], r.stderr[-800:])


# One process per PE, as the reference runs them under mpirun: the launcher
# starts P copies, rocshmem_init exchanges HIP IPC handles of the per-process
# heaps through a rendezvous file, and every transfer between PEs crosses a
# process boundary through a mapped peer heap.
SOS_NOT_AS_PROCESSES = {
    "bigput": "hands addresses of static variables to a reduction; only heap objects are symmetric",
    "query_thread": "branches on a variable it never initialises",
}
SOS_TWO_PROCESSES_ONLY = {"put_ctx_mbw_mr"}  # says so itself


# Every program runs as 2 processes; as 8 processes, the ones that cannot run
# as PE threads (this mode is their only run with more than one PE) and the
# collective ones.  ROCSHMEM_TEST_FULL_PROCESS_MATRIX=1 runs everything at both
# sizes and the whole functional matrix as processes (about 100 s more).
FULL_PROCESS_MATRIX = os.environ.get("ROCSHMEM_TEST_FULL_PROCESS_MATRIX", "0") not in ("", "0")
SOS_EIGHT_PROCESSES = set(SOS_NOT_AS_PE_THREADS) | {
    "barrier", "bcast", "broadcast_active_set", "big_reduction", "max_reduction", "reduce_active_set",
    "reduce_in_place", "shmem_team_reduce", "shmem_team_b2b_collectives", "circular_shift", "atomic_inc"}


def sos_process_cases():
    cases = []
    for name in sos_programs():
        if name in SOS_NOT_AS_PROCESSES:
            continue
        cases.append((name, 2))
        if name not in SOS_TWO_PROCESSES_ONLY and (FULL_PROCESS_MATRIX or name in SOS_EIGHT_PROCESSES):
            cases.append((name, 8))
    return cases


@pytest.mark.skipif(not sos_programs(), reason="oracle/_ref/sos is built where the reference tree exists")
@pytest.mark.parametrize("name,npes", sos_process_cases())
def test_reference_host_programs_run_with_a_process_per_pe(rt, name, npes):
    """The unchanged programs (the build that runs as one PE above) started as
    2 and 8 processes by rocshmem_amd.launch.  This covers the programs that
    cannot share one address space (file-scope symmetric pointers, threads of
    their own, unsynchronised start-up) as well as the rest."""
    from rocshmem_amd import launch
    rt.down()
    env = dict(os.environ, ROCSHMEM_HEAP_SIZE=str(1 << 30))
    env.pop("ROCSHMEM_EMU_NPES", None)
    status, outs = launch.run(npes, [os.path.join(SOS_DIR, name)], timeout=90, env=env, capture=True)
    assert status == 0, (name, npes, [o[-600:] for o in outs])


# ------------------------------------- the reference's device-API functional tests
# The test matrix of scripts/functional_tests/driver.sh:142-320 (all of it runs
# with 2 ranks): (test name, number of the TestType enum in
# tests/functional_tests/tester.hpp, work-groups, threads per work-group,
# largest message size or None).
FUNCTIONAL_MATRIX = [
    ("put", 2, 1, 1, 1048576), ("put", 2, 1, 1024, 512), ("put", 2, 8, 1, 1048576),
    ("put", 2, 16, 128, 8), ("put", 2, 32, 256, 512), ("put", 2, 64, 1024, 8),
    ("wgput", 27, 1, 64, 1048576), ("wgput", 27, 2, 64, 1048576), ("wgput", 27, 16, 64, 8),
    ("waveput", 31, 1, 64, 1048576), ("waveput", 31, 2, 64, 1048576),
    ("waveput", 31, 2, 128, 1048576), ("waveput", 31, 16, 128, 8),
    ("teamctxput", 37, 1, 1, 1048576), ("get", 0, 1, 1, 1048576), ("get", 0, 1, 1024, 512),
    ("get", 0, 8, 1, 1048576), ("get", 0, 16, 128, 8), ("get", 0, 32, 256, 512),
    ("get", 0, 64, 1024, 8), ("wgget", 25, 1, 64, 1048576), ("wgget", 25, 2, 64, 1048576),
    ("wgget", 25, 16, 64, 8), ("waveget", 29, 1, 64, 1048576), ("waveget", 29, 2, 64, 1048576),
    ("waveget", 29, 2, 128, 1048576), ("waveget", 29, 16, 128, 8),
    ("teamctxget", 35, 1, 1, 1048576), ("putnbi", 3, 1, 1, 1048576), ("putnbi", 3, 1, 1024, 512),
    ("putnbi", 3, 8, 1, 1048576), ("putnbi", 3, 16, 128, 8), ("putnbi", 3, 32, 256, 512),
    ("putnbi", 3, 64, 1024, 8), ("wgputnbi", 28, 1, 64, 1048576), ("wgputnbi", 28, 2, 64, 1048576),
    ("wgputnbi", 28, 16, 64, 8), ("waveputnbi", 32, 1, 64, 1048576),
    ("waveputnbi", 32, 2, 64, 1048576), ("waveputnbi", 32, 2, 128, 1048576),
    ("waveputnbi", 32, 16, 128, 8), ("teamctxputnbi", 38, 1, 1, 1048576),
    ("getnbi", 1, 1, 1, 1048576), ("getnbi", 1, 1, 1024, 512), ("getnbi", 1, 8, 1, 1048576),
    ("getnbi", 1, 16, 128, 8), ("getnbi", 1, 32, 256, 512), ("getnbi", 1, 64, 1024, 8),
    ("wggetnbi", 26, 1, 64, 1048576), ("wggetnbi", 26, 2, 64, 1048576),
    ("wggetnbi", 26, 16, 64, 8), ("wavegetnbi", 30, 1, 64, 1048576),
    ("wavegetnbi", 30, 2, 64, 1048576), ("wavegetnbi", 30, 2, 128, 1048576),
    ("wavegetnbi", 30, 16, 128, 8), ("teamctxgetnbi", 36, 1, 1, 1048576),
    ("amo_fetch", 7, 1, 1, None), ("amo_fetch", 7, 1, 1024, None), ("amo_fetch", 7, 8, 1, None),
    ("amo_fetch", 7, 32, 128, None), ("amo_set", 41, 1, 1, None), ("amo_set", 41, 8, 1, None),
    ("amo_set", 41, 32, 1, None), ("amo_fcswap", 8, 1, 1, None), ("amo_fcswap", 8, 32, 1, None),
    ("amo_fcswap", 8, 8, 1, None), ("amo_finc", 6, 1, 1, None), ("amo_finc", 6, 1, 1024, None),
    ("amo_finc", 6, 8, 1, None), ("amo_finc", 6, 32, 128, None), ("amo_inc", 10, 1, 1, None),
    ("amo_inc", 10, 1, 1024, None), ("amo_inc", 10, 8, 1, None), ("amo_inc", 10, 32, 128, None),
    ("amo_fadd", 5, 1, 1, None), ("amo_fadd", 5, 1, 1024, None), ("amo_fadd", 5, 8, 1, None),
    ("amo_fadd", 5, 32, 128, None), ("amo_add", 9, 1, 1, None), ("amo_add", 9, 1, 1024, None),
    ("amo_add", 9, 8, 1, None), ("amo_add", 9, 32, 128, None), ("amo_fetchand", 43, 1, 1, None),
    ("amo_and", 46, 1, 1, None), ("amo_xor", 48, 1, 1, None), ("putsignal", 50, 1, 1, 1048576),
    ("putsignal", 50, 2, 32, 1048576), ("wgputsignal", 51, 2, 32, 1048576),
    ("waveputsignal", 52, 1, 32, 1048576), ("waveputsignal", 52, 2, 64, 1048576),
    ("putsignalnbi", 53, 1, 1, 1048576), ("putsignalnbi", 53, 2, 32, 1048576),
    ("wgputsignalnbi", 54, 2, 32, 1048576), ("waveputsignalnbi", 55, 1, 32, 1048576),
    ("waveputsignalnbi", 55, 2, 64, 1048576), ("signalfetch", 56, 1, 1, None),
    ("wgsignalfetch", 57, 2, 32, None), ("wavesignalfetch", 58, 1, 32, None),
    ("wavesignalfetch", 58, 1, 64, None), ("barrierall", 15, 1, 1, None), ("sync", 17, 1, 1, None),
    ("syncall", 16, 1, 1, None), ("alltoall", 20, 1, 1, 512), ("teambroadcast", 33, 1, 1, 32768),
    ("fcollect", 19, 1, 1, 512), ("fcollect", 19, 1, 1, 32768), ("teamreduction", 34, 1, 1, 32768),
    ("init", 12, 1, 1, None), ("pingpong", 13, 1, 1, None), ("pingpong", 13, 8, 1, None),
    ("pingpong", 13, 32, 1, None), ("teamctxinfra", 39, 1, 1, None),
]
FUNCTIONAL_DRIVER = os.path.join(ROOT, "oracle", "_ref", "functional", "rocshmem_example_driver")
# Nothing is left out: kernels that both ranks launch find their PE through the
# hardware queue their PE thread bound, and team handles kept in file-scope
# variables (team_reduction_tester.cpp:71, team_ctx_primitive_tester.cpp:29)
# are the same value in every PE thread.
FUNCTIONAL_NEEDS_ONE_PROCESS_PER_PE = set()


def functional_cases():
    if not os.path.exists(FUNCTIONAL_DRIVER):
        return []
    return [c for c in FUNCTIONAL_MATRIX if c[0] not in FUNCTIONAL_NEEDS_ONE_PROCESS_PER_PE]


@pytest.mark.skipif(not functional_cases(),
                    reason="oracle/_ref/functional is built where the reference tree exists")
@pytest.mark.parametrize("name,number,wgs,threads,max_size", functional_cases(),
                         ids=["%s-w%d-z%d-%s" % (c[0], c[2], c[3], c[4]) for c in functional_cases()])
def test_reference_functional_driver(rt, name, number, wgs, threads, max_size):
    """The reference's own functional test driver (tests/functional_tests: the
    testers' kernels call rocshmem_putmem/getmem/_wg/_wave, the atomics,
    put_signal, signal_fetch, team alltoall/broadcast/fcollect ... and each
    tester verifies the data itself), compiled unchanged against these headers
    by oracle/Makefile, run with 2 PEs as two host threads, with the arguments
    of the reference's driver script.  Exit status 0 = the tester's own
    verification passed for every message size.  Work-groups of different PEs
    wait for each other inside kernels, so each PE thread's stream needs a
    hardware queue of its own: 16 queues instead of HIP's default 4."""
    rt.down()
    env = dict(os.environ, ROCSHMEM_EMU_NPES="2", GPU_MAX_HW_QUEUES="16",
               ROCSHMEM_MAX_NUM_CONTEXTS="1024" if name == "teamctxinfra" else str(wgs))
    cmd = [FUNCTIONAL_DRIVER, "-a", str(number), "-w", str(wgs), "-z", str(threads)]
    if max_size is not None:
        cmd += ["-s", str(max_size)]
    r = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, (name, r.stdout[-600:], r.stderr[-600:])


# Device waits between processes are bounded in these runs: a wait that would
# never end (a lost signal, kernels of two processes that cannot run side by
# side) gives up after this many polls and the tester's own check then fails,
# instead of a kernel that never exits.
PROCESS_RUN_SPIN_LIMIT = str(40_000_000)


def functional_process_cases():
    """One row of the matrix per tester (the cheapest one: a bounded message
    size where the script has one), all pingpong rows; the whole matrix with
    ROCSHMEM_TEST_FULL_PROCESS_MATRIX=1.  The whole matrix always runs with
    the ranks as PE threads, above."""
    if FULL_PROCESS_MATRIX:
        return functional_cases()
    best = {}
    for c in functional_cases():
        cost = (c[4] if c[4] is not None else 0, c[2] * c[3])
        if c[0] == "pingpong":
            best[(c[0], c[2])] = (cost, c)
        elif c[0] not in best or cost < best[c[0]][0]:
            best[c[0]] = (cost, c)
    keep = {id(v[1]) for v in best.values()}
    return [c for c in functional_cases() if id(c) in keep]


@pytest.mark.skipif(not functional_cases(),
                    reason="oracle/_ref/functional is built where the reference tree exists")
@pytest.mark.parametrize("name,number,wgs,threads,max_size", functional_process_cases(),
                         ids=["%s-w%d-z%d-%s" % (c[0], c[2], c[3], c[4]) for c in functional_process_cases()])
def test_reference_functional_driver_with_a_process_per_pe(rt, name, number, wgs, threads, max_size):
    """The same driver with the 2 ranks as 2 processes, the way the reference's
    script runs it (mpirun -np 2): every put, get, atomic and signal issued
    inside a kernel lands in the other process's heap through its HIP IPC
    mapping, and the device-side barriers and collectives of the testers meet
    across the process boundary."""
    from rocshmem_amd import launch
    rt.down()
    env = dict(os.environ, ROCSHMEM_EMU_SPIN_LIMIT=PROCESS_RUN_SPIN_LIMIT,
               ROCSHMEM_MAX_NUM_CONTEXTS="1024" if name == "teamctxinfra" else str(wgs))
    env.pop("ROCSHMEM_EMU_NPES", None)
    cmd = [FUNCTIONAL_DRIVER, "-a", str(number), "-w", str(wgs), "-z", str(threads)]
    if max_size is not None:
        cmd += ["-s", str(max_size)]
    status, outs = launch.run(2, cmd, timeout=90, env=env, capture=True)
    assert status == 0, (name, [o[-600:] for o in outs])


# ------------------------------------------------- the reference's example programs
EXAMPLES_DIR = os.path.join(ROOT, "oracle", "_ref", "examples")


def example_programs():
    if not os.path.isdir(EXAMPLES_DIR):
        return []
    return sorted(f for f in os.listdir(EXAMPLES_DIR) if os.access(os.path.join(EXAMPLES_DIR, f), os.X_OK))


@pytest.mark.skipif(not example_programs(), reason="oracle/_ref/examples is built where the reference tree exists")
@pytest.mark.parametrize("npes", [2, 8])
@pytest.mark.parametrize("name", example_programs())
def test_reference_examples_run_with_a_thread_per_pe(rt, name, npes):
    """examples/*.cc of the reference (all-reduce, alltoall, broadcast, getmem,
    put_signal + wait_until inside kernels that every PE launches with
    kernel<<<...>>> on its default stream), built unchanged by oracle/Makefile
    with a per-thread default stream, one host thread per PE.  Each PE checks
    its own result and prints [PASS] or [FAIL] (the broadcast root checks
    nothing)."""
    rt.down()
    env = dict(os.environ, ROCSHMEM_EMU_NPES=str(npes), GPU_MAX_HW_QUEUES="16")
    r = subprocess.run([os.path.join(EXAMPLES_DIR, name)], env=env, capture_output=True, text=True,
                       timeout=100)
    assert r.returncode == 0, (name, npes, r.stdout[-600:], r.stderr[-600:])
    assert r.stdout.count("[FAIL]") == 0, r.stdout[-600:]
    assert r.stdout.count("[PASS]") >= npes - 1, r.stdout[-600:]


@pytest.mark.skipif(not example_programs(), reason="oracle/_ref/examples is built where the reference tree exists")
@pytest.mark.parametrize("npes", [2, 8])
@pytest.mark.parametrize("name", example_programs())
def test_reference_examples_run_with_a_process_per_pe(rt, name, npes):
    """The examples as 2 and 8 processes (mpirun -np in the reference): their
    kernels' collectives and signals cross process boundaries."""
    from rocshmem_amd import launch
    rt.down()
    env = dict(os.environ, ROCSHMEM_EMU_SPIN_LIMIT=PROCESS_RUN_SPIN_LIMIT)
    env.pop("ROCSHMEM_EMU_NPES", None)
    status, outs = launch.run(npes, [os.path.join(EXAMPLES_DIR, name)], timeout=90, env=env, capture=True)
    assert status == 0, (name, npes, [o[-600:] for o in outs])
    text = "".join(outs)
    assert text.count("[FAIL]") == 0, text[-600:]
    assert text.count("[PASS]") >= npes - 1, text[-600:]
