"""One process per PE on one GPU, through the C entry points: the reference's
deployment (a process per PE, peers' heaps mapped through HIP IPC,
src/ipc_policy.cpp:34-118) with this library's rendezvous in the place of MPI.
Every process checks its own slice bit for bit against the CPU oracle."""
import os
import sys

import pytest

pytestmark = pytest.mark.gpu

WORKER = [sys.executable, os.path.join(os.path.dirname(os.path.abspath(__file__)), "procs_gpu_worker.py")]


@pytest.mark.parametrize("nprocs", [2, 4, 7])
def test_every_operation_between_processes_matches_the_oracle(rt, nprocs):
    from rocshmem_amd import launch
    rt.down()
    env = dict(os.environ, ROCSHMEM_EMU_SPIN_LIMIT=str(40_000_000))
    env.pop("ROCSHMEM_EMU_NPES", None)
    status, outs = launch.run(nprocs, WORKER, timeout=100, env=env, capture=True)
    assert status == 0, [o[-1500:] for o in outs]
    for pe, o in enumerate(outs):
        assert "ok %d" % pe in o, o[-1500:]


def test_processes_that_disagree_about_the_heap_are_stopped_at_init(rt):
    """A peer's barrier pads are found at the same offset as one's own, so a
    job whose processes bring different heap sizes must not get as far as a
    kernel: rocshmem_init compares the announced layouts and ends the job."""
    from rocshmem_amd import launch
    rt.down()
    env = dict(os.environ)
    env.pop("ROCSHMEM_EMU_NPES", None)
    status, outs = launch.run(2, WORKER + ["unequal-heaps"], timeout=60, env=env, capture=True)
    assert status != 0, outs
    text = "".join(outs)
    assert "disagree about the job" in text, text[-800:]
    assert "init returned" not in text
