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
