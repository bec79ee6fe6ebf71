"""The rendezvous that lets one process per PE find each other and meet
(rocshmem_amd/csrc/proc_group.cpp) and the launcher that starts them
(rocshmem_amd/launch.py), on the CPU.  The reference's counterpart is its MPI
bootstrap (src/ipc_policy.cpp:34-118, src/ipc/backend_ipc.cpp:274-357)."""
import os
import sys
import time

import pytest

from rocshmem_amd import launch
from rocshmem_amd import lib as L

WORKER = [sys.executable, os.path.join(os.path.dirname(os.path.abspath(__file__)), "procs_worker.py")]

pytestmark = pytest.mark.skipif(not os.path.exists(L.LIB_PATH), reason="library not built")


def test_file_size_covers_the_shared_state():
    n = launch.rendezvous_bytes()
    # 64 header bytes, 128 barrier slots of 16, 64 publish areas of 8 + 192
    assert n == 64 + 128 * 16 + 64 * 200


@pytest.mark.parametrize("nprocs", [2, 5, 8])
def test_meetings_and_publish_areas(nprocs):
    status, outs = launch.run(nprocs, WORKER + ["rounds", "300"], timeout=60, capture=True)
    assert status == 0, outs
    for r, o in enumerate(outs):
        assert "rounds ok %d" % r in o, o


def test_a_meeting_gives_up_after_the_timeout():
    env = dict(os.environ, ROCSHMEM_EMU_RDV_TIMEOUT_S="1")
    t0 = time.monotonic()
    status, outs = launch.run(3, WORKER + ["late"], timeout=30, env=env, capture=True)
    assert status == 0, outs
    assert "gave up 1." in outs[0] and "gave up 1." in outs[2], outs
    assert "stayed away" in outs[1]
    assert time.monotonic() - t0 < 15


def test_a_request_to_end_the_job_reaches_waiting_processes():
    status, outs = launch.run(3, WORKER + ["abort"], timeout=30, capture=True)
    assert status == 0, outs
    assert "left 7" in outs[0] and "left 7" in outs[2], outs
    assert "asked" in outs[1]


def test_launcher_returns_the_first_failure_and_ends_the_rest():
    t0 = time.monotonic()
    status, outs = launch.run(4, WORKER + ["fail"], timeout=30, capture=True)
    assert status == 5, outs
    assert time.monotonic() - t0 < 15  # did not wait for the 30 s limit
    for r in (0, 1, 3):
        assert "barrier 0" not in outs[r]


def test_launcher_timeout():
    status, _ = launch.run(2, [sys.executable, "-c", "import time; time.sleep(30)"], timeout=1.0, capture=True)
    assert status == 124


def test_bad_arguments_are_refused():
    status, outs = launch.run(2, WORKER + ["bad"], timeout=30, capture=True)
    assert status == 0, outs
    with pytest.raises(ValueError):
        launch.run(0, WORKER + ["bad"])
    with pytest.raises(ValueError):
        launch.run(17, WORKER + ["bad"])
