"""One PE of a rendezvous test: started by tests/test_proc_group.py through the
launcher, talks to the other processes through the library's rendezvous entry
points only (no GPU)."""
import ctypes as C
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from rocshmem_amd import lib as L  # noqa: E402


def main():
    what = sys.argv[1]
    n = int(os.environ["ROCSHMEM_EMU_PROCS"])
    me = int(os.environ["ROCSHMEM_EMU_RANK"])
    lib = L.load()
    assert lib.procs_attach(os.environ["ROCSHMEM_EMU_RDV"].encode(), n, me) == 0
    # a second attach of the same process is refused
    assert lib.procs_attach(os.environ["ROCSHMEM_EMU_RDV"].encode(), n, me) == -1
    word = (C.c_uint64 * 2)()
    seen = (C.c_uint64 * 2)()
    if what == "rounds":
        rounds = int(sys.argv[2])
        for r in range(1, rounds + 1):
            word[0], word[1] = r, me * 1000003 + r
            assert lib.procs_publish(word, 16) == 0
            assert lib.procs_barrier(0, 1, n) == 0
            for q in range(n):
                assert lib.procs_fetch(q, seen, 16) == 0
                assert (seen[0], seen[1]) == (r, q * 1000003 + r), (me, q, r, seen[0], seen[1])
            assert lib.procs_barrier(0, 1, n) == 0
            # the two halves (even and odd ranks) meet on their own in between
            half = (n - (me & 1) + 1) // 2
            assert lib.procs_barrier(me & 1, 2, half) == 0
            if me & 1 == 0 and r % 7 == 0:
                time.sleep(0.002)  # the halves drift apart
        print("rounds ok", me)
    elif what == "late":
        # rank 1 never comes to the meeting: the others give up after the timeout
        if me == 1:
            time.sleep(3.0)
            print("stayed away")
        else:
            t0 = time.monotonic()
            rc = lib.procs_barrier(0, 1, n)
            print("gave up" if rc == -1 else "met", "%.1f" % (time.monotonic() - t0))
    elif what == "abort":
        if me == 1:
            time.sleep(0.3)
            assert lib.procs_abort_requested() == -1
            assert lib.procs_request_abort(7) == 0
            assert lib.procs_request_abort(9) == 0  # the first request stands
            print("asked")
        else:
            rc = lib.procs_barrier(0, 1, n)
            print("left" if rc == -1 else "met", lib.procs_abort_requested())
    elif what == "fail":
        if me == 2:
            sys.exit(5)
        rc = lib.procs_barrier(0, 1, n)  # never completes: rank 2 is gone
        print("barrier", rc)
    elif what == "bad":
        assert lib.procs_barrier(0, 0, n) == -1
        assert lib.procs_barrier(-1, 1, n) == -1
        assert lib.procs_barrier(0, 1, 1) == 0  # a set of one needs nobody
        big = (C.c_ubyte * 193)()
        assert lib.procs_publish(big, 193) == -1
        assert lib.procs_publish(big, 192) == 0
        assert lib.procs_fetch(n, big, 8) == -1
        print("bad ok")


if __name__ == "__main__":
    main()
