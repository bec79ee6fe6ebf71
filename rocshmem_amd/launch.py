"""Start a program as P processes, one per PE, on one GPU:

    python -m rocshmem_amd.launch -n P [--timeout SECONDS] prog [args...]

what `mpirun -n P prog` is to the reference.  The launcher creates the
rendezvous file (zero-filled, in /dev/shm), gives every process its rank
through ROCSHMEM_EMU_PROCS / ROCSHMEM_EMU_RANK / ROCSHMEM_EMU_RDV, waits for
all of them and returns the first non-zero exit status; when a process fails
or the time runs out it ends the others.  It never touches the GPU itself.
"""
import argparse
import os
import signal
import subprocess
import sys
import tempfile
import time

MAX_PROCS = 16  # a one-GPU box allows at most 16 processes on its card


def rendezvous_bytes():
    """Size of the rendezvous file, asked of the library (loading it touches no GPU)."""
    from . import lib
    return lib.load().procs_file_bytes()


def run(nprocs, argv, timeout=300.0, env=None, capture=False):
    """Runs argv as nprocs PEs.  Returns (status, outputs): the first non-zero
    exit status (124 after a timeout) and, with capture, each rank's combined
    output."""
    if not 1 <= nprocs <= MAX_PROCS:
        raise ValueError("between 1 and %d processes" % MAX_PROCS)
    fd, path = tempfile.mkstemp(prefix="rocshmem_rdv_", dir="/dev/shm" if os.path.isdir("/dev/shm") else None)
    procs, outs = [], []
    try:
        os.ftruncate(fd, rendezvous_bytes())
        os.close(fd)
        base = dict(os.environ if env is None else env)
        base.update(ROCSHMEM_EMU_PROCS=str(nprocs), ROCSHMEM_EMU_RDV=path)
        base.setdefault("ROCSHMEM_EMU_RDV_TIMEOUT_S", str(max(5, int(timeout))))
        for rank in range(nprocs):
            e = dict(base, ROCSHMEM_EMU_RANK=str(rank))
            out = tempfile.TemporaryFile() if capture else None
            outs.append(out)
            procs.append(subprocess.Popen(argv, env=e, stdout=out, stderr=subprocess.STDOUT if capture else None))
        deadline = time.monotonic() + timeout
        status = 0
        left = set(range(nprocs))
        while left:
            for r in sorted(left):
                rc = procs[r].poll()
                if rc is not None:
                    left.discard(r)
                    if rc != 0 and status == 0:
                        status = rc if rc > 0 else 128 - rc
            if status != 0 and left:
                time.sleep(1.0)  # the others leave at their next meeting; then they are ended
                break
            if time.monotonic() > deadline:
                status = status or 124
                break
            time.sleep(0.01)
        for r in left:
            if procs[r].poll() is None:
                procs[r].send_signal(signal.SIGTERM)
        for r in left:
            try:
                procs[r].wait(5)
            except subprocess.TimeoutExpired:
                procs[r].kill()
                procs[r].wait()
        texts = []
        for out in outs:
            if out is None:
                texts.append("")
            else:
                out.seek(0)
                texts.append(out.read().decode(errors="replace"))
                out.close()
        return status, texts
    finally:
        # whatever ended the wait (an exception included), no PE outlives its launcher
        for proc in procs:
            if proc.poll() is None:
                proc.kill()
                proc.wait()
        try:
            os.unlink(path)
        except OSError:
            pass


def main():
    ap = argparse.ArgumentParser(prog="python -m rocshmem_amd.launch")
    ap.add_argument("-n", type=int, required=True, help="number of PEs (processes)")
    ap.add_argument("--timeout", type=float, default=300.0)
    ap.add_argument("prog", nargs=argparse.REMAINDER)
    a = ap.parse_args()
    if not a.prog:
        ap.error("no program given")
    status, _ = run(a.n, a.prog, a.timeout)
    sys.exit(status)


if __name__ == "__main__":
    main()
