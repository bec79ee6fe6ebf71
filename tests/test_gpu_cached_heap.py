"""The library on a CACHED heap (ROCSHMEM_EMU_HEAP_CACHED=1: plain hipMalloc,
what the reference's IPC build uses, src/memory/heap_type.hpp:41-51).  On the
default uncached heap no line of the heap is ever held in an L2, so the
ordering tests pass whether or not the library's releases and acquires are
right; here a consumer's L2 does hold stale lines of the destination from the
round before, and a producer's plain stores do sit dirty in its L2.  The
ordering, barrier, all-reduce, alltoall and dispatch tests of the other modules
run again in this mode, through the C entry points, against the same oracle."""
import os

import numpy as np
import pytest

from tests import test_gpu_amo_signal as amo_tests
from tests import test_gpu_collectives as coll_tests
from tests import test_gpu_reduce as reduce_tests
from tests import test_gpu_rma as rma_tests

pytestmark = pytest.mark.gpu

P, HEAP = 8, 1 << 30


@pytest.fixture(scope="module")
def cached(rt, L):
    rt.down()
    os.environ["ROCSHMEM_EMU_HEAP_CACHED"] = "1"
    try:
        l = rt.up(P, HEAP)
        assert l.heap_is_uncached() == 0
        yield l
    finally:
        rt.down()
        os.environ.pop("ROCSHMEM_EMU_HEAP_CACHED", None)


@pytest.fixture(scope="module")
def env(rt, L, orc, cached):
    l = cached
    size = 8 << 20
    src, dst = l.malloc(size), l.malloc(size)
    assert src and dst
    host = orc.fill_u8(size, 0, 11)
    rt.put_bytes(src, host)
    yield dict(l=l, src=src, dst=dst, size=size, host=host)
    l.free(src)
    l.free(dst)


@pytest.mark.parametrize("with_signal", [0, 1, 2, 3, 4, 5])
@pytest.mark.parametrize("ctx_options", [0, 1])
@pytest.mark.parametrize("nbytes,pairs,wg", [(4096, 1, 64), (65536, 16, 256), (1 << 20, 64, 1024),
                                             (262144 + 4, 128, 256)])
def test_put_quiet_flag_seen_in_order(rt, L, env, ctx_options, with_signal, nbytes, pairs, wg):
    """Payload before flag inside one kernel, 20 rounds with a new pattern
    each: the consumer's XCD read the previous round's payload, so it finds the
    new one only if its wait acquires and the producer's quiet / signal
    releases."""
    assert env["l"].heap_is_uncached() == 0
    if with_signal >= 4 and nbytes > 65536:
        nbytes = 32768 + 4  # the LDS-staged modes hold the message in one work-group's LDS
    rma_tests.test_put_quiet_flag_seen_in_order(rt, L, env, ctx_options, with_signal, nbytes, pairs, wg)


@pytest.mark.parametrize("gran_name,wg_size,n,ctx_options", [("WG", 256, 4099, 0), ("WG", 256, 4099, 1),
                                                            ("WAVE", 64, 1000, 1), ("THREAD", 64, 100, 0)])
def test_local_buffer_in_lds(rt, L, orc, env, gran_name, wg_size, n, ctx_options):
    rma_tests.test_local_buffer_in_lds(rt, L, orc, env, gran_name, wg_size, n, ctx_options)


@pytest.mark.parametrize("gran", ["THREAD", "WAVE", "WG"])
def test_copies_with_guards(rt, L, orc, env, gran):
    for op in ("PUT", "GET"):
        for n, soff, doff in [(0, 0, 0), (1, 3, 5), (777, 1, 9), (100001, 7, 2)]:
            rma_tests.run_case(rt, L, orc, env, getattr(L, op), getattr(L, gran), n, soff, doff, 2, 128)


@pytest.mark.parametrize("fn", ["BARRIER_ALL", "SYNC_ALL", "TEAM_SYNC"])
def test_barriers_order_puts(rt, L, cached, fn):
    coll_tests.test_barriers_order_puts(rt, L, fn)
    assert cached.heap_is_uncached() == 0


@pytest.mark.parametrize("dtype_name,op_name,n", [("FLOAT", "SUM", 100003), ("LONG", "XOR", 4099),
                                                  ("BF16", "SUM", 70001)])
@pytest.mark.parametrize("mode", ["wg", "to_all"])
def test_all_reduce(rt, L, orc, cached, dtype_name, op_name, n, mode):
    """Sources written by the host's copies, then reduced twice in a row with
    fresh inputs: the second pass re-reads lines the first left in the L2s."""
    for seed in (0, 1):
        reduce_tests.check_all(rt, cached, orc, L, P, dtype_name, op_name, n, mode, seed=seed)
    assert cached.heap_is_uncached() == 0


@pytest.mark.parametrize("kind", ["alltoall", "broadcast", "fcollect"])
@pytest.mark.parametrize("mode", ["wg", "grid"])
def test_block_moves(rt, L, orc, cached, kind, mode):
    for seed in (0, 1):
        coll_tests.run_move(rt, cached, L, orc, kind, mode, 4, 5001, list(range(P)), cached.team_world(),
                            root=3, seed=seed)
    assert cached.heap_is_uncached() == 0


@pytest.mark.parametrize("rows_per_call", [7, 64])
def test_dispatch_put_signal(rt, L, orc, cached, rows_per_call):
    """The reduced-size MoE dispatch: receivers wait on put_signal totals and
    the host compares every received row."""
    amo_tests.test_dispatch_put_signal(rt, L, orc, rows_per_call)
    assert cached.heap_is_uncached() == 0


@pytest.mark.parametrize("nbytes,pairs", [(8, 1), (4096, 8), (65536, 2)])
def test_pingpong(rt, L, orc, cached, nbytes, pairs):
    amo_tests.test_pingpong(rt, L, orc, nbytes, pairs)
    assert cached.heap_is_uncached() == 0


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_polling_with_gets_sees_the_put(rt, L, env, kind):
    rma_tests.test_polling_with_gets_sees_the_put(rt, L, env, 0, kind, 64, 256)
