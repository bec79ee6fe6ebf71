"""The workloads of the benchmark that are otherwise only timed, at their
full size and checked: the headline put in its exact launch, the put_signal dispatch (4096 tokens per PE, rows of
7168 bf16, top-8-of-256 Zipf(1.1) routing) and 16 Mi int64 fetch_add onto 4096
counters.  Through the C entry points, default and NOSTORE contexts."""
import ctypes

import numpy as np
import pytest

from tests.test_gpu_amo_signal import Counters, check_fetch_chain, run_amo, zipf_routing

pytestmark = pytest.mark.gpu

P = 8
MiB = 1 << 20


@pytest.fixture(params=[0, 1], ids=["default_ctx", "nostore_ctx"])
def ctx_kind(request):
    return request.param


def test_headline_launch_moves_every_byte(rt, L, orc, ctx_kind, monkeypatch):
    """The benchmark's headline launch exactly: a 256 MiB message between two of
    8 slices in the spread layout (ROCSHMEM_EMU_SPREAD=1, 8 GiB per PE), one
    rocshmem_ctx_putmem_wg of a 4 KiB tile per work-group of 128 (65536
    work-groups), one quiet per work-group, on a ROCSHMEM_CTX_NOSTORE context
    and on a default one (src/ipc/context_ipc_device.cpp:109-125).  All 256 MiB
    and the bytes either side compared with the source on the host, and once
    more on the device with the compare the benchmark uses; a flipped byte is
    found by that compare."""
    monkeypatch.setenv("ROCSHMEM_EMU_SPREAD", "1")
    rt.down()
    l = rt.up(P, 8 << 30)
    assert l.pe_stride() >= 16 << 30
    n, tile, wg = 256 * MiB, 4096, 128
    src, dst = l.malloc(n), l.malloc(n + 4096)
    assert src and dst
    me, pe = 3, 4
    T = 4 * MiB
    host_tile = orc.fill_u8(T, 21, me)
    base = l.pe_ptr(src, me)
    rt.put_bytes(base, host_tile)
    done = T
    while done < n:
        assert l.putmem(base + done, base, done, me, me, None) == 0
        done *= 2
    l.fill(l.pe_ptr(dst, pe), 0x5A, n + 4096)
    before = l.set_ctx_options(ctx_kind)
    rc = l.rma(L.PUT, L.WG, l.pe_ptr(dst, me), l.pe_ptr(src, me), n, tile, me, pe, n // tile, wg, 1, None)
    l.set_ctx_options(before)
    assert rc == 0
    l.stream_sync(None)
    got = rt.get_bytes(l.pe_ptr(dst, pe), n + 4096)
    assert np.array_equal(got[:n].reshape(-1, T), np.broadcast_to(host_tile, (n // T, T)))
    assert (got[n:] == 0x5A).all()
    del got
    differing = ctypes.c_uint64(99)
    assert l.compare(l.pe_ptr(dst, pe), l.pe_ptr(src, me), n, ctypes.byref(differing), None) == 0
    assert differing.value == 0
    for at in (123456789, n - 1):
        l.fill(l.pe_ptr(dst, pe) + at, int(host_tile[at % T]) ^ 0xFF, 1)
    assert l.compare(l.pe_ptr(dst, pe), l.pe_ptr(src, me), n, ctypes.byref(differing), None) == 0
    assert differing.value == 2
    l.free(src)
    l.free(dst)
    rt.down()


def test_dispatch_put_signal_full_size(rt, L, orc, ctx_kind):
    """src/ipc/context_ipc_device.cpp:221-298 at the benchmark's shape: 262144
    rows of 14336 bytes leave the 8 PEs, two thirds of them for PE 0.  Rows are
    made on the device from a seeded 4 MiB tile per PE (the tile length is not a
    multiple of the row length, so consecutive rows differ).  After two
    dispatches in a row with running totals: every signal word equals twice the
    pair's row count, and every received row equals the packed source row, byte
    for byte."""
    rt.down()
    l = rt.up(P, 8 << 30)
    tokens, experts, topk, row = 4096, 256, 8, 7168 * 2
    counts, _ = zipf_routing(orc, P, tokens, experts, topk, 0)
    send_row = np.zeros((P, P), np.uint32)
    recv_row = np.zeros((P, P), np.uint32)
    for s in range(P):
        send_row[s] = np.r_[0, np.cumsum(counts[s])[:-1]]
    for d in range(P):
        recv_row[:, d] = np.r_[0, np.cumsum(counts[:, d])[:-1]]
    rows_out, rows_in = tokens * topk, int(counts.sum(0).max())
    assert int(counts.sum()) == P * rows_out and counts.sum(0)[0] > 0.5 * counts.sum()
    recv, send, sig = l.malloc(rows_in * row), l.malloc(rows_out * row), l.malloc(8 * P)
    assert recv and send and sig
    T = 4 * MiB
    tiles = [orc.fill_u8(T, 11, s) for s in range(P)]
    for s in range(P):
        base = l.pe_ptr(send, s)
        rt.put_bytes(base, tiles[s])
        done = T
        while done < rows_out * row:
            step = min(done, rows_out * row - done)
            assert l.putmem(base + done, base, step, s, s, None) == 0
            done += step
    l.stream_sync(None)
    expect = l.dev_alloc(8 * P * P)
    l.fill(expect, 0, 8 * P * P)
    assert l.fill_every_pe(sig, 0, 8 * P, None) == 0
    tabs = [np.ascontiguousarray(a, np.uint32) for a in (counts, send_row, recv_row)]
    before = l.set_ctx_options(ctx_kind)
    # (rows per call, work-group size): the shape bench.py times, and a second one
    rows_per_call, wg_size = (7, 1024) if ctx_kind else (16, 256)
    try:
        for _ in range(2):
            assert l.dispatch_put_signal(recv, send, sig, tabs[0].ctypes.data, tabs[1].ctypes.data,
                                         tabs[2].ctypes.data, row, rows_per_call, wg_size, expect,
                                         None) == 0
        l.stream_sync(None)
    finally:
        l.set_ctx_options(max(before, 0))
    for d in range(P):
        sigs = rt.get_bytes(l.pe_ptr(sig, d), 8 * P, np.uint64)
        assert np.array_equal(sigs, 2 * counts[:, d].astype(np.uint64)), d
        got = rt.get_bytes(l.pe_ptr(recv, d), int(counts[:, d].sum()) * row)
        for s in range(P):
            a, b, n = int(send_row[s, d]) * row, int(recv_row[s, d]) * row, int(counts[s, d]) * row
            pos = 0
            while pos < n:  # the source is the tile repeated: compare tile by tile
                first = (a + pos) % T
                m = min(T - first, n - pos)
                assert np.array_equal(got[b + pos:b + pos + m], tiles[s][first:first + m]), (s, d, pos)
                pos += m
        del got
    l.dev_free(expect)
    for x in (send, recv, sig):
        l.free(x)
    rt.down()


@pytest.mark.parametrize("dist", ["uniform", "zipf"])
def test_fetch_add_16mi_on_4096_counters(rt, L, orc, dist, ctx_kind):
    """src/ipc_policy.hpp:69-99 at the benchmark's size and launch shape (4096
    work-groups of 256): the final histogram is exact, and on the hottest
    counter and 32 sampled ones the fetched values are a serialisation
    0, 1, 2, ... of the increments (each value exactly once)."""
    l = rt.up(P, 1 << 30)
    K, n = 4096, 1 << 24
    if dist == "uniform":
        ids = (orc.fill_u64(n, 0, 1) % K).astype(np.uint32)
    else:
        ids = orc.fill_zipf_u32(n, 0, 2, K, 1.1)
    ctr = Counters(rt, l, K // P, np.int64)
    before = l.set_ctx_options(ctx_kind)
    try:
        fetched = run_amo(rt, l, L, L.AMO_FETCH_ADD, "LONG", ctr, ids, n_wgs=4096, wg=256)
    finally:
        l.set_ctx_options(max(before, 0))
    hist = np.bincount(ids, minlength=K)
    assert np.array_equal(ctr.read_all(), hist)
    hottest = int(hist.argmax())
    sample = np.unique(np.r_[hottest, np.random.default_rng(5).integers(0, K, 32)])
    for c in sample:
        f = np.sort(fetched[ids == c])
        assert np.array_equal(f, np.arange(hist[c], dtype=np.int64)), int(c)
    keep = np.isin(ids, sample)
    check_fetch_chain(ids[keep], fetched[keep], np.ones(int(keep.sum()), np.int64), 0)
    ctr.free()
