#!/usr/bin/env python3
"""Throughput of the symmetric-heap data path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

Prints ONE JSON line.  The headline (`metric`/`value`) is the bulk putmem
workload of BASELINE.json's configs[1]: one 256 MiB message between two of
P=8 PE slices of one symmetric heap, moved by all CUs through the device API
(rocshmem_ctx_putmem_wg, one 4 KiB tile per work-group of 128, on a context
created with ROCSHMEM_CTX_NOSTORE); a step is one such message and `value`
counts algorithmic bytes (N read + N written).  The same workload through a
default context and through the host-side rocshmem_putmem, and every other
configuration (all-reduce, alltoall, put_signal dispatch, atomics, ping-pong),
are carried as scalar keys of `roofline` — one figure per configuration first,
then the same in the packed default layout and on a cached heap, then the rest
— and in full under `all_configs`, beside a CPU baseline (the oracle's
threaded routines on the host cores).  After the timed loops the last
destination of the headline put is compared with its source on the device
(`roofline.verified`).

The run has three bring-ups of the library: slices spread over half of the
device memory (ROCSHMEM_EMU_SPREAD=1, 8 GiB per PE: every configuration), the
default packed layout (1 GiB per PE: the layout a plain rocshmem_init gives),
and a cached heap (ROCSHMEM_EMU_HEAP_CACHED=1: what a consumer that re-reads
symmetric data gains, and what ordering then costs).  The CPU baseline's legs
run between them.

Inputs are resident in HBM before any timed region starts.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X, published
# HBM bytes one launch of the headline kernel moves, from FETCH_SIZE + WRITE_SIZE
# under rocprofv3 --pmc (profiles/putmem_wg_tiled_256MiB_hbm_traffic.txt).
PUT_TRAFFIC_BYTES = 536952840
P = 8
MiB = 1 << 20


# Contexts the device-API configurations run through: default, and created with
# ROCSHMEM_CTX_NOSTORE (completion without the L2 write-back, relaxed AMOs).
CTX_KINDS = (("default_ctx", 0), ("nostore_ctx", 1))


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--quick", action="store_true", help="headline only, no CPU baseline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--with-processes", action="store_true",
                    help="also run the headline between two processes (one process per PE, HIP IPC); "
                         "the record gains all_configs.process_per_pe_2_processes")
    ap.add_argument("--process-leg", action="store_true",
                    help="(internal) run as one PE of a two-process job started by rocshmem_amd.launch")
    ap.add_argument("--profile-kernels", action="store_true",
                    help="a short run for rocprofv3: a few launches each of the headline put, the "
                         "fp32 sum all-reduce, the alltoall and the dispatch, and three 256 MiB "
                         "hipMemcpy calls to calibrate the byte counters; prints the launch counts")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run three 256 MiB device-to-device hipMemcpy calls (the HIP "
                         "runtime's copy kernel) for calibrating FETCH_SIZE / WRITE_SIZE")
    return ap.parse_args()


class Bench:
    def __init__(self, L):
        self.L = L
        self.l = L.load()
        self.probes = L.load_probes()
        self.timer = self.l.timer_create()

    def time_ms(self, fn, steps, warmup):
        """Average milliseconds per call of fn over `steps` calls, HIP events
        on the stream the kernels are launched on (the null stream)."""
        l = self.l
        for _ in range(warmup):
            fn()
        l.stream_sync(None)
        l.timer_start(self.timer, None)
        for _ in range(steps):
            fn()
        l.timer_stop(self.timer, None)
        return l.timer_elapsed_ms(self.timer) / steps

    def fill_random(self, ptr, nbytes, pe, seed, kind="u8"):
        """Random payload resident on the device: a seeded 4 MiB tile uploaded
        once and doubled in place by on-device copies.  kind: "u8" uniform
        bytes, "f32" / "bf16" N(0,1) values (bf16 by truncating the fp32)."""
        l = self.l
        tile = min(nbytes, 4 * MiB)
        rng = np.random.default_rng(seed)
        if kind == "u8":
            host = rng.integers(0, 256, tile, dtype=np.uint8)
        else:
            f = rng.standard_normal(tile // (4 if kind == "f32" else 2), dtype=np.float32)
            host = f if kind == "f32" else (f.view(np.uint32) >> 16).astype(np.uint16)
        l.copy_in(ptr, host.ctypes.data, tile)
        done = tile
        while done < nbytes:
            step = min(done, nbytes - done)
            assert l.putmem(ptr + done, ptr, step, pe, pe, None) == 0
            done += step
        l.stream_sync(None)


# Launch shapes of the tiled device-API put, from sweeps over work-group size
# {64..1024} x tile {1..16 vectors per lane} x {one tile per work-group, 256..2048
# work-groups that loop} on MI355X:
#   NOSTORE context: one 4 KiB tile per work-group of 128 (each lane loads two
#     vectors, stores them, and the work-group leaves) - the closest a
#     putmem_wg loop gets to the one-vector work-groups of the bulk kernel;
#     with more in flight per CU the rate drops again (four vectors per lane:
#     -3 %, eight: -5 %);
#   default context: every work-group ends in a quiet, an L2 write-back of
#     35-70 ns for its XCD, so fewer work-groups that loop: 1024 work-groups
#     of 1024 lanes, 48 KiB tiles (three vectors per lane and call).
PUT_SHAPES = {"nostore_ctx": (128, 4096, None), "default_ctx": (1024, 49152, 1024)}


def headline(b, steps, warmup):
    """configs[1]: bulk putmem, 256 MiB messages, all CUs.  Step k sends from
    PE k%8 to PE (k+1)%8, so consecutive steps touch different 256 MiB buffers
    (4 GiB in rotation): nothing is served from the 256 MB memory-side cache and
    the rate is what HBM sustains."""
    l, L = b.l, b.L
    n = 256 * MiB
    src, dst = l.malloc(n), l.malloc(n)
    assert src and dst
    for p in range(P):
        b.fill_random(l.pe_ptr(src, p), n, p, 1 + p)
    srcs = [l.pe_ptr(src, p) for p in range(P)]
    dsts = [l.pe_ptr(dst, p) for p in range(P)]
    k = [0]

    def rotating(fn):
        def step():
            me = k[0] % P
            k[0] += 1
            assert fn(me, (me + 1) % P) == 0
        return step

    def tiled_put(kind):
        wg, tile, n_wgs = PUT_SHAPES[kind]
        n_wgs = n_wgs or n // tile
        return rotating(lambda me, pe: l.rma(L.PUT, L.WG, dsts[me], srcs[me], n, tile, me, pe, n_wgs, wg,
                                             1, None))

    out = {"bytes_per_step": 2 * n}

    def moves_every_byte(step):
        """What a timed loop moved: every destination is cleared, one more step
        runs, and its destination is compared with its source on the device."""
        for p in range(P):
            l.fill(dsts[p], 0, n)
        step()
        me = (k[0] - 1) % P
        bad = C.c_uint64(1)
        assert l.compare(dsts[(me + 1) % P], srcs[me], n, C.byref(bad), None) == 0
        return bad.value == 0

    # The host-side rocshmem_putmem / getmem (one whole-GPU kernel per message).
    # Measured first: whatever runs first in the process comes out about 3 %
    # low (the GPU's first milliseconds of work run below its sustained rate,
    # whichever kernel they are spent on), and these two are timed again for
    # the curve below.
    for _ in range(2):
        out["host_putmem_gbs"] = 2 * n / b.time_ms(
            rotating(lambda me, pe: l.putmem(dsts[me], srcs[me], n, me, pe, None)), steps, warmup) / 1e6
        out["host_getmem_gbs"] = 2 * n / b.time_ms(
            rotating(lambda me, pe: l.getmem(dsts[me], srcs[me], n, me, pe, None)), steps, warmup) / 1e6
    # The device API, rocshmem_ctx_putmem_wg from every CU: the headline.
    l.set_ctx_options(1)
    out["ms"] = b.time_ms(tiled_put("nostore_ctx"), steps, warmup)
    out["gbs"] = 2 * n / out["ms"] / 1e6
    out["verified"] = moves_every_byte(tiled_put("nostore_ctx"))
    l.set_ctx_options(0)
    out["default_ctx_gbs"] = 2 * n / b.time_ms(tiled_put("default_ctx"), steps, warmup) / 1e6
    out["verified"] = moves_every_byte(tiled_put("default_ctx")) and out["verified"]
    # rocshmem_ctx_getmem_wg from every CU, the shape of the headline put
    l.set_ctx_options(1)
    wg, tile, _ = PUT_SHAPES["nostore_ctx"]
    out["getmem_wg_gbs"] = 2 * n / b.time_ms(
        rotating(lambda me, pe: l.rma(L.GET, L.WG, dsts[me], srcs[me], n, tile, me, pe, n // tile, wg, 1,
                                      None)), steps, warmup) / 1e6
    l.set_ctx_options(0)
    if b.quick or b.short:
        l.free(src)
        l.free(dst)
        return out
    # The bandwidth curve, 8 B .. 256 MiB (26 sizes).  One work-group of 64, 256
    # and 1024 threads issuing rocshmem_putmem_wg / getmem_wg: the call is
    # repeated inside the kernel (as the reference's testers loop inside theirs)
    # so the launch does not count; small messages are then re-read from cache.
    # All CUs: the host-initiated copy, one launch per message, launch included.
    curve = {}
    reps = max(3, min(steps, 10))
    for e in range(3, 29):
        m = 1 << e
        inner = 200 if e <= 16 else (20 if e <= 24 else 2)
        point = {}
        for threads in (64, 256, 1024):
            t = b.time_ms(rotating(lambda me, pe: l.rma(L.PUT, L.WG, dsts[me], srcs[me], m, 0, me, pe,
                                                        1, threads, inner, None)), 3, 1) / inner
            point["putmem_wg_1wg_%dthr_gbs" % threads] = round(2 * m / t / 1e6, 3)
        t = b.time_ms(rotating(lambda me, pe: l.rma(L.GET, L.WG, dsts[me], srcs[me], m, 0, me, pe,
                                                    1, 1024, inner, None)), 3, 1) / inner
        point["getmem_wg_1wg_1024thr_gbs"] = round(2 * m / t / 1e6, 3)
        tg = b.time_ms(rotating(lambda me, pe: l.putmem(dsts[me], srcs[me], m, me, pe, None)), reps, 2)
        tget = b.time_ms(rotating(lambda me, pe: l.getmem(dsts[me], srcs[me], m, me, pe, None)), reps, 2)
        point["putmem_all_cus_gbs"] = round(2 * m / tg / 1e6, 3)
        point["getmem_all_cus_gbs"] = round(2 * m / tget / 1e6, 3)
        curve[str(m)] = point
    out["curve"] = curve
    # One-directional ceilings of the memory system, same buffers and rotation:
    # a copy that reads N and writes N cannot beat 2 / (1/read + 1/write).
    t_rd = b.time_ms(rotating(lambda me, pe: b.probes.hbm_probe(0, srcs[me], n, None)), steps, warmup)
    t_wr = b.time_ms(rotating(lambda me, pe: b.probes.hbm_probe(1, dsts[pe], n, None)), steps, warmup)
    rd, wr = n / t_rd / 1e6, n / t_wr / 1e6
    out["ceilings"] = {"read_only_gbs": round(rd, 1), "write_only_gbs": round(wr, 1),
                       "copy_bound_gbs": round(2 / (1 / rd + 1 / wr), 1)}
    # What one agent-scope release (the write-back in a default context's quiet)
    # costs while the copy runs: 1024 work-groups of 256, 16 KiB tiles.
    rp = {}
    for mode in (0, 1, 2):
        rp[mode] = b.time_ms(rotating(lambda me, pe: b.probes.release_probe(mode, dsts[pe], srcs[me], n, 16384,
                                                                     1024, 256, None)), 5, 2)
    out["release_ns_each_per_tile"] = round((rp[2] - rp[0]) * 1e6 / (n // 16384), 1)
    out["release_ns_each_at_end"] = round((rp[1] - rp[0]) * 1e6 / 1024, 1)
    # The tiled put of the headline in other shapes, both kinds of context.
    tiled = {}
    for name, opt in CTX_KINDS:
        l.set_ctx_options(opt)
        for wg, tile, n_wgs in ((256, 16384, None), (512, 32768, 256), (1024, 65536, 1024),
                                (1024, 65536, 4096)):
            t = b.time_ms(rotating(lambda me, pe: l.rma(L.PUT, L.WG, dsts[me], srcs[me], n, tile, me, pe,
                                                        n_wgs or n // tile, wg, 1, None)), 5, 2)
            tiled["%s_wg%d_tile%d_%dwgs_gbs" % (name, wg, tile, n_wgs or n // tile)] = round(2 * n / t / 1e6, 1)
    l.set_ctx_options(0)
    out["tiled"] = tiled
    l.free(src)
    l.free(dst)
    return out


# Launch shape of the many-teams device all-reduce (teams, lanes per work-group,
# elements per call; 0 = one contiguous slice per team), from sweeps on MI355X.
TEAM_SHAPE = (32, 256, 0)


def to_all_configs(b, steps, warmup, which=("int64_xor", "fp32_sum", "fp32_max", "bf16_sum"), device_api=True):
    """configs[2]: all-reduce over P=8 slices x 64 Mi elements; and configs[0],
    the int32 sum over P=2 x 1 Mi, as the same host call on an active set of
    two PEs."""
    l, L = b.l, b.L
    n = 1 << 26
    res = {}
    table = {"int64_xor": (L.LONG, L.XOR, 8), "fp32_sum": (L.FLOAT, L.SUM, 4),
             "fp32_max": (L.FLOAT, L.MAX, 4), "bf16_sum": (L.BF16, L.SUM, 2)}
    # largest buffers first: freed blocks are never merged by the allocator
    for name in which:
        dt, op, es = table[name]
        src, dst = l.malloc(n * es), l.malloc(n * es)
        assert src and dst, name
        kind = {L.FLOAT: "f32", L.BF16: "bf16"}.get(dt, "u8")
        for p in range(P):
            b.fill_random(l.pe_ptr(src, p), n * es, p, 10 + p, kind)
        ms = b.time_ms(lambda: l.to_all(dt, op, dst, src, n, 0, 0, P, None), max(10, steps), 5)
        alg = 2 * P * n * es
        res[name] = {"ms": round(ms, 4), "gbs": round(alg / ms / 1e6, 1),
                     "frac": round(alg / ms / 1e6 / HBM_PEAK_GBS, 4)}
        if name == "fp32_sum" and device_api:
            # configs[0]: int32 sum, P=2 x 1 Mi elements (the reference's CPU-runnable
            # case, src/rocshmem.cpp:974-980), through the same host call
            m = 1 << 20
            ms1 = b.time_ms(lambda: l.to_all(L.INT, L.SUM, dst, src, m, 0, 0, 2, None), 200, 20)
            res["int32_sum_P2_1Mi"] = {"ms": round(ms1, 5), "gbs": round(2 * 2 * m * 4 / ms1 / 1e6, 1)}
            # The device call rocshmem_ctx_float_sum_wg_reduce: by its contract ONE
            # work-group per PE takes part, so 8 of the 256 CUs do all the work.
            ms = b.time_ms(lambda: l.wg_reduce(dt, op, l.team_world(), dst, src, n, 1024, None), 3, 1)
            res["fp32_sum_wg_reduce_one_wg_per_pe"] = {"ms": round(ms, 4),
                                                       "gbs": round(alg / ms / 1e6, 1)}
            # ... and the way the reference's testers scale it: one team per
            # work-group, many teams x 8 PEs at once, the call repeated four
            # times inside the kernel.  Through the entry point that allocates
            # nothing, so no hipMalloc sits inside the timed call.
            NT, wg, chunk = TEAM_SHAPE
            inner = 4
            teams = (C.c_void_p * NT)()
            for t in range(NT):
                h = C.c_void_p()
                assert l.team_split_strided(l.team_world(), 0, 1, P, C.byref(h)) == 0 and h.value
                teams[t] = h.value
            for cname, opt in CTX_KINDS:
                l.set_ctx_options(opt)
                ms = b.time_ms(lambda: l.wg_reduce_teams_static(dt, op, teams, NT, dst, src, n, chunk, wg,
                                                                inner, None), 3, 1) / inner
                res["fp32_sum_wg_reduce_teams_" + cname] = {
                    "ms": round(ms, 4), "gbs": round(alg / ms / 1e6, 1),
                    "frac": round(alg / ms / 1e6 / HBM_PEAK_GBS, 4), "teams": NT, "wg": wg,
                    "chunk_elems": chunk}
            l.set_ctx_options(0)
            for t in range(NT):
                l.team_destroy(teams[t])
        l.free(src)
        l.free(dst)
    return res


def message_rates(b, steps):
    """Two thirds of the reference's test matrix is thread- and
    wavefront-granularity traffic (scripts/functional_tests/driver.sh:142-218;
    src/ipc/context_ipc_device.cpp:62-88,137-164): rocshmem_putmem of 8 B, 64 B
    and 4 KiB per lane and rocshmem_putmem_wave of 512 B and 4 KiB per
    wavefront from every CU, with lanes (wavefronts) that continue one another
    and with their messages scattered, on both kinds of context."""
    l, L = b.l, b.L
    cap = 1 << 30
    src, dst = l.malloc(cap), l.malloc(cap)
    assert src and dst
    b.fill_random(l.pe_ptr(src, 0), cap, 0, 77)
    res = {}
    for gran, gname, msg in ((L.THREAD, "putmem", 8), (L.THREAD, "putmem", 64), (L.THREAD, "putmem", 4096),
                             (L.WAVE, "putmem_wave", 512), (L.WAVE, "putmem_wave", 4096)):
        count = min(1 << 24, cap // msg)
        groups_per_wg = 256 if gran == L.THREAD else 4
        n_wgs = max(256, min(8192, count // groups_per_wg))
        for scattered in (0, 1):
            for cname, opt in CTX_KINDS:
                # thread-level puts also without the coalescing front end (on by
                # default), which looks for one run across the wavefront before
                # every call
                for coalesce in ((1, 0) if gran == L.THREAD else (1,)):
                    l.set_ctx_options(opt)
                    l.set_coalesce_puts(coalesce)
                    ms = b.time_ms(lambda: l.rma_messages(L.PUT, gran, l.pe_ptr(dst, 0), l.pe_ptr(src, 0),
                                                          count * msg, msg, scattered, 0, 1, n_wgs, 256, 1,
                                                          None), max(3, steps // 10), 1)
                    key = "%s_%dB_%s_%s%s" % (gname, msg, "scattered" if scattered else "contiguous", cname,
                                              "" if coalesce else "_no_coalescing")
                    res[key] = {"ms": round(ms, 4), "msgs": count, "mmsg_per_s": round(count / ms / 1e3, 1),
                                "gbs": round(2 * count * msg / ms / 1e6, 1)}
    l.set_coalesce_puts(1)
    l.set_ctx_options(0)
    l.free(src)
    l.free(dst)
    return res


def reuse_config(b, steps):
    """What a consumer that re-reads symmetric data gets from the caches: a
    256 MiB symmetric buffer read four times, tile by tile (each 64 KiB tile
    four times in a row by its work-group of 1024 lanes, one work-group per
    CU), against one pass.  A tile is larger than a CU's vector L1, and the
    tiles in flight on an XCD (32 x 64 KiB) fit its 4 MiB L2: on cached memory
    the later passes are L2 hits."""
    l = b.l
    n = 256 * MiB
    buf = l.malloc(n)
    assert buf
    b.fill_random(buf, n, 0, 91)
    res = {}
    for passes in (1, 4):
        ms = b.time_ms(lambda: b.probes.reuse_probe(buf, n, 64 << 10, passes, 256, 1024, None),
                       max(5, steps // 4), 2)
        res["read_x%d_gbs" % passes] = round(passes * n / ms / 1e6, 1)
    l.free(buf)
    return res


def alltoall_config(b, steps):
    """configs[4] part 1: alltoall, 512 tokens x 7168 bf16 per PE pair; fcollect
    and broadcast of the same block beside it."""
    l = b.l
    blk = 512 * 7168 * 2
    src, dst = l.malloc(P * blk), l.malloc(P * blk)
    assert src and dst
    for p in range(P):
        b.fill_random(l.pe_ptr(src, p), P * blk, p, 30 + p)
    n = max(10, steps)

    def entry(ms, alg):
        return {"ms": round(ms, 4), "gbs": round(alg / ms / 1e6, 1),
                "frac": round(alg / ms / 1e6 / HBM_PEAK_GBS, 4)}

    res = entry(b.time_ms(lambda: l.alltoallmem(l.team_world(), dst, src, blk, None), n, 5),
                2 * P * P * blk)
    # every block is read once and written P times (P-1 for the broadcast)
    res["fcollect_same_block"] = entry(
        b.time_ms(lambda: l.fcollectmem(l.team_world(), dst, src, blk, None), n, 5),
        (P + P * P) * blk)
    res["broadcast_P_blocks_from_pe0"] = entry(
        b.time_ms(lambda: l.broadcastmem(l.team_world(), dst, src, P * blk, 0, None), n, 5),
        P * P * blk)
    l.free(src)
    l.free(dst)
    return res


def zipf_table(K, s):
    w = 1.0 / np.power(np.arange(1, K + 1, dtype=np.float64), s)
    return np.cumsum(w / w.sum())


def dispatch_config(b, steps, shapes=((7, 1024),)):
    """configs[4] part 2: put_signal dispatch, 4096 tokens/PE, top-8 of 256
    experts by Zipf(1.1), rows of 7168 bf16.  shapes: (rows per
    putmem_signal_wg call, work-group size)."""
    l = b.l
    tokens, experts, topk, row = 4096, 256, 8, 7168 * 2
    rng = np.random.default_rng(0)
    cdf = zipf_table(experts, 1.1)
    counts = np.zeros((P, P), np.uint32)
    for s in range(P):
        # top-k distinct by Gumbel-free sequential redraw on a vectorised batch
        chosen = np.full((tokens, topk), -1, np.int64)
        for k in range(topk):
            pick = np.searchsorted(cdf, rng.random(tokens))
            dup = (chosen[:, :k] == pick[:, None]).any(1)
            while dup.any():
                pick[dup] = np.searchsorted(cdf, rng.random(int(dup.sum())))
                dup = (chosen[:, :k] == pick[:, None]).any(1)
            chosen[:, k] = np.minimum(pick, experts - 1)
        counts[s] = np.bincount((chosen // (experts // P)).ravel(), minlength=P)
    send_row = np.zeros((P, P), np.uint32)
    recv_row = np.zeros((P, P), np.uint32)
    for s in range(P):
        send_row[s] = np.r_[0, np.cumsum(counts[s])[:-1]]
    for d in range(P):
        recv_row[:, d] = np.r_[0, np.cumsum(counts[:, d])[:-1]]
    rows_out = tokens * topk
    rows_in = int(counts.sum(0).max())
    recv, send, sig = l.malloc(rows_in * row), l.malloc(rows_out * row), l.malloc(8 * P)
    assert send and recv and sig, (rows_in * row, rows_out * row)
    for p in range(P):
        b.fill_random(l.pe_ptr(send, p), rows_out * row, p, 40 + p)
    tabs = [np.ascontiguousarray(a, np.uint32) for a in (counts, send_row, recv_row)]
    # Signal words are never cleared: the receivers keep running totals.
    expect = l.dev_alloc(8 * P * P)
    l.fill(expect, 0, 8 * P * P)
    assert l.fill_every_pe(sig, 0, 8 * P, None) == 0
    l.stream_sync(None)

    shape = [shapes[0]]

    def step():
        assert l.dispatch_put_signal(recv, send, sig, tabs[0].ctypes.data, tabs[1].ctypes.data,
                                     tabs[2].ctypes.data, row, shape[0][0], shape[0][1], expect, None) == 0

    alg = 2 * int(counts.sum()) * row
    res = {"rows": int(counts.sum())}
    for name, opt in CTX_KINDS:
        l.set_ctx_options(opt)
        for sh in shapes:
            shape[0] = sh
            # This configuration runs first in the process (its buffers need the
            # heap while it is empty), and the GPU's first milliseconds of work
            # run about 3 % below its sustained rate: ten launches before the
            # timed ones.
            ms = b.time_ms(step, max(5, steps // 2), 10)
            key = name if len(shapes) == 1 else "%s_rows%d_wg%d" % (name, sh[0], sh[1])
            res[key] = {"ms": round(ms, 4), "gbs": round(alg / ms / 1e6, 1),
                        "frac": round(alg / ms / 1e6 / HBM_PEAK_GBS, 4)}
    l.set_ctx_options(0)
    l.dev_free(expect)
    for x in (send, recv, sig):
        l.free(x)
    return res


def amo_config(b, steps):
    """configs[5] part 1: 16 Mi int64 fetch_add onto 4096 counters."""
    l, L = b.l, b.L
    K, n = 4096, 1 << 24
    ctr = l.malloc(K // P * 8)
    res = {}
    rng = np.random.default_rng(0)
    cdf = zipf_table(K, 1.1)
    for dist in ("uniform", "zipf"):
        if dist == "uniform":
            ids = rng.integers(0, K, n, dtype=np.uint32)
        else:
            ids = np.minimum(np.searchsorted(cdf, rng.random(n)), K - 1).astype(np.uint32)
        d_ids = l.dev_alloc(n * 4)
        d_out = l.dev_alloc(n * 8)
        l.copy_in(d_ids, ids.ctypes.data, n * 4)
        for p in range(P):
            l.fill(l.pe_ptr(ctr, p), 0, K // P * 8)
        res[dist] = {}
        for name, opt in CTX_KINDS:
            l.set_ctx_options(opt)
            ms = b.time_ms(lambda: l.amo(L.AMO_FETCH_ADD, L.LONG, ctr, K // P, d_ids, None, None, d_out,
                                         n, 0, 4096, 256, None), max(3, steps // 10), 1)
            res[dist][name] = {"ms": round(ms, 4), "mops": round(n / ms / 1e3, 1)}
        l.set_ctx_options(0)
        l.dev_free(d_ids)
        l.dev_free(d_out)
    l.free(ctr)
    return res


def pingpong_config(b):
    """configs[5] part 2: put_signal / wait_until ping-pong between work-groups
    acting as two PEs: one pair over 14 payload sizes, and 8 and 32 pairs at
    once at 8 B and 4 KiB (aggregate message rate)."""
    l = b.l
    max_pairs = 32
    buf, sig = l.malloc(65536 * max_pairs), l.malloc(8 * max_pairs)
    res = {}
    iters = 2000

    def run(n, pairs):
        out = {}
        for name, opt in CTX_KINDS:
            l.set_ctx_options(opt)
            assert l.fill_every_pe(sig, 0, 8 * max_pairs, None) == 0
            ticks, hz = C.c_uint64(), C.c_double()
            assert l.pingpong(buf, sig, n, iters, pairs, 0, 1, 256, C.byref(ticks), C.byref(hz),
                              None) == 0
            one_way_us = ticks.value / hz.value / iters / 2 * 1e6
            out[name] = {"latency_us": round(one_way_us, 3),
                         "msg_per_s": round(pairs * 1e6 / one_way_us, 1)}
        return out

    for k in range(3, 17):
        res[str(1 << k)] = run(1 << k, 1)
    for pairs in (8, 32):
        for n in (8, 4096):
            res["%d_x%dpairs" % (n, pairs)] = run(n, pairs)
    l.set_ctx_options(0)
    l.free(buf)
    l.free(sig)
    return res


def barrier_config(b):
    """One work-group per PE, P=8: rounds of (store to the next PE, barrier,
    read the received word).  Per-round time from two launches that differ
    only in the number of rounds."""
    l, L = b.l, b.L
    scratch = l.malloc(8)
    res = {}
    for name, fn in (("barrier_all", L.BARRIER_ALL), ("sync_all", L.SYNC_ALL), ("team_sync", L.TEAM_SYNC)):
        ms = {}
        for rounds in (200, 2200):
            assert l.fill_every_pe(scratch, 0, 8, None) == 0
            ms[rounds] = b.time_ms(lambda: l.wg_sync(fn, l.team_world(), scratch, rounds, 64, None), 3, 1)
        res[name + "_round_us"] = round((ms[2200] - ms[200]) / 2000 * 1e3, 3)
    l.free(scratch)
    return res


# ---- CPU baseline: the oracle's threaded routines on this host's cores, bounded
# samples of the same workloads.  (The only place outside tests/ and smoke()
# that touches oracle/.)  Three legs, run between the GPU bring-ups.
def cpu_threads(orc):
    # a one-GPU box gives a job 16 cores, whatever the machine has
    return max(1, min(16, orc.lib.orc_hardware_threads()))


def cpu_copy_leg():
    from oracle import pyoracle as orc
    threads = cpu_threads(orc)
    # bulk copy: 256 MiB messages, as the headline
    n = 256 * MiB
    src = np.random.default_rng(0).integers(0, 256, n, dtype=np.uint8)
    # eight buffer pairs taken in turn, as on the GPU: 4 GiB in all, more than the
    # last-level cache of the host holds
    srcs = [src] + [src.copy() for _ in range(P - 1)]
    dsts = [np.empty_like(src) for _ in range(P)]
    for k in range(P):
        orc.lib.orc_copy_threaded(dsts[k].ctypes.data, srcs[k].ctypes.data, n, threads)
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 4.0:
        k = reps % P
        orc.lib.orc_copy_threaded(dsts[(k + 1) % P].ctypes.data, srcs[k].ctypes.data, n, threads)
        reps += 1
    return {"cores": threads, "putmem_256MiB_gbs": round(2 * n * reps / (time.perf_counter() - t0) / 1e9, 2)}


def cpu_reduce_leg():
    from oracle import pyoracle as orc
    threads = cpu_threads(orc)
    # configs[0] as BASELINE.json states it: int32 sum, P=2 x 1 Mi elements, values
    # uniform in [-1000, 1000] from seed 0, both destinations written
    rng = np.random.default_rng(0)
    small = [rng.integers(-1000, 1001, 1 << 20, dtype=np.int32) for _ in range(2)]
    orc.to_all(orc.INT, orc.SUM, small, ndst=2, nthreads=threads)
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 1.0:
        orc.to_all(orc.INT, orc.SUM, small, ndst=2, nthreads=threads)
        reps += 1
    small_gbs = 2 * 2 * (1 << 20) * 4 * reps / (time.perf_counter() - t0) / 1e9
    # fp32 sum all-reduce at the GPU's size: P=8 x 64 Mi elements, result written to
    # all 8 destinations (4 GiB of host memory), at least two passes
    m = 1 << 26
    tile = np.random.default_rng(1).standard_normal(1 << 22).astype(np.float32)
    srcs = [np.tile(np.roll(tile, p), m // tile.size) for p in range(P)]
    orc.to_all(orc.FLOAT, orc.SUM, srcs, ndst=P, nthreads=threads)
    t0 = time.perf_counter()
    reps = 0
    while reps < 2 or time.perf_counter() - t0 < 4.0:
        orc.to_all(orc.FLOAT, orc.SUM, srcs, ndst=P, nthreads=threads)
        reps += 1
    red_gbs = 2 * P * m * 4 * reps / (time.perf_counter() - t0) / 1e9
    return {"to_all_int32_P2_1Mi_gbs": round(small_gbs, 2), "to_all_fp32_sum_gbs": round(red_gbs, 2)}


def cpu_amo_leg():
    from oracle import pyoracle as orc
    threads = cpu_threads(orc)
    # atomics at the GPU's size: 16 Mi seq_cst fetch_adds onto 4096 counters
    k = 1 << 24
    ids = np.random.default_rng(1).integers(0, 4096, k, dtype=np.uint32)
    counters = np.zeros(4096, np.int64)
    fetched = np.zeros(k, np.int64)
    sec = orc.lib.orc_amo_fetch_add_threaded(counters.ctypes.data, ids.ctypes.data, None,
                                             fetched.ctypes.data, k, threads)
    pp = orc.lib.orc_pingpong_threaded(8, 200000) / 200000 / 2 * 1e6
    return {"amo_fetch_add_mops": round(k / sec / 1e6, 1), "pingpong_8B_us": round(pp, 3)}


def cpu_baseline_record(legs):
    return {"value": legs["putmem_256MiB_gbs"], "unit": "GB/s", "cores": legs["cores"], "kind": "port",
            "sample": "threaded memcpy of 256 MiB messages for 4 s, eight buffer pairs in turn "
                      "(2N bytes per message); config 1: int32 sum P=2 x 1 Mi for 1 s; all-reduce: P=8 "
                      "x 64 Mi fp32, ascending fold, all 8 destinations written, >= 2 passes; atomics: "
                      "16 Mi seq_cst fetch_add on 4096 counters, uniform; ping-pong: 200000 round trips "
                      "of 8 B between two threads",
            "to_all_int32_P2_1Mi_gbs": legs["to_all_int32_P2_1Mi_gbs"],
            "to_all_fp32_sum_gbs": legs["to_all_fp32_sum_gbs"],
            "amo_fetch_add_mops": legs["amo_fetch_add_mops"],
            "pingpong_8B_us": legs["pingpong_8B_us"],
            "putmem_256MiB_gbs": legs["putmem_256MiB_gbs"]}


def profile_kernels():
    """What rocprofv3 --pmc / --kernel-trace is pointed at: each dominant kernel
    a few times on full-size inputs, and the HIP runtime's own copy kernel on
    256 MiB as the yardstick of the byte counters."""
    os.environ.setdefault("ROCSHMEM_EMU_SPREAD", "1")
    from rocshmem_amd import lib as L
    b = Bench(L)
    b.quick = True
    b.short = False
    l = b.l
    assert l.init(P, 8 << 30) == 0
    disp = dispatch_config(b, 10)                      # 10 warm-up + 5 timed launches per context kind
    n = 256 * MiB
    cs, cd = l.malloc(n), l.malloc(n)
    for _ in range(3):
        l.copy_dev(cd, cs, n)
    l.free(cs)
    l.free(cd)
    head = headline(b, 8, 2)                           # 10 launches of each of the put routes
    m = 1 << 26
    src, dst = l.malloc(m * 4), l.malloc(m * 4)
    for p in range(P):
        b.fill_random(l.pe_ptr(src, p), m * 4, p, 10 + p, "f32")
    ms_red = b.time_ms(lambda: l.to_all(L.FLOAT, L.SUM, dst, src, m, 0, 0, P, None), 6, 2)
    l.free(src)
    l.free(dst)
    a2a = alltoall_config(b, 6)
    red = to_all_configs(b, 6, 2, which=("fp32_sum",))  # includes the many-teams device all-reduce
    reuse = {"uncached_heap": reuse_config(b, 8)}       # 7 launches per number of passes (1, then 4)
    l.finalize()
    # the same reads once more on a cached heap: the later launches of reuse_probe_kernel
    bring_up(L, 1 << 30, ROCSHMEM_EMU_SPREAD=None, ROCSHMEM_EMU_HEAP_CACHED="1")
    reuse["cached_heap"] = reuse_config(b, 8)
    l.finalize()
    os.environ.pop("ROCSHMEM_EMU_HEAP_CACHED", None)
    print(json.dumps({"putmem_wg_nostore_gbs": round(head["gbs"], 1),
                      "wg_reduce_teams": {k: v for k, v in red.items() if "teams" in k},
                      "reuse_256MiB": reuse,
                      "putmem_wg_default_gbs": round(head["default_ctx_gbs"], 1),
                      "host_putmem_gbs": round(head["host_putmem_gbs"], 1),
                      "to_all_fp32_sum_gbs": round(2 * P * m * 4 / ms_red / 1e6, 1),
                      "alltoall_gbs": a2a["gbs"], "dispatch": disp}))


def process_leg(steps, warmup):
    """One PE of a job of two processes (started by process_per_pe_config through
    rocshmem_amd.launch): PE 0 runs the headline's tiled rocshmem_ctx_putmem_wg
    and getmem_wg, and the host rocshmem_putmem, with PE 1 — another process,
    its heap mapped here through HIP IPC — as the target.  Three buffer pairs
    of 256 MiB in rotation (1.5 GiB, the heap of a process stays below 2 GiB)
    keep the memory-side cache out of it.  PE 1 checks what arrived against PE
    0's source, which it reads through its own mapping.  PE 0 prints the record."""
    from rocshmem_amd import lib as L
    b = Bench(L)
    l = b.l
    assert l.init(0, 1900 * MiB) == 0
    me, n, pairs = l.my_pe(), 256 * MiB, 3
    assert l.n_pes() == 2
    bufs = [(l.malloc(n), l.malloc(n)) for _ in range(pairs)]
    assert all(s and d for s, d in bufs)
    for i, (s, d) in enumerate(bufs):
        b.fill_random(s, n, me, 10 * me + i)
        l.fill(d, 0, n)
    l.barrier_all()
    out = {}
    if me == 0:
        k = [0]

        def rotating(fn):
            def step():
                s, d = bufs[k[0] % pairs]
                k[0] += 1
                assert fn(s, d) == 0
            return step

        wg, tile, _ = PUT_SHAPES["nostore_ctx"]
        l.set_ctx_options(1)
        put = rotating(lambda s, d: l.rma(L.PUT, L.WG, d, s, n, tile, 0, 1, n // tile, wg, 1, None))
        for _ in range(2):
            out["putmem_wg_nostore_gbs"] = round(2 * n / b.time_ms(put, steps, warmup) / 1e6, 1)
        out["getmem_wg_nostore_gbs"] = round(2 * n / b.time_ms(
            rotating(lambda s, d: l.rma(L.GET, L.WG, d, s, n, tile, 0, 1, n // tile, wg, 1, None)),
            steps, warmup) / 1e6, 1)
        l.set_ctx_options(0)
        wg, tile, n_wgs = PUT_SHAPES["default_ctx"]
        out["putmem_wg_default_ctx_gbs"] = round(2 * n / b.time_ms(
            rotating(lambda s, d: l.rma(L.PUT, L.WG, d, s, n, tile, 0, 1, n_wgs, wg, 1, None)),
            steps, warmup) / 1e6, 1)
        out["host_putmem_gbs"] = round(2 * n / b.time_ms(
            rotating(lambda s, d: l.putmem(d, s, n, 0, 1, None)), steps, warmup) / 1e6, 1)
        # one more tiled put per pair into cleared destinations, for PE 1 to check
        l.barrier_all()            # the timed loops are over
        l.barrier_all()            # PE 1 has cleared its destinations
        l.set_ctx_options(1)
        for s, d in bufs:
            assert l.rma(L.PUT, L.WG, d, s, n, 4096, 0, 1, n // 4096, 128, 1, None) == 0
        l.set_ctx_options(0)
        l.barrier_all()            # the puts have landed
        print("PROCESS_LEG " + json.dumps(out), flush=True)
    else:
        l.barrier_all()            # PE 0 has finished its timed loops
        for _, d in bufs:
            l.fill(d, 0, n)
        l.barrier_all()            # PE 0 may put
        l.barrier_all()            # PE 0 has put
        ok = True
        for s, d in bufs:
            bad = C.c_uint64(1)
            assert l.compare(d, l.pe_ptr(s, 0), n, C.byref(bad), None) == 0
            ok = ok and bad.value == 0
        print("PROCESS_LEG_VERIFIED %d" % ok, flush=True)
    l.finalize()


def process_per_pe_config(steps, warmup):
    """The headline between two processes (the reference's deployment: one
    process per PE, peers mapped through HIP IPC).  Run while this process
    holds no runtime, so that the two children have the GPU to themselves."""
    from rocshmem_amd import launch
    env = dict(os.environ)
    for name in ("ROCSHMEM_EMU_SPREAD", "ROCSHMEM_EMU_HEAP_CACHED", "ROCSHMEM_EMU_NPES"):
        env.pop(name, None)
    status, outs = launch.run(2, [sys.executable, os.path.abspath(__file__), "--process-leg", "--steps",
                                  str(steps), "--warmup", str(warmup)], timeout=120, env=env, capture=True)
    rec = {"exit_status": status}
    for o in outs:
        for ln in o.splitlines():
            if ln.startswith("PROCESS_LEG "):
                rec.update(json.loads(ln[len("PROCESS_LEG "):]))
            elif ln.startswith("PROCESS_LEG_VERIFIED "):
                rec["verified"] = ln.split()[1] == "1"
    rec.setdefault("verified", False)
    if status != 0:
        rec["output_tail"] = [o[-300:] for o in outs]
    return rec


def bring_up(L, heap_bytes, **env):
    """rocshmem_init with the given layout / heap switches in the environment
    (a value of None removes the variable)."""
    for name, value in env.items():
        if value is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = value
    l = L.load()
    assert l.init(P, heap_bytes) == 0
    return {"pe_stride_bytes": l.pe_stride(), "heap_alloc_bytes": l.heap_alloc_bytes(),
            "heap_uncached": l.heap_is_uncached()}


def main():
    a = parse()
    if a.profile_kernels:
        profile_kernels()
        return
    if a.process_leg:
        process_leg(a.steps, a.warmup)
        return
    if a.gpus != 1:
        print("bench.py measures one GPU: every PE is a slice of one symmetric heap on a single "
              "MI355X; --gpus %d is not supported (use --gpus 1)." % a.gpus, file=sys.stderr)
        sys.exit(2)
    os.environ.setdefault("ROCSHMEM_MAX_NUM_TEAMS", "140")
    from rocshmem_amd import lib as L
    b = Bench(L)
    b.quick = a.quick
    b.short = False
    full = not a.quick
    with_cpu = full and not a.no_cpu
    legs = {}
    allc = {}

    # ---- first bring-up: the slices spread over half of the device memory (16 GiB
    # apart): kernels that write to all 8 slices at once sustain about 10 % more
    # than with packed slices.  8 slices of 8 GiB: with Zipf(1.1) routing the
    # busiest PE receives 2.3 GiB of rows, a 4 GiB block of the power-of-two
    # allocator.  That request goes first because the allocator never merges
    # freed blocks.
    layout = bring_up(L, 8 << 30, ROCSHMEM_EMU_SPREAD="1", ROCSHMEM_EMU_HEAP_CACHED=None)
    if full:
        allc["dispatch_put_signal"] = dispatch_config(b, a.steps)
    if a.calibrate:
        cs, cd = b.l.malloc(256 * MiB), b.l.malloc(256 * MiB)
        for _ in range(3):
            b.l.copy_dev(cd, cs, 256 * MiB)
        b.l.free(cs)
        b.l.free(cd)
    head = headline(b, a.steps, a.warmup)
    if full:
        allc["to_all_P8_64Mi"] = to_all_configs(b, a.steps, a.warmup)
        allc["alltoall_512x7168_bf16"] = alltoall_config(b, a.steps)
        allc["atomic_fetch_add_16Mi"] = amo_config(b, a.steps)
        allc["pingpong"] = pingpong_config(b)
        allc["barrier_P8"] = barrier_config(b)
        allc["message_rates"] = message_rates(b, a.steps)
        allc["reuse_256MiB"] = {"uncached_heap": reuse_config(b, a.steps)}
        allc["putmem_curve"] = head["curve"]
        allc["hbm_one_direction_256MiB"] = head["ceilings"]
        allc["putmem_wg_tiled_256MiB"] = head["tiled"]
    b.l.finalize()
    if full and a.with_processes:
        allc["process_per_pe_2_processes"] = process_per_pe_config(a.steps, a.warmup)
    if with_cpu:
        legs.update(cpu_copy_leg())

    # ---- second bring-up: the default layout, slices packed (stride = heap size),
    # 1 GiB per PE — what a plain rocshmem_init gives, and the layout BASELINE.json
    # names ("one 8 GiB symmetric heap").
    packed = {}
    if full:
        b.short = True
        packed["layout"] = bring_up(L, 1 << 30, ROCSHMEM_EMU_SPREAD=None)
        packed["putmem_wg"] = headline(b, a.steps, a.warmup)
        packed["to_all"] = to_all_configs(b, a.steps, a.warmup, which=("fp32_sum",), device_api=False)
        packed["alltoall"] = alltoall_config(b, a.steps)
        b.l.finalize()
        allc["packed_layout_1GiB_per_pe"] = {
            "layout": packed["layout"],
            "putmem_wg_nostore_gbs": round(packed["putmem_wg"]["gbs"], 1),
            "putmem_wg_default_ctx_gbs": round(packed["putmem_wg"]["default_ctx_gbs"], 1),
            "host_putmem_gbs": round(packed["putmem_wg"]["host_putmem_gbs"], 1),
            "to_all_fp32_sum": packed["to_all"]["fp32_sum"], "alltoall": packed["alltoall"]}
    if with_cpu:
        legs.update(cpu_reduce_leg())

    # ---- third bring-up: a cached heap (plain hipMalloc, what the reference's IPC
    # build uses), packed, 8 GiB per PE for the dispatch: what a consumer that
    # re-reads symmetric data gains, and what ordering costs there.
    cached = {}
    if full:
        cached["layout"] = bring_up(L, 8 << 30, ROCSHMEM_EMU_HEAP_CACHED="1")
        cached["dispatch"] = dispatch_config(b, a.steps)
        cached["putmem_wg"] = headline(b, a.steps, a.warmup)
        cached["reuse"] = reuse_config(b, a.steps)
        b.l.finalize()
        os.environ.pop("ROCSHMEM_EMU_HEAP_CACHED", None)
        allc["reuse_256MiB"]["cached_heap"] = cached["reuse"]
        allc["cached_heap_8GiB_per_pe"] = {
            "layout": cached["layout"],
            "putmem_wg_nostore_gbs": round(cached["putmem_wg"]["gbs"], 1),
            "putmem_wg_default_ctx_gbs": round(cached["putmem_wg"]["default_ctx_gbs"], 1),
            "host_putmem_gbs": round(cached["putmem_wg"]["host_putmem_gbs"], 1),
            "dispatch_put_signal": cached["dispatch"]}
        b.short = False
    if with_cpu:
        legs.update(cpu_amo_leg())
    cpu = cpu_baseline_record(legs) if with_cpu else None

    def frac(gbs):
        return round(gbs / HBM_PEAK_GBS, 4)

    verified = bool(head["verified"])
    # One figure per configuration first (a record that keeps only the leading
    # keys still carries every configuration), then the rest.
    roof = {"bound": "hbm", "achieved": round(head["gbs"], 1), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": frac(head["gbs"]),
            # FETCH_SIZE + WRITE_SIZE per launch under rocprofv3 --pmc, scaled by the
            # HIP runtime's own copy kernel (profiles/putmem_wg_tiled_256MiB_hbm_traffic.txt)
            "traffic": PUT_TRAFFIC_BYTES, "kernel": "rma_kernel<PUT, WG> (rocshmem_ctx_putmem_wg)"}
    if full:
        ta, a2a = allc["to_all_P8_64Mi"], allc["alltoall_512x7168_bf16"]
        dp, amo, pp = allc["dispatch_put_signal"], allc["atomic_fetch_add_16Mi"], allc["pingpong"]
        mr, ru = allc["message_rates"], allc["reuse_256MiB"]
        verified = verified and bool(packed["putmem_wg"]["verified"]) and bool(cached["putmem_wg"]["verified"])
        if "process_per_pe_2_processes" in allc:
            verified = verified and bool(allc["process_per_pe_2_processes"]["verified"])
        roof.update({
            # configs[1]: bulk putmem through the device API, both kinds of context
            "verified": verified,
            "putmem_wg_frac": frac(head["default_ctx_gbs"]),
            "putmem_wg_frac_nostore": frac(head["gbs"]),
            # configs[2]: all-reduce P=8 x 64 Mi, host call and device call
            "to_all_fp32_sum_frac": ta["fp32_sum"]["frac"],
            "to_all_bf16_sum_frac": ta["bf16_sum"]["frac"],
            "to_all_int64_xor_frac": ta["int64_xor"]["frac"],
            "wg_reduce_teams_frac": ta["fp32_sum_wg_reduce_teams_default_ctx"]["frac"],
            # configs[3]: alltoall and put_signal dispatch
            "alltoall_frac": a2a["frac"],
            "dispatch_frac": dp["default_ctx"]["frac"],
            "dispatch_frac_nostore": dp["nostore_ctx"]["frac"],
            # configs[4]: atomics and ping-pong
            "amo_uniform_mops": amo["uniform"]["default_ctx"]["mops"],
            "amo_zipf_mops": amo["zipf"]["default_ctx"]["mops"],
            "pingpong_8B_us": pp["8"]["default_ctx"]["latency_us"],
            # the default (packed) layout, 1 GiB per PE
            "to_all_fp32_sum_frac_packed": packed["to_all"]["fp32_sum"]["frac"],
            "putmem_wg_frac_nostore_packed": frac(packed["putmem_wg"]["gbs"]),
            # configs[0]: int32 sum, P=2 x 1 Mi
            "to_all_int32_P2_1Mi_gbs": ta["int32_sum_P2_1Mi"]["gbs"],
            "to_all_fp32_max_frac": ta["fp32_max"]["frac"],
            # ---- beyond the leading keys
            "wg_reduce_teams_frac_nostore": ta["fp32_sum_wg_reduce_teams_nostore_ctx"]["frac"],
            "amo_uniform_mops_nostore": amo["uniform"]["nostore_ctx"]["mops"],
            "amo_zipf_mops_nostore": amo["zipf"]["nostore_ctx"]["mops"],
            "putmem_8B_per_lane_mmsg_per_s": mr["putmem_8B_contiguous_default_ctx"]["mmsg_per_s"],
            "putmem_8B_per_lane_scattered_mmsg_per_s": mr["putmem_8B_scattered_default_ctx"]["mmsg_per_s"],
            "putmem_64B_per_lane_gbs": mr["putmem_64B_contiguous_default_ctx"]["gbs"],
            "putmem_4KiB_per_lane_gbs": mr["putmem_4096B_contiguous_default_ctx"]["gbs"],
            "putmem_wave_512B_gbs": mr["putmem_wave_512B_contiguous_default_ctx"]["gbs"],
            "putmem_wave_4KiB_gbs": mr["putmem_wave_4096B_contiguous_default_ctx"]["gbs"],
            "putmem_wave_4KiB_gbs_nostore": mr["putmem_wave_4096B_contiguous_nostore_ctx"]["gbs"],
            "reuse_read_x4_gbs_uncached_heap": ru["uncached_heap"]["read_x4_gbs"],
            "reuse_read_x4_gbs_cached_heap": ru["cached_heap"]["read_x4_gbs"],
            "putmem_wg_frac_cached_heap": frac(cached["putmem_wg"]["default_ctx_gbs"]),
            "putmem_wg_frac_nostore_cached_heap": frac(cached["putmem_wg"]["gbs"]),
            "dispatch_frac_cached_heap": cached["dispatch"]["default_ctx"]["frac"],
            "dispatch_frac_nostore_cached_heap": cached["dispatch"]["nostore_ctx"]["frac"],
            "alltoall_frac_packed": packed["alltoall"]["frac"],
            "algorithmic_bytes_per_launch": head["bytes_per_step"],
            "host_putmem_frac": frac(head["host_putmem_gbs"]),
            "host_getmem_frac": frac(head["host_getmem_gbs"]),
            "getmem_wg_frac_nostore": frac(head["getmem_wg_gbs"]),
            "hbm_read_only_gbs": head["ceilings"]["read_only_gbs"],
            "hbm_write_only_gbs": head["ceilings"]["write_only_gbs"],
            "l2_release_ns_each_per_tile": head["release_ns_each_per_tile"],
            "l2_release_ns_each_at_end": head["release_ns_each_at_end"],
            "wg_reduce_fp32_sum_one_wg_per_pe_gbs": ta["fp32_sum_wg_reduce_one_wg_per_pe"]["gbs"],
            "fcollect_frac": a2a["fcollect_same_block"]["frac"],
            "broadcast_frac": a2a["broadcast_P_blocks_from_pe0"]["frac"],
            "pingpong_8B_us_nostore": pp["8"]["nostore_ctx"]["latency_us"],
            "pingpong_64KiB_us": pp["65536"]["default_ctx"]["latency_us"],
            "pingpong_32pairs_msg_per_s": pp["8_x32pairs"]["nostore_ctx"]["msg_per_s"],
            "barrier_all_round_us": allc["barrier_P8"]["barrier_all_round_us"],
        })
        if "process_per_pe_2_processes" in allc:
            roof["putmem_wg_frac_nostore_between_processes"] = frac(
                allc["process_per_pe_2_processes"].get("putmem_wg_nostore_gbs", 0.0))
    else:
        roof.update({"verified": verified, "putmem_wg_frac": frac(head["default_ctx_gbs"]),
                     "putmem_wg_frac_nostore": frac(head["gbs"]),
                     "host_putmem_frac": frac(head["host_putmem_gbs"])})
    line = {
        "metric": "HBM GB/s (% of MI355X peak) for to_all/alltoall/putmem; atomic Mops/s",
        "value": round(head["gbs"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(head["ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": "configs[1] largest size: 256 MiB putmem per step, PE k%8 -> (k+1)%8 of P=8, "
                               "every CU calling rocshmem_ctx_putmem_wg",
                   "detail": "one %d-byte tile per work-group of %d, ROCSHMEM_CTX_NOSTORE context, one quiet "
                             "per work-group; buffers rotate so no step re-reads cached data" % (
                                 PUT_SHAPES["nostore_ctx"][1], PUT_SHAPES["nostore_ctx"][0]),
                   "n_pes": P, "message_bytes": 256 * MiB, "heap_bytes_per_pe": 8 << 30,
                   "layout": "ROCSHMEM_EMU_SPREAD=1",
                   "pe_stride_bytes": layout["pe_stride_bytes"],
                   "heap_alloc_bytes": layout["heap_alloc_bytes"],
                   "verified": verified},
        "roofline": roof,
        # the reference's own convention (tests/functional_tests/tester.cpp:505-508):
        # payload bytes per second in GiB/s, counting each byte once
        "reference_convention_payload_gib_s": round(256 * MiB / (head["ms"] * 1e-3) / 2**30, 1),
        "cpu_baseline": cpu,
        "all_configs": allc,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
