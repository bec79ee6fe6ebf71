"""C1-C3, H3: putmem/getmem at thread, wavefront and work-group granularity,
and the host-initiated whole-GPU copy, byte-exact against the oracle's copy
with guard bytes either side.  Through the C entry points."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P, HEAP = 8, 1 << 30
GUARD = 64


@pytest.fixture(scope="module")
def env(rt, L, orc):
    l = rt.up(P, HEAP)
    size = 8 << 20
    src = l.malloc(size)
    dst = l.malloc(size)
    assert src and dst
    host = orc.fill_u8(size, 0, 11)
    rt.put_bytes(src, host)
    yield dict(l=l, src=src, dst=dst, size=size, host=host)
    l.free(src)
    l.free(dst)


def run_case(rt, L, orc, env, op, gran, n, soff, doff, n_wgs, wg_size, my_pe=0, pe=1, tile=0,
             ctx_options=0):
    """Copies n bytes from src+soff to dst+doff across PEs and checks the
    destination window including GUARD bytes on both sides."""
    l = env["l"]
    src, dst, host = env["src"], env["dst"], env["host"]
    base = GUARD + 16  # room for the low guard
    if op in (L.PUT, L.PUT_NBI):
        local = l.pe_ptr(src, my_pe) + soff
        remote_mine = l.pe_ptr(dst, my_pe) + base + doff
        landing = l.pe_ptr(dst, pe) + base + doff
        d_arg, s_arg = remote_mine, local
        if my_pe != 0:
            rt.put_bytes(l.pe_ptr(src, my_pe), host[:soff + n + 1])
    else:
        remote_mine = l.pe_ptr(src, my_pe) + soff
        origin = l.pe_ptr(src, pe)
        rt.put_bytes(origin, host[:soff + n + 1])
        landing = l.pe_ptr(dst, my_pe) + base + doff
        d_arg, s_arg = landing, remote_mine
    l.fill(landing - GUARD, 0xA5, n + 2 * GUARD)
    before = l.set_ctx_options(ctx_options)
    rc = l.rma(op, gran, d_arg, s_arg, n, tile, my_pe, pe, n_wgs, wg_size, 1, None)
    l.set_ctx_options(before)
    assert rc == 0
    l.stream_sync(None)
    got = rt.get_bytes(landing - GUARD, n + 2 * GUARD)
    want = np.full(n + 2 * GUARD, 0xA5, np.uint8)
    if n:
        exp = np.empty(n, np.uint8)
        orc.lib.orc_copy(exp.ctypes.data, host[soff:soff + n].ctypes.data, n)
        want[GUARD:GUARD + n] = exp
    assert np.array_equal(got, want), (op, gran, n, soff, doff, n_wgs, wg_size)


GRANS = ["THREAD", "WAVE", "WG"]


@pytest.mark.parametrize("gran", GRANS)
@pytest.mark.parametrize("op", ["PUT", "GET"])
def test_every_size_up_to_300(rt, L, orc, env, op, gran):
    for n in range(0, 301):
        run_case(rt, L, orc, env, getattr(L, op), getattr(L, gran), n, 3, 5, 1, 64)


@pytest.mark.parametrize("gran", GRANS)
def test_all_256_alignment_pairs(rt, L, orc, env, gran):
    for n in (1, 15, 16, 17, 100, 1000):
        for soff in range(16):
            for doff in range(16):
                run_case(rt, L, orc, env, L.PUT, getattr(L, gran), n, soff, doff, 1, 128)


def test_sizes_to_4096_one_alignment_each(rt, L, orc, env):
    rng = np.random.default_rng(0)
    for n in range(301, 4097, 7):
        run_case(rt, L, orc, env, L.PUT, L.WG, n, int(rng.integers(16)), int(rng.integers(16)), 1, 256)
        run_case(rt, L, orc, env, L.GET, L.WAVE, n, int(rng.integers(16)), int(rng.integers(16)), 1, 64)


@pytest.mark.parametrize("wg_size", [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 768, 1024])
def test_block_sizes_iota(rt, L, orc, env, wg_size):
    """tests/unit_tests/ipc_impl_simple_fine_gtest.cpp:71-177: work-group copies
    with block sizes 1..1024 (and 768)."""
    for n in (32 * 4, 4099):
        run_case(rt, L, orc, env, L.PUT, L.WG, n, 0, 0, 1, wg_size)
        run_case(rt, L, orc, env, L.GET, L.WG, n, 0, 0, 1, wg_size)


@pytest.mark.parametrize("lanes", [1, 2, 3, 7, 31, 32, 33, 63, 64])
def test_wave_lane_counts(rt, L, orc, env, lanes):
    """Wavefront copies with 1..64 active lanes (same gtest, wave fixtures)."""
    for n in (128, 1027):
        run_case(rt, L, orc, env, L.PUT, L.WAVE, n, 1, 2, 1, lanes)
        run_case(rt, L, orc, env, L.GET, L.WAVE, n, 1, 2, 1, lanes)


@pytest.mark.parametrize("gran", GRANS)
def test_tiled_multi_group_transfers(rt, L, orc, env, gran):
    """tests/functional_tests/extended_primitives.cpp:49-51: several groups each
    moving their own tile."""
    for n, n_wgs, wg, tile in [(1 << 16, 8, 256, 0), (100001, 7, 192, 0), (1 << 20, 64, 256, 4096),
                               (5000, 4, 64, 17)]:
        run_case(rt, L, orc, env, L.PUT, getattr(L, gran), n, 1, 9, n_wgs, wg, tile=tile)
        run_case(rt, L, orc, env, L.GET, getattr(L, gran), n, 6, 0, n_wgs, wg, tile=tile)


@pytest.mark.parametrize("gran", GRANS)
def test_nostore_context_moves_the_same_bytes(rt, L, orc, env, gran):
    """A context created with ROCSHMEM_CTX_NOSTORE (src/fence_policy.hpp:45-63)
    completes its puts without the L2 write-back; the bytes that land are the
    same for every size class, alignment and tiling."""
    g = getattr(L, gran)
    for n in list(range(0, 70)) + [255, 256, 1000, 4099, 65536, 65537, 100001]:
        run_case(rt, L, orc, env, L.PUT, g, n, 3, 5, 1, 128, ctx_options=L.CTX_NOSTORE)
    for soff in range(0, 16, 3):
        for doff in range(16):
            run_case(rt, L, orc, env, L.PUT, g, 777, soff, doff, 2, 64, ctx_options=L.CTX_NOSTORE)
    for n, n_wgs, wg, tile in [(1 << 20, 64, 256, 4096), (1 << 22, 128, 1024, 65536), (5000, 4, 64, 17)]:
        run_case(rt, L, orc, env, L.PUT, g, n, 1, 9, n_wgs, wg, tile=tile, ctx_options=L.CTX_NOSTORE)
        run_case(rt, L, orc, env, L.GET, g, n, 6, 0, n_wgs, wg, tile=tile, ctx_options=L.CTX_NOSTORE)


@pytest.mark.parametrize("ctx_options", [0, 1])
@pytest.mark.parametrize("gran", GRANS)
@pytest.mark.parametrize("op", ["PUT_NBI", "GET_NBI"])
def test_non_blocking_forms(rt, L, orc, env, op, gran, ctx_options):
    """rocshmem_putmem_nbi / getmem_nbi and their _wave / _wg forms
    (rocshmem_RMA.hpp:259-264,640-645): many calls per thread, wavefront or
    work-group, one quiet at the end; the bytes that land are those of the
    blocking calls."""
    o, g = getattr(L, op), getattr(L, gran)
    for n in list(range(0, 40)) + [255, 256, 1000, 4099, 65537]:
        run_case(rt, L, orc, env, o, g, n, 3, 5, 1, 128, ctx_options=ctx_options)
    for soff in range(0, 16, 5):
        for doff in range(0, 16, 3):
            run_case(rt, L, orc, env, o, g, 777, soff, doff, 2, 64, ctx_options=ctx_options)
    # small tiles: every group issues many calls before its quiet
    for n, n_wgs, wg, tile in [(1 << 18, 2, 256, 64), (100001, 3, 192, 17), (1 << 20, 64, 256, 4096)]:
        if gran == "WG" and tile < 4096:
            n = n // 16
        run_case(rt, L, orc, env, o, g, n, 1, 9, n_wgs, wg, tile=tile, ctx_options=ctx_options)


@pytest.mark.parametrize("with_signal", [0, 1, 2, 3])
@pytest.mark.parametrize("ctx_options", [0, 1])
@pytest.mark.parametrize("nbytes,pairs,wg", [(4096, 1, 64), (65536, 16, 256), (1 << 20, 64, 1024),
                                             (262144 + 4, 128, 256)])
def test_put_quiet_flag_seen_in_order(rt, L, env, ctx_options, with_signal, nbytes, pairs, wg):
    """Message passing inside one kernel: the receiver, released by a relaxed
    flag that follows rocshmem_ctx_quiet (src/ipc/context_ipc_device.cpp:100-102)
    or by the signal of putmem_signal_wg (:221-247), must find every word of the
    payload, on a default context and on a ROCSHMEM_CTX_NOSTORE one, over 20
    rounds with a new pattern each.  with_signal 2 / 3: the payload leaves as
    many putmem_nbi_wave / putmem_nbi calls which only the quiet completes."""
    import ctypes as C
    l = env["l"]
    data = l.malloc(nbytes * pairs)
    flags = l.malloc(16 * pairs)
    assert data and flags
    bad, timed_out = C.c_uint64(99), C.c_int(99)
    before = l.set_ctx_options(ctx_options)
    rc = l.put_flag_check(l.pe_ptr(data, 1), l.pe_ptr(flags, 1), nbytes, pairs, 20, 1, 6, wg,
                          with_signal, C.byref(bad), C.byref(timed_out), None)
    l.set_ctx_options(before)
    assert rc == 0
    assert timed_out.value == 0
    assert bad.value == 0
    l.free(data)
    l.free(flags)


@pytest.mark.parametrize("with_signal", [4, 5])
@pytest.mark.parametrize("ctx_options", [0, 1])
@pytest.mark.parametrize("nbytes,pairs,wg", [(4096, 1, 64), (65536, 16, 256), (16384 + 4, 128, 1024)])
def test_put_from_lds_then_flag_seen_in_order(rt, L, env, ctx_options, with_signal, nbytes, pairs, wg):
    """The same message passing with the producer's source in its LDS: the copy
    then takes the path for local buffers that global loads cannot reach, and
    its stores to the destination must be complete before the flag (quiet on
    either kind of context, or the signal of putmem_signal_wg) like any other
    put's."""
    test_put_quiet_flag_seen_in_order(rt, L, env, ctx_options, with_signal, nbytes, pairs, wg)


@pytest.mark.parametrize("gran", GRANS)
@pytest.mark.parametrize("op", ["PUT", "GET", "PUT_NBI"])
@pytest.mark.parametrize("ctx_options", [0, 1])
def test_scattered_messages(rt, L, orc, env, op, gran, ctx_options):
    """Many small messages whose neighbours in the wavefront are far apart
    (every message visited once through a permutation of the slots), and the
    same messages with lanes that continue one another: the destination is the
    source either way, byte for byte, guards untouched."""
    l = env["l"]
    src, dst, host = env["src"], env["dst"], env["host"]
    o, g = getattr(L, op), getattr(L, gran)
    for msg, count in [(8, 1 << 14), (64, 1 << 12), (24, 1 << 10), (4096, 64), (1, 256)]:
        n = msg * count
        for scattered in (1, 0):
            landing = l.pe_ptr(dst, 1) + GUARD
            l.fill(landing - GUARD, 0xA5, n + 2 * GUARD)
            before = l.set_ctx_options(ctx_options)
            if o == L.GET:
                rt.put_bytes(l.pe_ptr(src, 1), host[:n])
                rc = l.rma_messages(o, g, l.pe_ptr(dst, 1) + GUARD, l.pe_ptr(src, 0), n, msg, scattered, 0,
                                    1, 8, 128, 1, None)
            else:
                rc = l.rma_messages(o, g, l.pe_ptr(dst, 0) + GUARD, l.pe_ptr(src, 0), n, msg, scattered, 0,
                                    1, 8, 128, 1, None)
            l.set_ctx_options(before)
            assert rc == 0
            l.stream_sync(None)
            got = rt.get_bytes(landing - GUARD, n + 2 * GUARD)
            assert np.array_equal(got[GUARD:GUARD + n], host[:n]), (op, gran, msg, count, scattered)
            assert (got[:GUARD] == 0xA5).all() and (got[GUARD + n:] == 0xA5).all()
    # a number of tiles that is no power of two cannot be permuted this way
    assert l.rma_messages(o, g, l.pe_ptr(dst, 0), l.pe_ptr(src, 0), 24 * 1000, 24, 1, 0, 1, 8, 128, 1,
                          None) == -1


@pytest.mark.parametrize("kind", [0, 1, 2])
@pytest.mark.parametrize("ctx_options", [0, 1])
@pytest.mark.parametrize("pairs,wg", [(1, 64), (64, 256)])
def test_polling_with_gets_sees_the_put(rt, L, env, ctx_options, kind, pairs, wg):
    """A poller that has the old value in its caches and then only calls
    rocshmem_<T>_g / getmem / getmem_wave in a loop (no wait_until,
    no fence) sees the value its partner puts, round after round: a get reads
    memory, not a cached line."""
    import ctypes as C
    l = env["l"]
    words, ready = l.malloc(64 * pairs), l.malloc(8 * pairs)
    timed_out = C.c_int(99)
    before = l.set_ctx_options(ctx_options)
    rc = l.poll_with_gets(l.pe_ptr(words, 1), l.pe_ptr(ready, 1), pairs, 20, 1, 6, kind, wg,
                          C.byref(timed_out), None)
    l.set_ctx_options(before)
    assert rc == 0 and timed_out.value == 0
    got = rt.get_bytes(l.pe_ptr(words, 6), 64 * pairs, np.uint64)
    assert (got == 20).all()
    l.free(words)
    l.free(ready)


def test_every_pe_pair(rt, L, orc, env):
    for me in range(P):
        for pe in range(P):
            run_case(rt, L, orc, env, L.PUT, L.WG, 777, 1, 1, 2, 128, my_pe=me, pe=pe)
    for me in (0, 3, 7):
        for pe in (0, 5):
            run_case(rt, L, orc, env, L.GET, L.WG, 777, 1, 1, 2, 128, my_pe=me, pe=pe)


def test_powers_of_two_to_256mib(rt, L, orc):
    """The bandwidth curve's message sizes, 8 B .. 256 MiB, checked whole:
    device-API work-group put from all CUs, and the host-initiated copy."""
    l = rt.up(P, HEAP)
    big = 256 << 20
    src, dst = l.malloc(big), l.malloc(big)
    assert src and dst
    host = orc.fill_u8(big, 0, 5)
    rt.put_bytes(src, host)
    for k in range(3, 29):
        n = 1 << k
        for mode in ("device", "host"):
            l.fill(l.pe_ptr(dst, 2), 0, n + 16)
            if mode == "device":
                assert l.rma(L.PUT, L.WG, dst, src, n, 0, 0, 2, min(1024, max(1, n // 4096)), 256, 1, None) == 0
            else:
                assert l.putmem(dst, src, n, 0, 2, None) == 0
            l.stream_sync(None)
            got = rt.get_bytes(l.pe_ptr(dst, 2), n + 16)
            assert np.array_equal(got[:n], host[:n]), (k, mode)
            assert not got[n:].any(), (k, mode)
    # getmem, misaligned, large
    n = (64 << 20) + 13
    l.fill(dst, 0, n + 32)
    assert l.getmem(dst + 3, l.pe_ptr(src, 0) + 5, n, 0, 0, None) == 0
    l.stream_sync(None)
    got = rt.get_bytes(dst, n + 32)
    assert np.array_equal(got[3:3 + n], host[5:5 + n]) and not got[:3].any() and not got[3 + n:].any()
    l.free(src)
    l.free(dst)


def test_hbm_probe_reads_and_writes_only_what_it_is_given(rt, L):
    """The one-direction probes behind the bench's copy bound: the write probe
    fills the buffer with (1, 2, 3, vector index) and stays inside it, the
    read probe changes nothing."""
    l = rt.up(P, HEAP)
    pr = L.load_probes()
    n = 4 << 20
    buf = l.malloc(n + 4096)
    l.fill(buf, 0x6B, n + 4096)
    assert pr.hbm_probe(0, buf, n, None) == 0
    assert pr.reuse_probe(buf, n, 65536, 3, 64, 256, None) == 0
    l.stream_sync(None)
    assert (rt.get_bytes(buf, n + 4096) == 0x6B).all()
    assert pr.reuse_probe(buf, n, 100, 3, 64, 256, None) == -1  # tiles are whole vectors
    assert pr.hbm_probe(1, buf, n, None) == 0
    l.stream_sync(None)
    got = rt.get_bytes(buf, n + 4096, np.uint32)
    body = got[:n // 4].reshape(-1, 4)
    idx = np.arange(n // 16, dtype=np.uint32)
    assert np.array_equal(body, np.stack([np.ones_like(idx), 2 * np.ones_like(idx),
                                          3 * np.ones_like(idx), idx], 1))
    assert (got[n // 4:].view(np.uint8) == 0x6B).all()   # nothing past the end
    assert pr.hbm_probe(0, buf + 4, n, None) == -1         # misaligned
    assert pr.hbm_probe(1, buf, 1024, None) == -1          # too small to mean anything
    assert pr.hbm_probe(1, None, n, None) == -1
    l.free(buf)


def test_argument_errors_launch_nothing(rt, L, env):
    l = env["l"]
    src, dst = env["src"], env["dst"]
    assert l.rma(L.PUT, L.WG, dst, src, 16, 0, 0, P, 1, 64, 1, None) == -1       # bad PE
    assert l.rma(L.PUT, L.WG, dst, src, 16, 0, 0, 1, 1, 2048, 1, None) == -1     # bad block
    assert l.rma(L.PUT, L.WG, None, src, 16, 0, 0, 1, 1, 64, 1, None) == -1      # null dest
    assert l.rma(L.PUT, L.WG, dst, src, HEAP + 1, 0, 0, 1, 1, 64, 1, None) == -1 # beyond the slice
    assert l.rma(L.PUT, L.WG, l.pe_ptr(dst, 1), src, 16, 0, 0, 1, 1, 64, 1, None) == -1  # not my_pe's address
    assert l.putmem(dst, src, HEAP, 0, 1, None) == -1
    assert l.rma(7, L.WG, dst, src, 16, 0, 0, 1, 1, 64, 1, None) == -1


@pytest.mark.parametrize("ctx_options", [0, 1])
@pytest.mark.parametrize("gran_name,wg_size", [("WG", 256), ("WG", 1024), ("WG", 192), ("WAVE", 128),
                                               ("THREAD", 64)])
@pytest.mark.parametrize("n", [1, 15, 16, 17, 4096, 4099, 24576])
def test_local_buffer_in_lds(rt, L, orc, env, gran_name, wg_size, n, ctx_options):
    """The local side of a put and of a get may be a __shared__ array, as with
    the reference's generic-pointer copy (src/util.hpp:170-262): put from LDS,
    get back into LDS at an odd offset, both byte-exact."""
    l = env["l"]
    src, dst, host = env["src"], env["dst"], env["host"]
    my_pe, pe, soff, doff = 2, 5, 5, GUARD + 3
    rt.put_bytes(l.pe_ptr(src, my_pe), host[:soff + n])
    landing = l.pe_ptr(dst, pe) + doff
    l.fill(landing - GUARD, 0xA5, n + 2 * GUARD)
    back = l.dev_alloc(n)
    l.fill(back, 0x5A, n)
    before = l.set_ctx_options(ctx_options)
    rc = l.rma_staged(getattr(L, gran_name), l.pe_ptr(dst, my_pe) + doff, l.pe_ptr(src, my_pe) + soff,
                      back, n, my_pe, pe, wg_size, None)
    l.set_ctx_options(before)
    assert rc == 0
    l.stream_sync(None)
    want = np.full(n + 2 * GUARD, 0xA5, np.uint8)
    exp = np.empty(n, np.uint8)
    orc.lib.orc_copy(exp.ctypes.data, host[soff:soff + n].ctypes.data, n)
    want[GUARD:GUARD + n] = exp
    assert np.array_equal(rt.get_bytes(landing - GUARD, n + 2 * GUARD), want)
    assert np.array_equal(rt.get_bytes(back, n), exp)
    l.dev_free(back)
    assert l.rma_staged(L.WG, l.pe_ptr(dst, my_pe), l.pe_ptr(src, my_pe), back, 24577, my_pe, pe, 256,
                        None) == -1


@pytest.mark.parametrize("shape", [(64, 1, 1), (256, 1, 1), (1024, 1, 1), (32, 8, 1), (16, 4, 4),
                                   (7, 5, 3), (1, 1, 64), (3, 1, 1), (1, 1000, 1)])
def test_work_group_rank_and_size_for_any_block_shape(env, shape):
    """Every thread of a 1-, 2- or 3-D block gets a distinct rank
    x + y*X + z*X*Y below X*Y*Z (src/util.hpp:100-118)."""
    l = env["l"]
    out = np.zeros(1026, np.uint32)
    assert l.flat_ids(shape[0], shape[1], shape[2], out.ctypes.data) == 0
    n = shape[0] * shape[1] * shape[2]
    assert out[0] == n
    assert (out[1:1 + n] == 1).all() and (out[1 + n:] == 0).all()


@pytest.mark.parametrize("lanes,gran_name", [(64, "WG"), (192, "WG"), (256, "WG"), (1024, "WG"),
                                             (64, "WAVE"), (37, "WAVE")])
def test_sizes_around_the_burst_boundaries(rt, L, orc, env, lanes, gran_name):
    """A lane moves bursts of eight 16-byte vectors: message sizes either side
    of 1, 7, 8, 9 and 16 vectors per lane, of the 64-byte single-wavefront
    path and of the non-temporal threshold, with misaligned ends."""
    g = getattr(L, gran_name)
    per = lanes * 16
    sizes = set()
    for k in (1, 7, 8, 9, 16):
        for d in (-17, -16, -1, 0, 1, 16, 33):
            sizes.add(k * per + d)
    sizes.update((63, 64, 65, 4095, 4096, 4097))
    for i, n in enumerate(sorted(s for s in sizes if 0 < s <= (4 << 20))):
        run_case(rt, L, orc, env, L.PUT, g, n, i % 16, (3 * i) % 16, 1, lanes, ctx_options=i & 1)
        run_case(rt, L, orc, env, L.GET, g, n, (5 * i) % 16, i % 16, 1, lanes)
