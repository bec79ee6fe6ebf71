"""The stream-taking entry points only launch kernels, so a caller can record
them into a HIP graph and replay it: a put, an all-reduce over what the put
delivered and an alltoall of the result are captured once and replayed with
fresh inputs between the replays; every replay must equal the oracle's result
for the inputs of that replay.  Through the C entry points; the stream and the
graph come from the HIP runtime directly."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P, HEAP = 4, 64 << 20


def hip():
    h = C.CDLL("libamdhip64.so")
    for name, args in {
        "hipStreamCreate": [C.POINTER(C.c_void_p)],
        "hipStreamDestroy": [C.c_void_p],
        "hipStreamSynchronize": [C.c_void_p],
        "hipStreamBeginCapture": [C.c_void_p, C.c_int],
        "hipStreamEndCapture": [C.c_void_p, C.POINTER(C.c_void_p)],
        "hipGraphInstantiate": [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t],
        "hipGraphLaunch": [C.c_void_p, C.c_void_p],
        "hipGraphExecDestroy": [C.c_void_p],
        "hipGraphDestroy": [C.c_void_p],
    }.items():
        fn = getattr(h, name)
        fn.restype = C.c_int
        fn.argtypes = args
    return h


def test_put_reduce_alltoall_replayed_from_a_graph(rt, L, orc):
    l = rt.up(P, HEAP)
    h = hip()
    n = 3 * 4096 + 4                      # int32 elements, divisible by P
    blk = n * 4 // P                      # bytes per alltoall block
    a, b, c, d = (l.malloc(n * 4) for _ in range(4))
    assert a and b and c and d
    stream = C.c_void_p()
    assert h.hipStreamCreate(C.byref(stream)) == 0
    graph, exe = C.c_void_p(), C.c_void_p()
    assert h.hipStreamBeginCapture(stream, 0) == 0        # hipStreamCaptureModeGlobal
    # every PE p puts its a into the b of PE (p+1)%P; all-reduce b -> c; alltoall c -> d
    for p in range(P):
        assert l.putmem(l.pe_ptr(b, p), l.pe_ptr(a, p), n * 4, p, (p + 1) % P, stream) == 0
    assert l.to_all(L.INT, L.SUM, c, b, n, 0, 0, P, stream) == 0
    assert l.alltoallmem(l.team_world(), d, c, blk, stream) == 0
    assert h.hipStreamEndCapture(stream, C.byref(graph)) == 0 and graph.value
    assert h.hipGraphInstantiate(C.byref(exe), graph, None, None, 0) == 0 and exe.value
    try:
        for replay in range(4):
            srcs = [orc.fill_i32_pm1000(n, 40 + replay, p) for p in range(P)]
            for p in range(P):
                rt.put_bytes(l.pe_ptr(a, p), srcs[p])
                for buf in (b, c, d):
                    l.fill(l.pe_ptr(buf, p), 0xEE, n * 4)
            l.stream_sync(None)
            assert h.hipGraphLaunch(exe, stream) == 0
            assert h.hipStreamSynchronize(stream) == 0
            total = orc.to_all(L.INT, L.SUM, srcs)       # a sum does not care who holds which
            want_d = orc.alltoall([total] * P, blk)
            for p in range(P):
                got_b = rt.get_bytes(l.pe_ptr(b, p), n * 4, np.int32)
                assert np.array_equal(got_b, srcs[(p - 1) % P]), (replay, p, "put")
                got_c = rt.get_bytes(l.pe_ptr(c, p), n * 4, np.int32)
                assert np.array_equal(got_c, total), (replay, p, "to_all")
                got_d = rt.get_bytes(l.pe_ptr(d, p), n * 4)
                assert np.array_equal(got_d, want_d[p]), (replay, p, "alltoall")
    finally:
        h.hipGraphExecDestroy(exe)
        h.hipGraphDestroy(graph)
        h.hipStreamDestroy(stream)
        for buf in (a, b, c, d):
            l.free(buf)
