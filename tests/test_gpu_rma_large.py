"""C3, H3 at the top of the size range: one message larger than 4 GiB, through
the host-initiated copy (more 1 KiB pieces than the grid has work-groups) and
through the device-API work-group put (several 1 GiB store windows per tile),
checked whole against the source.  Through the C entry points."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P, HEAP = 2, 8 << 30


def test_message_beyond_4gib(rt, L):
    l = rt.up(P, HEAP)
    n = (4 << 30) + (1 << 20) + 13
    room = n + 64
    dst = l.malloc(room)                      # the 8 GiB bin: the whole slice
    assert dst
    words = np.arange((room + 7) // 8, dtype=np.uint64)
    words *= np.uint64(0x9E3779B97F4A7C15)    # every 8 bytes differ
    host = words.view(np.uint8)[:room]
    src = l.dev_alloc(room)
    assert src
    assert l.copy_in(src, host.ctypes.data, room) == 0
    for mode in ("host", "device"):
        assert l.fill(l.pe_ptr(dst, 1), 0, room) == 0
        if mode == "host":
            assert l.putmem(dst + 3, src + 5, n, 0, 1, None) == 0
        else:
            assert l.rma(L.PUT, L.WG, dst + 3, src + 5, n, 0, 0, 1, 2, 1024, 1, None) == 0
        l.stream_sync(None)
        got = rt.get_bytes(l.pe_ptr(dst, 1), room)
        assert np.array_equal(got[3:3 + n], host[5:5 + n]), mode
        assert not got[:3].any() and not got[3 + n:].any(), mode
        del got
    l.dev_free(src)
    l.free(dst)
