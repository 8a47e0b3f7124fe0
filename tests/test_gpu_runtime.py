"""GPU tests of the runtime half of the C ABI: the memory, stream, event and
graph contract that every kernel test (and the C engine) relies on.

The cases are those of the reference's tests/test_device_memory.c (copies in
every direction through offsets and odd sizes, stream-ordered fills, the
device-side index copy and position add, ordering across streams by events,
pinned sources, capture once / replay many, a capture broken by a sync) and of
tests/test_decode_position.c:70-112, driven through ctypes with host buffers
held by numpy.
"""
import ctypes as C

import numpy as np
import pytest

from gpu_util import dev

pytestmark = pytest.mark.gpu


def alloc(n):
    p = C.c_void_p()
    assert dev.vv_dev_alloc(C.byref(p), n) == dev.VV_OK and p.value
    return p.value


def new_stream():
    s = C.c_void_p()
    assert dev.vv_dev_stream_create(C.byref(s)) == dev.VV_OK and s.value
    return s.value


def pattern(n, seed):
    i = np.arange(n, dtype=np.uint64)
    return (((i * 131 + seed * 7) ^ (i >> 8)) & 0xFF).astype(np.uint8)


def h2d(dst, arr, st=None):
    assert dev.vv_dev_memcpy_h2d(dst, arr.ctypes.data, arr.nbytes, st) == dev.VV_OK


def d2h(src, n, st=None):
    out = np.zeros(n, dtype=np.uint8)
    assert dev.vv_dev_memcpy_d2h(out.ctypes.data, src, n, st) == dev.VV_OK
    if st:
        assert dev.vv_dev_stream_sync(st) == dev.VV_OK
    return out


def dev_int(v):
    p = alloc(4)
    h2d(p, np.array([v], dtype=np.int32))
    return p


def read_int(p, st=None):
    return int(d2h(p, 4, st).view(np.int32)[0])


def test_device_info():
    assert dev.vv_dev_device_count() >= 1
    total, free, cus = C.c_size_t(), C.c_size_t(), C.c_int()
    assert dev.vv_dev_get_device_info(0, C.byref(total), C.byref(free), C.byref(cus)) == dev.VV_OK
    assert total.value > 0 and free.value <= total.value and cus.value > 0
    name = C.create_string_buffer(128)
    assert dev.vv_dev_get_device_name(0, name, 128) == dev.VV_OK and name.value
    assert dev.vv_dev_set_device(0) == dev.VV_OK
    assert dev.vv_dev_enable_peer(0, 0) == dev.VV_OK


def test_copies_offsets_and_odd_sizes():
    N = (1 << 20) + 37
    h = pattern(N, 1)
    a, b = alloc(N), alloc(N)
    st = new_stream()
    h2d(a, h)
    assert np.array_equal(d2h(a, N), h)                   # round trip, default stream
    for o in (0, 1, 3, 16, 4093):
        for n in (1, 7, 16, 4096, 65537):
            assert dev.vv_dev_memset_async(b, 0xEE, N, st) == dev.VV_OK
            assert dev.vv_dev_memcpy_d2d(b + o, a + 5, n, st) == dev.VV_OK
            back = d2h(b, o + n + 1, st)
            assert np.array_equal(back[o:o + n], h[5:5 + n]), (o, n)
            assert (back[:o] == 0xEE).all() and back[o + n] == 0xEE, (o, n)
    # a host copy queued behind a fill on the same stream lands after it
    src = pattern(N, 9)
    assert dev.vv_dev_memset_async(b, 0x11, N, st) == dev.VV_OK
    assert dev.vv_dev_memcpy_h2d(b + 100, src.ctypes.data, 3000, st) == dev.VV_OK
    assert dev.vv_dev_memcpy_h2d(b + 5000, src.ctypes.data, 200000, st) == dev.VV_OK
    got = d2h(b, 205000, st)
    assert np.array_equal(got[100:3100], src[:3000]) and np.array_equal(got[5000:205000], src[:200000])
    assert got[99] == 0x11 and got[3100] == 0x11 and got[4999] == 0x11
    # synchronous fill
    assert dev.vv_dev_memset(a, 0x5A, 1000) == dev.VV_OK
    got = d2h(a, 1001, st)
    assert (got[:1000] == 0x5A).all() and got[1000] == h[1000]
    assert dev.vv_dev_stream_destroy(st) == dev.VV_OK
    assert dev.vv_dev_free(a) == dev.VV_OK and dev.vv_dev_free(b) == dev.VV_OK


@pytest.mark.parametrize("off,size", [(0, 1), (1, 15), (5, 16), (7, 100), (16, 4096), (3, 1 << 20),
                                      (0, (64 << 20) + 5)])
def test_memset_async_fill_kernel_any_alignment(off, size):
    n = size + off + 64
    p = alloc(n)
    st = new_stream()
    assert dev.vv_dev_memset(p, 0, n) == dev.VV_OK
    assert dev.vv_dev_memset_async(p + off, 0xA7, size, st) == dev.VV_OK
    got = d2h(p, n, st)
    assert not got[:off].any() and (got[off:off + size] == 0xA7).all() and not got[off + size:].any()
    dev.vv_dev_stream_destroy(st)
    dev.vv_dev_free(p)


def test_device_side_index_and_position():
    """tests/test_decode_position.c:70-112 and test_device_memory.c:106-136."""
    a, b = dev_int(41), dev_int(0)
    assert dev.vv_pos_add_dev(b, a, 1, None) == dev.VV_OK and read_int(b) == 42
    assert dev.vv_pos_add_dev(a, a, 1, None) == dev.VV_OK and read_int(a) == 42   # in place

    st = new_stream()
    RB, NR = 48, 64
    pos, pos2, rows, row = alloc(4), alloc(4), alloc(RB * NR), alloc(RB)
    h2d(pos, np.array([7], dtype=np.int32), st)
    assert dev.vv_pos_add_dev(pos2, pos, 5, st) == dev.VV_OK
    assert read_int(pos2, st) == 12
    h = (200 + np.arange(48)).astype(np.uint8)
    assert dev.vv_dev_memset_async(rows, 0, RB * NR, st) == dev.VV_OK
    h2d(row, h, st)
    assert dev.vv_dev_memcpy_d2d_at(rows, row, RB, pos2, st) == dev.VV_OK     # 16-byte rows
    assert dev.vv_dev_memcpy_d2d_at(rows, row, 20, pos, st) == dev.VV_OK      # odd row size
    back = d2h(rows, RB * NR, st)
    assert np.array_equal(back[12 * RB:13 * RB], h)
    assert np.array_equal(back[7 * 20:8 * 20], h[:20])
    assert back[12 * RB - 1] == 0 and back[13 * RB] == 0

    # one 512-byte row at index 7 of 16, nothing else touched
    base, src, idx = alloc(512 * 16), alloc(512), dev_int(7)
    assert dev.vv_dev_memset(base, 0, 512 * 16) == dev.VV_OK
    pat = ((np.arange(512) * 7 + 3) & 0xFF).astype(np.uint8)
    h2d(src, pat)
    assert dev.vv_dev_memcpy_d2d_at(base, src, 512, idx, None) == dev.VV_OK
    assert dev.vv_dev_stream_sync(None) == dev.VV_OK
    got = d2h(base, 512 * 16)
    assert np.array_equal(got[7 * 512:8 * 512], pat)
    assert not got[:7 * 512].any() and not got[8 * 512:].any()
    dev.vv_dev_stream_destroy(st)
    for p in (a, b, pos, pos2, rows, row, base, src, idx):
        dev.vv_dev_free(p)


def test_events_order_two_streams_and_pinned_source():
    N = 8 << 20
    h = pattern(N, 3)
    x, y, z = alloc(N), alloc(N), alloc(N)
    s1, s2 = new_stream(), new_stream()
    ev = C.c_void_p()
    assert dev.vv_dev_event_create(C.byref(ev)) == dev.VV_OK
    h2d(x, h)
    for _ in range(4):
        assert dev.vv_dev_memset_async(z, 0, N, s2) == dev.VV_OK
        assert dev.vv_dev_stream_sync(s2) == dev.VV_OK
        for _ in range(8):
            assert dev.vv_dev_memcpy_d2d(y, x, N, s1) == dev.VV_OK
        assert dev.vv_dev_event_record(ev, s1) == dev.VV_OK
        assert dev.vv_dev_stream_wait_event(s2, ev) == dev.VV_OK
        assert dev.vv_dev_memcpy_d2d(z, y, N, s2) == dev.VV_OK
        assert dev.vv_dev_event_sync(ev) == dev.VV_OK
        assert np.array_equal(d2h(z, N, s2), h)

    pin = C.c_void_p()
    assert dev.vv_dev_alloc_pinned(C.byref(pin), N) == dev.VV_OK and pin.value
    C.memmove(pin.value, h.ctypes.data, N)
    assert dev.vv_dev_memset_async(z, 0, N, s1) == dev.VV_OK
    assert dev.vv_dev_memcpy_h2d(z, pin.value, N, s1) == dev.VV_OK
    assert dev.vv_dev_event_record(ev, s1) == dev.VV_OK
    assert dev.vv_dev_event_sync(ev) == dev.VV_OK
    C.memset(pin.value, 0, N)                 # safe: the copy has run
    assert np.array_equal(d2h(z, N, s1), h)
    assert dev.vv_dev_free_pinned(pin.value) == dev.VV_OK
    assert dev.vv_dev_event_destroy(ev.value) == dev.VV_OK
    dev.vv_dev_stream_destroy(s1)
    dev.vv_dev_stream_destroy(s2)
    for p in (x, y, z):
        dev.vv_dev_free(p)


def test_graph_capture_once_replay_many():
    """test_device_memory.c:164-212: the captured step writes a row at *pos and
    advances *pos; every replay is checked, with eager work between replays."""
    RB, NR = 32, 16
    pos, rows, row = alloc(4), alloc(RB * NR), alloc(RB)
    st = new_stream()
    h2d(pos, np.array([0], dtype=np.int32), st)
    assert dev.vv_dev_memset_async(rows, 0, RB * NR, st) == dev.VV_OK
    h = (np.arange(32) + 1).astype(np.uint8)
    h2d(row, h, st)
    assert dev.vv_dev_stream_sync(st) == dev.VV_OK

    assert dev.vv_dev_graph_begin(st) == dev.VV_OK
    assert dev.vv_dev_memcpy_d2d_at(rows, row, RB, pos, st) == dev.VV_OK
    assert dev.vv_pos_add_dev(pos, pos, 1, st) == dev.VV_OK
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) == dev.VV_OK and g.value
    assert read_int(pos, st) == 0                       # capture ran nothing
    for i in range(5):
        assert dev.vv_dev_graph_launch(g.value, st) == dev.VV_OK
        assert read_int(pos, st) == i + 1               # eager read-back + sync between replays
        back = d2h(rows, RB * NR, st).reshape(NR, RB)
        assert (back[:i + 1] == h).all() and not back[i + 1:].any()
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(st)
    for p in (pos, rows, row):
        dev.vv_dev_free(p)


def test_graph_with_fill_and_rope_at_device_position():
    """A decode-step-shaped graph: stream-ordered fill (a kernel here, so it is
    capturable), RoPE reading its position from device memory, position add.
    Each replay must equal the eager call at that position, bit for bit."""
    import torch
    import oracle
    from gpu_util import bits_of, to_dev

    NQ, HD = 28, 128
    q0 = oracle.normal_f16((1, NQ, HD), 77)
    work = torch.empty(1, NQ, HD, dtype=torch.float16, device="cuda")
    src = to_dev(q0)
    scratch = torch.ones(1024, dtype=torch.uint8, device="cuda")
    d_pos = torch.tensor([100], dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    st = new_stream()
    assert dev.vv_dev_graph_begin(st) == dev.VV_OK
    assert dev.vv_dev_memset_async(scratch.data_ptr(), 0x3C, 1000, st) == dev.VV_OK
    assert dev.vv_dev_memcpy_d2d(work.data_ptr(), src.data_ptr(), NQ * HD * 2, st) == dev.VV_OK
    assert dev.vv_rope_dev(work.data_ptr(), 1, NQ, HD, 0, d_pos.data_ptr(), 1e6, st) == dev.VV_OK
    assert dev.vv_pos_add_dev(d_pos.data_ptr(), d_pos.data_ptr(), 1, st) == dev.VV_OK
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) == dev.VV_OK and g.value
    for i in range(4):
        scratch.fill_(1)
        torch.cuda.synchronize()
        assert dev.vv_dev_graph_launch(g.value, st) == dev.VV_OK
        assert dev.vv_dev_stream_sync(st) == dev.VV_OK
        eager = to_dev(q0)
        assert dev.vv_rope_dev(eager.data_ptr(), 1, NQ, HD, 100 + i, None, 1e6, None) == dev.VV_OK
        assert np.array_equal(bits_of(work), bits_of(eager)), f"replay {i}"
        sc = scratch.cpu().numpy()
        assert (sc[:1000] == 0x3C).all() and (sc[1000:] == 1).all()
        assert int(d_pos.item()) == 101 + i
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(st)


def test_sync_inside_a_capture_breaks_it_cleanly():
    """test_device_memory.c:203-208: an uncapturable call fails the capture
    instead of running, and the error does not linger."""
    st = new_stream()
    assert dev.vv_dev_graph_begin(st) == dev.VV_OK
    dev.vv_dev_stream_sync(st)                          # not capturable
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) != dev.VV_OK and not g.value
    # the stream and the device are still usable afterwards
    p = dev_int(5)
    assert dev.vv_pos_add_dev(p, p, 2, st) == dev.VV_OK
    assert read_int(p, st) == 7
    dev.vv_dev_free(p)
    dev.vv_dev_stream_destroy(st)
