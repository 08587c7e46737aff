"""The thin runtime layer (include/nslm_rt.h) on the GPU: the calls the reference's C99 hosts make of the CUDA runtime beyond
plain allocation and copies - mapped host memory, asynchronous fills and copies on a stream, a fill inside a replayed graph,
events across two streams (engine/mova_cuda.c:352, 892-896, 1160, 1289-1303; engine/qwen4_cuda.c:186, 397)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from nanoseedlm_amd import backend
    backend.require_gpu()
    return backend.hip()


def ok(rc, what):
    assert rc == 0, (what, rc)


def test_mapped_host_memory_is_written_by_the_gpu(rt):
    """nh_host_alloc_mapped: a fill on the device address of pinned host memory is what the host reads after the stream's end
    (results a kernel leaves for the host; expert units a copy kernel reads from host memory go the other way)."""
    n = 1 << 16
    host, dev, dev2, s = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
    ok(rt.nh_host_alloc_mapped(C.byref(host), C.byref(dev), C.c_size_t(n)), "nh_host_alloc_mapped")
    ok(rt.nh_host_device_ptr(C.byref(dev2), host), "nh_host_device_ptr")
    assert dev.value == dev2.value and dev.value
    view = np.ctypeslib.as_array(C.cast(host, C.POINTER(C.c_uint8)), shape=(n,))
    view[:] = 7
    ok(rt.nh_stream_create(C.byref(s)), "nh_stream_create")
    ok(rt.nh_memset_async(C.c_void_p(dev.value + 5), 0xAB, C.c_size_t(n - 9), s), "nh_memset_async")   # ragged ends on both sides
    ok(rt.nh_stream_sync(s), "nh_stream_sync")
    assert (view[:5] == 7).all() and (view[5:n - 4] == 0xAB).all() and (view[n - 4:] == 7).all()
    # the other way: the device copies from the mapped memory
    d = C.c_void_p()
    ok(rt.nh_malloc(C.byref(d), C.c_size_t(n)), "nh_malloc")
    view[:] = np.arange(n, dtype=np.uint32).astype(np.uint8)
    ok(rt.nh_memcpy_async(d, dev, C.c_size_t(n), s), "nh_memcpy_async")
    back = np.zeros(n, dtype=np.uint8)
    ok(rt.nh_memcpy_d2h_async(back.ctypes.data_as(C.c_void_p), d, C.c_size_t(n), s), "nh_memcpy_d2h_async")
    ok(rt.nh_stream_sync(s), "nh_stream_sync")
    assert np.array_equal(back, view)
    ok(rt.nh_free(d), "nh_free"); ok(rt.nh_stream_destroy(s), "nh_stream_destroy"); ok(rt.nh_host_free(host), "nh_host_free")


def test_async_fill_in_a_replayed_graph(rt):
    """nh_memset_async is a kernel, so it may be captured: every replay clears the buffer again (checked on three replays with
    the buffer dirtied in between), sizes from one byte to ragged megabytes."""
    from nanoseedlm_amd import backend
    K = backend.host()
    K.nslm_graph_end.restype = C.c_void_p
    s = C.c_void_p()
    ok(rt.nh_stream_create(C.byref(s)), "nh_stream_create")
    for n, off in ((1, 0), (15, 1), (16, 0), (4097, 3), (3 * 1024 * 1024 + 5, 7)):
        d = C.c_void_p()
        ok(rt.nh_malloc(C.byref(d), C.c_size_t(n + 32)), "nh_malloc")
        ok(K.nslm_graph_begin(s), "nslm_graph_begin")
        ok(rt.nh_memset_async(C.c_void_p(d.value + off), 0x5A, C.c_size_t(n), s), "nh_memset_async")
        g = C.c_void_p(K.nslm_graph_end(s))
        assert g.value
        for rep in range(3):
            ok(rt.nh_memset(d, rep + 1, C.c_size_t(n + 32)), "nh_memset")
            ok(rt.nh_device_sync(), "nh_device_sync")     # the fill of the default stream is not ordered before work on s
            ok(K.nslm_graph_launch(g, s), "nslm_graph_launch")
            ok(rt.nh_stream_sync(s), "nh_stream_sync")
            back = np.zeros(n + 32, dtype=np.uint8)
            ok(rt.nh_memcpy_d2h(back.ctypes.data_as(C.c_void_p), d, C.c_size_t(n + 32)), "nh_memcpy_d2h")
            assert (back[:off] == rep + 1).all() and (back[off:off + n] == 0x5A).all() and (back[off + n:] == rep + 1).all(), (n, rep)
        K.nslm_graph_free(g)
        ok(rt.nh_free(d), "nh_free")
    ok(rt.nh_stream_destroy(s), "nh_stream_destroy")


def test_events_order_two_streams(rt):
    """The copy-stream pattern of the engine (record on the compute stream, wait on the copy stream, record there, wait back:
    engine/mova_cuda.c:1296-1302) with untimed events, on streams made through the priority calls (one priority here)."""
    lo, hi = C.c_int(9), C.c_int(9)
    ok(rt.nh_stream_priority_range(C.byref(lo), C.byref(hi)), "nh_stream_priority_range")
    assert (lo.value, hi.value) == (0, 0)
    a, b, e1, e2 = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
    ok(rt.nh_stream_create(C.byref(a)), "nh_stream_create")
    ok(rt.nh_stream_create_prio(C.byref(b), hi.value), "nh_stream_create_prio")
    ok(rt.nh_event_create_untimed(C.byref(e1)), "nh_event_create_untimed")
    ok(rt.nh_event_create_untimed(C.byref(e2)), "nh_event_create_untimed")
    n = 8 << 20
    x, y, z = C.c_void_p(), C.c_void_p(), C.c_void_p()
    for p in (x, y, z):
        ok(rt.nh_malloc(C.byref(p), C.c_size_t(n)), "nh_malloc")
    for rep in range(4):
        ok(rt.nh_memset_async(x, 0x10 + rep, C.c_size_t(n), a), "fill x on a")
        ok(rt.nh_event_record(e1, a), "record")
        ok(rt.nh_stream_wait_event(b, e1), "wait")
        ok(rt.nh_memcpy_d2d_async(y, x, C.c_size_t(n), b), "copy x -> y on b")
        ok(rt.nh_event_record(e2, b), "record")
        ok(rt.nh_stream_wait_event(a, e2), "wait")
        ok(rt.nh_memcpy_d2d_async(z, y, C.c_size_t(n), a), "copy y -> z on a")
        ok(rt.nh_stream_sync(a), "sync")
        back = np.zeros(n, dtype=np.uint8)
        ok(rt.nh_memcpy_d2h(back.ctypes.data_as(C.c_void_p), z, C.c_size_t(n)), "d2h")
        assert (back == 0x10 + rep).all(), rep
    dev = C.c_int(-1)
    ok(rt.nh_get_device(C.byref(dev)), "nh_get_device")
    assert dev.value == 0
    for p in (x, y, z):
        ok(rt.nh_free(p), "nh_free")
    for e in (e1, e2):
        ok(rt.nh_event_destroy(e), "nh_event_destroy")
    for s in (a, b):
        ok(rt.nh_stream_destroy(s), "nh_stream_destroy")
