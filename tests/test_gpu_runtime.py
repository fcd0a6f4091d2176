"""The library's memory, stream, event and timing entry points, called through the C ABI the way a
host binding would: every one of them is exercised here with a checkable effect."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_device_and_memory_info(gpu):
    info = gpu.device_info()
    assert info["arch"].startswith("gfx950") and info["wavefront"] == 64 and info["cu_count"] > 0
    free, total = C.c_int64(0), C.c_int64(0)
    gpu.api.anc_mem_info(C.byref(free), C.byref(total))
    assert 0 < free.value <= total.value == info["hbm_bytes"]
    p = C.c_uint64(0)
    gpu.api.anc_malloc(C.byref(p), 1 << 30)
    free2 = C.c_int64(0)
    gpu.api.anc_mem_info(C.byref(free2), C.byref(total))
    assert free.value - free2.value >= 0.9 * (1 << 30)      # the runtime reports in its own granules
    gpu.api.anc_free(p.value)


def test_pinned_buffers_async_copies_and_fill(gpu):
    """Pinned host memory from the library, asynchronous copies on a created stream, the fill
    kernel and a device-to-device copy: what arrives is what was sent."""
    api = gpu.api
    n = 1 << 20
    s = gpu.stream_create()
    h_in, h_out = C.c_void_p(), C.c_void_p()
    api.anc_host_alloc(C.byref(h_in), 4 * n)
    api.anc_host_alloc(C.byref(h_out), 8 * n)
    a_in = np.ctypeslib.as_array(C.cast(h_in, C.POINTER(C.c_uint32)), (n,))
    a_out = np.ctypeslib.as_array(C.cast(h_out, C.POINTER(C.c_uint32)), (2 * n,))
    a_in[:] = np.random.default_rng(0).integers(0, 2**32, n, dtype=np.uint32)
    a_out[:] = 0
    d0, d1 = C.c_uint64(0), C.c_uint64(0)
    api.anc_malloc(C.byref(d0), 4 * n)
    api.anc_malloc(C.byref(d1), 8 * n)
    api.anc_memcpy_h2d(d0.value, h_in, 4 * n, s)
    api.anc_fill_u32(d1.value, 0xDEADBEEF, 2 * n, s)
    api.anc_memcpy_d2d(d1.value + 4 * n, d0.value, 4 * n, s)
    api.anc_memcpy_d2h(h_out, d1.value, 8 * n, s)
    api.anc_stream_sync(s)
    assert np.all(a_out[:n] == 0xDEADBEEF) and np.array_equal(a_out[n:], a_in)
    # ragged fill: only the words asked for
    api.anc_fill_u32(d1.value, 7, 3, s)
    api.anc_memcpy_d2h(h_out, d1.value, 32, s)
    api.anc_stream_sync(s)
    assert list(a_out[:5]) == [7, 7, 7, 0xDEADBEEF, 0xDEADBEEF]
    for d in (d0, d1):
        api.anc_free(d.value)
    api.anc_host_free(h_in)
    api.anc_host_free(h_out)
    api.anc_stream_destroy(s)


def test_events_order_two_streams(gpu):
    """Stream B waits for an event recorded on stream A behind a long fill: B's copy sees the
    filled values; the elapsed time between two events around the fill is positive."""
    api = gpu.api
    n = 1 << 28                                   # 1 GiB: the fill takes a fraction of a ms
    sa, sb = gpu.stream_create(), gpu.stream_create()
    d, tail = C.c_uint64(0), C.c_uint64(0)
    api.anc_malloc(C.byref(d), 4 * n)
    api.anc_malloc(C.byref(tail), 4096)
    api.anc_fill_u32(d.value, 1, n, 0)
    api.anc_fill_u32(tail.value, 0, 1024, 0)
    api.anc_device_sync()
    e0, e1 = gpu.Event(), gpu.Event()
    e0.record(sa)
    api.anc_fill_u32(d.value, 0x5A5A5A5A, n, sa)
    e1.record(sa)
    e1.wait_on(sb)
    api.anc_memcpy_d2d(tail.value, d.value + 4 * n - 4096, 4096, sb)
    host = np.zeros(1024, np.uint32)
    api.anc_memcpy_d2h(host.ctypes.data_as(C.c_void_p), tail.value, 4096, sb)
    api.anc_stream_sync(sb)
    assert np.all(host == 0x5A5A5A5A)
    e1.sync()
    ms = e0.elapsed_ms(e1)
    assert 0.05 < ms < 50.0, ms                   # 1 GiB written: some tenths of a ms
    api.anc_free(d.value)
    api.anc_free(tail.value)
    api.anc_stream_destroy(sa)
    api.anc_stream_destroy(sb)


def test_profile_counts_the_launches_of_a_kind(gpu):
    api = gpu.api
    d = C.c_uint64(0)
    api.anc_malloc(C.byref(d), 1 << 20)
    gpu.profile_enable(True)
    gpu.profile_read()
    for _ in range(3):
        api.anc_fill_u32(d.value, 0, 1 << 18, 0)
    got = gpu.profile_read()
    gpu.profile_enable(False)
    assert got["misc"][1] == 3 and got["misc"][0] > 0.0
    assert all(v[1] == 0 for k, v in got.items() if k != "misc")
    api.anc_fill_u32(d.value, 0, 1 << 18, 0)
    assert all(v[1] == 0 for v in gpu.profile_read().values())     # disabled: nothing recorded
    api.anc_free(d.value)


def test_errors_carry_a_status_and_a_message(gpu):
    """Raw status codes, without the raising wrapper: a bad argument returns ANC_ERR_ARG and
    leaves its text in anc_last_error; a later good call returns 0."""
    lib = gpu.load()
    lib.anc_fill_u32.restype = C.c_int
    rc = lib.anc_fill_u32(C.c_uint64(0), C.c_uint32(0), C.c_int64(16), C.c_uint64(0))
    assert rc == 2
    assert b"anc_fill_u32" in lib.anc_last_error() or len(lib.anc_last_error()) > 0
    p = C.c_uint64(0)
    assert lib.anc_malloc(C.byref(p), C.c_int64(-1)) != 0
    assert lib.anc_malloc(C.byref(p), C.c_int64(4096)) == 0
    assert lib.anc_fill_u32(C.c_uint64(p.value), C.c_uint32(0), C.c_int64(16), C.c_uint64(0)) == 0
    assert lib.anc_free(C.c_uint64(p.value)) == 0
