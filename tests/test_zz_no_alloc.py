"""The allocation-free grad-norm entry point against the caller-buffer pair of entry points."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _ctl_bytes(ctl):
    return ctl.to_numpy().tobytes()


def _reference_ctl(api, DevBuf, g, n, code, max_norm, eps):
    parts = DevBuf.empty((api.anc_gradnorm_num_partials(n),), np.float64)
    ctl = DevBuf.zeros((8,), np.uint32)
    api.anc_gradnorm_partials(g.ptr, n, code, parts.ptr, 0, 0)
    api.anc_gradnorm_finalize(parts.ptr, parts.size, max_norm, eps, 0, ctl.ptr, 0)
    out = _ctl_bytes(ctl)
    parts.free(); ctl.free()
    return out


def test_static_gradnorm_matches_caller_buffer_entry(gpu):
    """Two calls in a row, the second on a smaller input (the built-in scratch keeps the first
    call's partial sums): each control block bit-equal to anc_gradnorm_partials + _finalize."""
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd.bf16 import bf16_bits
    api = _lib.api
    rng = np.random.default_rng(5)
    for n, dtype in ((3 * 8192 * 1024 + 4104, np.uint16), (8192 * 37 + 8, np.uint16), (123456 * 8, np.float32),
                     (64, np.float32)):
        x = (1e-3 * rng.standard_normal(n)).astype(np.float32)
        host = bf16_bits(x) if dtype == np.uint16 else x
        code = _lib.BF16 if dtype == np.uint16 else _lib.F32
        g = DevBuf(host)
        want = _reference_ctl(api, DevBuf, g, n, code, 1.0, 1e-6)
        ctl = DevBuf.zeros((8,), np.uint32)
        api.anc_gradnorm_static(g.ptr, n, code, 1.0, 1e-6, ctl.ptr, 0)
        assert _ctl_bytes(ctl) == want, (n, dtype)
        g.free(); ctl.free()


def test_static_gradnorm_nonfinite_and_limits(gpu):
    from ancora_cutile_amd import DevBuf, _lib
    api = _lib.api
    x = np.ones(8192 * 3, np.float32)
    x[9000] = np.inf
    g = DevBuf(x)
    ctl = DevBuf.zeros((8,), np.uint32)
    api.anc_gradnorm_static(g.ptr, x.size, _lib.F32, 1.0, 1e-6, ctl.ptr, 0)
    assert _ctl_bytes(ctl) == _reference_ctl(api, DevBuf, g, x.size, _lib.F32, 1.0, 1e-6)
    assert ctl.to_numpy()[4] == 1                      # skip flag
    assert api.anc_gradnorm_static_max_elements() == 2 ** 31
    with pytest.raises(_lib.AncoraError):
        api.anc_gradnorm_static(g.ptr, 2 ** 31 + 1, _lib.F32, 1.0, 1e-6, ctl.ptr, 0)
    g.free(); ctl.free()


def test_static_gradnorm_allocates_nothing(gpu):
    """Free device memory is the same before and after the calls, on the null stream and on a
    created one; calls on one stream are ordered, so back-to-back calls there need nothing else."""
    import ctypes
    from ancora_cutile_amd import DevBuf, _lib
    api = _lib.api
    n = 1 << 26
    g = DevBuf.zeros((n,), np.uint16)
    ctl, ctl2 = DevBuf.zeros((8,), np.uint32), DevBuf.zeros((8,), np.uint32)
    s1 = _lib.stream_create()
    for st in (0, s1):
        api.anc_gradnorm_static(g.ptr, n, _lib.BF16, 1.0, 1e-6, ctl.ptr, st)       # symbol looked up, stream warm
        _lib.stream_sync(st)
    free0, free1, total = ctypes.c_int64(0), ctypes.c_int64(0), ctypes.c_int64(0)
    api.anc_mem_info(ctypes.byref(free0), ctypes.byref(total))
    for _ in range(3):
        api.anc_gradnorm_static(g.ptr, n, _lib.BF16, 1.0, 1e-6, ctl.ptr, 0)
    _lib.stream_sync(0)
    for _ in range(3):
        api.anc_gradnorm_static(g.ptr, n, _lib.BF16, 1.0, 1e-6, ctl2.ptr, s1)
    _lib.stream_sync(s1)
    api.anc_mem_info(ctypes.byref(free1), ctypes.byref(total))
    assert free1.value == free0.value
    assert _ctl_bytes(ctl) == _ctl_bytes(ctl2)
    api.anc_stream_destroy(s1)
    g.free(); ctl.free(); ctl2.free()


def test_static_gradnorm_first_call_without_init(gpu, tmp_path):
    """A process that never calls anc_init: the first anc_gradnorm_static looks the scratch array's
    address up itself and gives the sum of squares of the fixed-order oracle."""
    import subprocess
    import sys
    from ancora_cutile_amd import _lib
    from oracle import gradnorm_ref as gn
    x = (1e-3 * np.random.default_rng(3).standard_normal(8192 * 5 + 24)).astype(np.float32)
    np.save(tmp_path / "x.npy", x)
    code = f"""
import ctypes as C, numpy as np
lib = C.CDLL({_lib.LIB_PATH!r})
x = np.load({str(tmp_path / 'x.npy')!r})
u64 = C.c_uint64
g, ctl = u64(0), u64(0)
assert lib.anc_malloc(C.byref(g), C.c_int64(x.nbytes)) == 0 and lib.anc_malloc(C.byref(ctl), C.c_int64(32)) == 0
assert lib.anc_memcpy_h2d(g, x.ctypes.data_as(C.c_void_p), C.c_int64(x.nbytes), u64(0)) == 0
assert lib.anc_gradnorm_static(g, C.c_int64(x.size), C.c_int(0), C.c_float(1.0), C.c_float(1e-6), ctl, u64(0)) == 0
out = np.zeros(4, np.float64)
assert lib.anc_memcpy_d2h(out.ctypes.data_as(C.c_void_p), ctl, C.c_int64(32), u64(0)) == 0
print(repr(float(out[0])))
"""
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    assert float(r.stdout.strip().splitlines()[-1]) == gn.gradnorm_fixed([x])
