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
