"""GPU parity of the MXFP8 weight re-quantisation against the numpy oracle: bit-exact bytes in
both output layouts, every bf16 bit pattern, degenerate blocks, and the lazy refresh protocol."""
import numpy as np
import pytest

from oracle.quant_ref import quant_mxfp8_w as ref_quant, dequant_mxfp8_w
from oracle.bf16_ref import bf16_rne_bits, bits_to_f32

pytestmark = pytest.mark.gpu


def _run(wb, E, K, N, cm):
    from ancora_cutile_amd import DevBuf, quant_mxfp8_w
    wd = DevBuf(wb.reshape(E * K, N))
    f = DevBuf.zeros((E * N, K) if cm else (E * K, N), np.uint8)
    s = DevBuf.zeros((E * N, K // 32) if cm else (E * K // 32, N), np.uint8)
    quant_mxfp8_w(wd, f, s, K, N, 0, E=E, col_major=cm)
    out = f.to_numpy(), s.to_numpy()
    for b in (wd, f, s):
        b.free()
    return out


@pytest.mark.parametrize("E,K,N", [(1, 128, 128), (1, 256, 384), (3, 128, 256), (1, 1024, 3072)])
@pytest.mark.parametrize("cm", [False, True])
def test_bytes_match_the_oracle(gpu, E, K, N, cm):
    rng = np.random.default_rng(E + K + N)
    w = (0.05 * rng.standard_normal((E, K, N))).astype(np.float32)
    w[:, ::7, ::5] *= 1e-4                      # elements far below their block's amax: subnormal / zero results
    w[0, :32, :8] = 0                           # blocks of zeros
    wb = bf16_rne_bits(w).reshape(E, K, N)
    f, s = _run(wb, E, K, N, cm)
    for e in range(E):
        wf, ws = ref_quant(wb[e], col_major=cm)
        rows_f, rows_s = wf.shape[0], ws.shape[0]
        assert np.array_equal(f[e * rows_f:(e + 1) * rows_f], wf)
        assert np.array_equal(s[e * rows_s:(e + 1) * rows_s], ws)


@pytest.mark.parametrize("cm", [False, True])
def test_every_bf16_bit_pattern(gpu, cm):
    """All 65536 patterns (Inf, NaN, subnormals, both zeros included) spread over columns whose
    amax ranges over every exponent, so that each pattern meets many block scales."""
    K, N = 2048, 1024
    rng = np.random.default_rng(9)
    wb = rng.permutation(np.arange(K * N, dtype=np.uint32) % 65536).astype(np.uint16).reshape(K, N)
    # cap each 32-block's magnitudes at a per-block random exponent so scales vary widely
    cap = rng.integers(1, 255, size=(K // 32, 1, N)).astype(np.uint16)
    blk = wb.reshape(K // 32, 32, N)
    eb = (blk >> 7) & 0xFF
    keep_special = rng.random(blk.shape) < 0.002                      # a few Inf / NaN / huge values stay
    blk = np.where((eb > cap) & ~keep_special, (blk & 0x807F) | (cap << 7), blk).astype(np.uint16)
    wb = blk.reshape(K, N)
    f, s = _run(wb, 1, K, N, cm)
    wf, ws = ref_quant(wb, col_major=cm)
    assert np.array_equal(s, ws)
    nan_w = ((wf & 0x7F) == 0x7F)
    assert np.array_equal((f & 0x7F) == 0x7F, nan_w)
    assert np.array_equal(f[~nan_w], wf[~nan_w])
    assert np.array_equal(f[nan_w] & 0x80, wf[nan_w] & 0x80)


def test_dequantised_weights_are_close(gpu):
    """The reference-held acceptance (tests/kernels/test_gpu_quant.py:45-47,68): max |deq - w| /
    max |w| below 8 %."""
    rng = np.random.default_rng(0)
    K, N = 1024, 1024
    wb = bf16_rne_bits((0.1 * rng.standard_normal((K, N))).astype(np.float32)).reshape(K, N)
    f, s = _run(wb, 1, K, N, False)
    w = bits_to_f32(wb).reshape(K, N).astype(np.float64)
    deq = dequant_mxfp8_w(f, s)
    assert np.abs(deq - w).max() / np.abs(w).max() < 0.08


def test_cache_refreshes_once_per_step(gpu):
    from ancora_cutile_amd import DevBuf, Mxfp8WeightCache
    rng = np.random.default_rng(3)
    K, N = 128, 256
    wb = bf16_rne_bits((0.1 * rng.standard_normal((K, N))).astype(np.float32)).reshape(K, N)
    p16 = DevBuf(wb)
    cache = Mxfp8WeightCache({"w": dict(p16=p16, K=K, N=N)}, col_major=True)
    assert cache.refresh(0) and not cache.refresh(0)
    wf, ws = ref_quant(wb, col_major=True)
    assert np.array_equal(cache.fp8("w").to_numpy(), wf) and np.array_equal(cache.scale("w").to_numpy(), ws)
    wb2 = bf16_rne_bits((0.3 * rng.standard_normal((K, N))).astype(np.float32)).reshape(K, N)
    p16.upload(wb2)
    cache.mark_dirty()
    assert cache.refresh(0)
    wf, ws = ref_quant(wb2, col_major=True)
    assert np.array_equal(cache.fp8("w").to_numpy(), wf) and np.array_equal(cache.scale("w").to_numpy(), ws)
    cache.free(); p16.free()


def test_shape_checks(gpu):
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd._lib import api
    b = DevBuf.zeros((128, 128), np.uint16)
    with pytest.raises(_lib.AncoraError):
        api.anc_quant_mxfp8_w(b.ptr, b.ptr, b.ptr, 1, 96, 128, 0, 0)
    with pytest.raises(_lib.AncoraError):
        api.anc_quant_mxfp8_w(0, b.ptr, b.ptr, 1, 128, 128, 0, 0)
    b.free()
