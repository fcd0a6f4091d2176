"""Pins the CPU restatement of the MXFP8 weight re-quantisation (oracle/quant_ref.py) without a
GPU: format constants, an independent integer-bit formulation of the rounding checked over every
bf16 input and every reachable block scale, special cases, and the error bound of the format."""
import numpy as np

from oracle.quant_ref import e4m3_table, e4m3_rne, quant_mxfp8_w, dequant_mxfp8_w, B
from oracle.bf16_ref import bf16_rne_bits, bits_to_f32


def e4m3_from_bf16_bits(bits, byte):
    """Integer-only E4M3FN(RNE) of bf16 `bits` scaled by 2**(127 - byte): the formulation the
    device kernel uses. Written independently of the table search in the oracle."""
    bits = np.asarray(bits, np.int64)
    byte = np.asarray(byte, np.int64)
    sign = (bits >> 8) & 0x80
    eb, m7 = (bits >> 7) & 0xFF, bits & 0x7F
    e = eb - byte + 7                                # E4M3 biased exponent before rounding
    v = (np.maximum(e, 0) << 7) | m7
    normal = (v + 7 + ((v >> 4) & 1)) >> 4
    sig = 0x80 | m7
    sh = np.clip(5 - e, 5, 10)                       # e <= 0: drop sh bits of the 8-bit significand
    sub = (sig + (1 << (sh - 1)) - 1 + ((sig >> sh) & 1)) >> sh
    out = np.where(e >= 1, normal, np.where(5 - e >= 10, 0, sub))
    out = np.where(eb == 0, 0, out)                  # zero and bf16 subnormals
    out = np.where(eb == 255, 0x7F, out)             # non-finite
    return (out | sign).astype(np.uint8)


def test_e4m3_table_matches_the_format():
    t = e4m3_table()
    assert t[0x00] == 0 and t[0x01] == 2.0 ** -9 and t[0x07] == 7 * 2.0 ** -9
    assert t[0x08] == 2.0 ** -6 and t[0x38] == 1.0 and t[0x40] == 2.0 and t[0x70] == 128.0
    assert t[0x78] == 256.0 and t[0x7E] == 448.0 and np.isnan(t[0x7F]) and np.isnan(t[0xFF])
    assert np.all(np.diff(t[:127]) > 0) and np.array_equal(t[128:255], -t[0:127])


def test_rounding_is_nearest_with_ties_to_even():
    t = e4m3_table()
    # midpoints between neighbours go to the even byte, anything off the midpoint to the nearer one
    for b in range(0, 126):
        mid = (t[b] + t[b + 1]) / 2
        even = b if b % 2 == 0 else b + 1
        assert e4m3_rne(mid) == even and e4m3_rne(-mid) == (even | 0x80)
        assert e4m3_rne(np.nextafter(mid, 0)) == b and e4m3_rne(np.nextafter(mid, 1e9)) == b + 1
    assert e4m3_rne(448.0) == 0x7E and e4m3_rne(1e9) == 0x7E
    assert e4m3_rne(np.inf) == 0x7F and e4m3_rne(-np.inf) == 0xFF and e4m3_rne(np.nan) & 0x7F == 0x7F
    assert np.array_equal(e4m3_rne(t[:127]), np.arange(127))          # representable values are fixed points


def test_integer_formulation_agrees_for_every_bf16_input_and_scale():
    bits = np.arange(65536, dtype=np.int64)
    eb = (bits >> 7) & 0xFF
    for byte in list(range(0, 249, 7)) + [1, 2, 120, 121, 247, 248]:
        ok = (eb <= byte + 7) | (eb == 255)          # an element cannot exceed its block's amax
        flushed = np.where(eb == 0, bits & 0x8000, bits)
        with np.errstate(invalid="ignore"):
            w = bits_to_f32(flushed.astype(np.uint16)).astype(np.float64)
        with np.errstate(invalid="ignore", over="ignore"):
            want = e4m3_rne(w * np.exp2(127.0 - byte))
        got = e4m3_from_bf16_bits(bits, byte)
        nan = eb == 255
        assert np.array_equal(got[ok & ~nan], want[ok & ~nan]), byte
        assert np.all((got[nan] & 0x7F) == 0x7F)


def test_block_scale_and_special_cases():
    rng = np.random.default_rng(0)
    K, N = 64, 128
    w = bf16_rne_bits((0.1 * rng.standard_normal((K, N))).astype(np.float32)).reshape(K, N)
    w[:32, 0] = bf16_rne_bits(np.full(32, 0.25, np.float32))           # amax a power of two
    w[:32, 1] = 0                                                       # a block of zeros
    w[:32, 2] = bf16_rne_bits(np.full(32, 1e-3, np.float32)); w[5, 2] = bf16_rne_bits(np.float32(3.0))[0]
    fp8, sc = quant_mxfp8_w(w)
    assert fp8.shape == (K, N) and sc.shape == (K // B, N)
    assert sc[0, 0] == 127 - 2 - 7 and np.all(fp8[:32, 0] == 0x70)      # 0.25 / 2**-9 = 128
    assert sc[0, 1] == 0 and np.all(fp8[:32, 1] == 0)
    assert sc[0, 2] == 127 + 1 - 7 and fp8[5, 2] == 0x74                # 3 / 2**-6 = 192
    assert np.all(fp8[:5, 2] == 0x18)                                   # 1e-3 / 2**-6 = 1.025 * 2**-4
    # amax / sc in [128, 256): the largest byte of every non-zero block is 0x70..0x78
    top = (fp8 & 0x7F).reshape(K // B, B, N).max(1)
    assert np.all((top >= 0x70) & (top <= 0x78) | (sc == 0))
    f2, s2 = quant_mxfp8_w(w, col_major=True)
    assert np.array_equal(f2, fp8.T) and np.array_equal(s2, sc.T)


def test_dequantisation_error_bound():
    rng = np.random.default_rng(1)
    K, N = 256, 128
    wf = (0.1 * rng.standard_normal((K, N))).astype(np.float32)
    wb = bf16_rne_bits(wf).reshape(K, N)
    w = bits_to_f32(wb).reshape(K, N).astype(np.float64)
    fp8, sc = quant_mxfp8_w(wb)
    deq = dequant_mxfp8_w(fp8, sc)
    scale = np.exp2(sc.astype(np.float64) - 127.0).repeat(B, axis=0)
    # half a unit in the last place of a 3-bit mantissa, or of the subnormal grid 2**-9
    bound = np.maximum(np.abs(w) * 2.0 ** -4, scale * 2.0 ** -10)
    assert np.all(np.abs(deq - w) <= bound)
    assert np.abs(deq - w).max() / np.abs(w).max() < 0.08              # tests/kernels/test_gpu_quant.py:68
    assert np.array_equal(dequant_mxfp8_w(*quant_mxfp8_w(wb, col_major=True), col_major=True), deq)
