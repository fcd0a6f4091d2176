"""MXFP8 weight re-quantisation, restated on the CPU. Test infrastructure only: nothing in the
product imports this file.

Follows the device kernels `_quant_mxfp8_w` / `_quant_mxfp8_w_cm` of
ancora/kernels/quant.py:60-100 as text: per block of 32 consecutive K (axis 0) and per column,
    amax  = max |w|                                    (quant.py:67)
    ea    = biased fp32 exponent of amax               (quant.py:68)
    byte  = ea - 7 if ea >= 7 else 0                   (quant.py:69)   E8M0 scale byte
    sc    = 2 ** (byte - 127)                          (quant.py:70)
    fp8   = E4M3FN(w / sc), round to nearest even      (quant.py:71)
so that amax / sc lies in [128, 256), below the E4M3 maximum of 448. The E4M3FN value table is the
one of quant.py:104-119 (bias 7, subnormals m/8 * 2**-6, 0x7F / 0xFF = NaN).

Pinned by tests/test_oracle_quant.py: the table against the closed form of the format, the
rounding against exhaustive nearest-value search with ties to the even byte over every bf16 input
and every reachable scale, special cases (powers of two, block of zeros, one outlier per block),
the dequantisation error bound of the format, and the reference-held tolerance (max |deq - w| /
max |w| < 8 %, tests/kernels/test_gpu_quant.py:45-47,68).

Parity unpinned (no reference-held vector fixes them): a block whose amax is below 2**-120 (ea < 7:
the reference's `exp2(byte - 127)` is then a subnormal fp32, whose handling inside cuda-tile is
not visible from its text) -- here such a block gets byte 0 and its elements are scaled by 2**127
exactly; bf16 subnormal inputs (exponent field 0) count as zero; non-finite inputs give the NaN
byte 0x7F | sign and set the block's scale byte to 248 through ea = 255.
"""
import numpy as np

B = 32                     # scale block (quant.py:19)


def e4m3_table():
    """The 256 E4M3FN values by byte (quant.py:104-119)."""
    v = np.zeros(256, np.float64)
    for b in range(256):
        s = -1.0 if b & 0x80 else 1.0
        e, m = (b >> 3) & 0xF, b & 7
        if e == 0:
            v[b] = s * (m / 8.0) * 2.0 ** -6
        elif e == 15 and m == 7:
            v[b] = np.nan
        else:
            v[b] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return v


_POS = e4m3_table()[:127]          # bytes 0x00..0x7E: 0 .. 448 ascending


def e4m3_rne(x):
    """float -> E4M3FN byte, nearest value, ties to the even byte (= even mantissa), magnitudes
    above 448 saturate to 448, non-finite inputs give NaN (0x7F | sign)."""
    x = np.asarray(x, np.float64)
    ax = np.abs(x)
    fin = np.isfinite(ax)
    a = np.where(fin, np.minimum(ax, 448.0), 0.0)
    hi = np.clip(np.searchsorted(_POS, a, side="left"), 1, 126)
    lo = hi - 1
    dlo, dhi = a - _POS[lo], _POS[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    byte = np.where(pick_hi, hi, lo).astype(np.uint8)
    byte = np.where(fin, byte, np.uint8(0x7F))
    return (byte | (np.signbit(x).astype(np.uint8) << 7)).astype(np.uint8)


def quant_mxfp8_w(w_bits, col_major=False):
    """w_bits (K, N) uint16 bf16 bits -> (fp8 (K, N) u8, scale (K//32, N) u8); with
    col_major=True the transposed layout of `_quant_mxfp8_w_cm`: fp8 (N, K), scale (N, K//32)."""
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    K, N = w_bits.shape
    assert K % B == 0
    bits = np.where((w_bits & 0x7F80) == 0, w_bits & 0x8000, w_bits).astype(np.uint16)   # subnormal -> 0
    w = (bits.astype(np.uint32) << 16).view(np.float32).reshape(K // B, B, N)
    amax = np.nanmax(np.where(np.isnan(w), np.inf, np.abs(w)), axis=1, keepdims=True).astype(np.float32)
    ea = (amax.view(np.uint32) >> 23) & 0xFF
    byte = np.where(ea >= 7, ea - 7, 0).astype(np.int64)
    with np.errstate(invalid="ignore", over="ignore"):
        x = w.astype(np.float64) * np.exp2(127.0 - byte)          # = w / sc, exact
    fp8 = e4m3_rne(x).reshape(K, N)
    sb = byte.astype(np.uint8).reshape(K // B, N)
    if col_major:
        return np.ascontiguousarray(fp8.T), np.ascontiguousarray(sb.T)
    return fp8, sb


def dequant_mxfp8_w(fp8, scale, col_major=False):
    """Inverse map for error checks: (K, N) float64."""
    if col_major:
        fp8, scale = fp8.T, scale.T
    K, N = fp8.shape
    v = e4m3_table()[fp8].reshape(K // B, B, N)
    return (v * np.exp2(scale.astype(np.float64) - 127.0)[:, None, :]).reshape(K, N)
