"""bf16 bit arithmetic and the stochastic-rounding hash. Test infrastructure only."""
import numpy as np


def bf16_rne_bits(x):
    """fp32 -> bf16 bits, round to nearest even: u + 0x7FFF + ((u >> 16) & 1), >> 16
    (ancora/optim/adamw.py:63-65; same formula ancora/optim/muon.py:83-85)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    u = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (u >> np.uint32(16)).astype(np.uint16)


def bits_to_f32(b):
    """bf16 bits -> fp32 value (ancora/optim/adamw.py:66)."""
    return (np.ascontiguousarray(b).astype(np.uint32) << np.uint32(16)).view(np.float32)


def bf16_round(x):
    return bits_to_f32(bf16_rne_bits(x)).reshape(np.shape(x))


def sr_dither(row, col, seed):
    """16-bit dither of the stochastic downcast, all arithmetic modulo 2**32
    (ancora/kernels/fused.py:154-161; tests/kernels/_probe_sr_ops.py:28-38):
    key = row*73856093 ^ col*19349663 ^ seed; h = key*0x9E3779B1; h ^= h>>16;
    h *= 0x85EBCA6B; h ^= h>>13; dither = h & 0xFFFF."""
    row = np.asarray(row, dtype=np.uint64)
    col = np.asarray(col, dtype=np.uint64)
    mask = np.uint64(0xFFFFFFFF)
    key = ((row * np.uint64(73856093)) & mask) ^ ((col * np.uint64(19349663)) & mask) \
        ^ (np.uint64(int(seed) & 0xFFFFFFFF))
    h = (key * np.uint64(0x9E3779B1)) & mask
    h = h ^ (h >> np.uint64(16))
    h = (h * np.uint64(0x85EBCA6B)) & mask
    h = h ^ (h >> np.uint64(13))
    return (h & np.uint64(0xFFFF)).astype(np.uint32)


def bf16_sr_bits(x, seed, first_index=0):
    """Stochastic fp32 -> bf16 bits over a flat tensor: element i uses the reference's
    (row, col) = (i // 64, i % 64) coordinates of its (numel/64, 64) view
    (ancora/optim/adamw.py:20) and out = (bits(x) + dither) >> 16
    (ancora/kernels/fused.py:160-161). Build-defined extension of the unguarded reference
    form: Inf and NaN pass through unchanged (a NaN keeps a non-zero mantissa)."""
    flat = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    u = flat.view(np.uint32).astype(np.uint64)
    i = np.arange(flat.size, dtype=np.uint64) + np.uint64(first_index)
    d = sr_dither(i >> np.uint64(6), i & np.uint64(63), seed).astype(np.uint64)
    out = ((u + d) & np.uint64(0xFFFFFFFF)) >> np.uint64(16)
    nonfinite = (u & np.uint64(0x7F800000)) == np.uint64(0x7F800000)
    passthru = (u >> np.uint64(16)) | np.where((u & np.uint64(0x007FFFFF)) != 0,
                                               np.uint64(0x0040), np.uint64(0))
    out = np.where(nonfinite, passthru, out)
    return out.astype(np.uint16).reshape(np.shape(x))
