"""Shared helpers of the parity tests."""
import numpy as np


def ulp_diff(a, b):
    """Element-wise distance in units in the last place between two fp32 arrays."""
    a = np.ascontiguousarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    b = np.ascontiguousarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, np.int64(-2147483648) - a, a)
    b = np.where(b < 0, np.int64(-2147483648) - b, b)
    return np.abs(a - b)


def max_ulp(a, b):
    d = ulp_diff(a, b)
    return int(d.max()) if d.size else 0


def bits_equal(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and bool(np.array_equal(a.view(np.uint8), b.view(np.uint8)))


def rel_fro(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / (np.linalg.norm(b) + 1e-300))


def bf16_grad(rng, shape, std=1e-3):
    """bf16 gradient ~N(0, std) as uint16 bit patterns, plus its fp32 value."""
    from oracle.bf16_ref import bf16_rne_bits, bits_to_f32
    g = (rng.standard_normal(shape) * std).astype(np.float32)
    bits = bf16_rne_bits(g)
    return bits, bits_to_f32(bits).reshape(shape)
