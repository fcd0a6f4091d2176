"""Host-side bf16 bit helpers (numpy has no bfloat16: bf16 lives in uint16).

Same integer formulas as the reference's host twins `_bf16_bits` / `_bits_f32`
(ancora/optim/adamw.py:63-66) and `_bf` (ancora/optim/muon.py:83-85).
"""
import numpy as np


def bf16_bits(x):
    """fp32 -> bf16 bit patterns, round-to-nearest-even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    u = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (u >> np.uint32(16)).astype(np.uint16)


def bits_f32(u):
    """bf16 bit patterns -> the fp32 values they denote."""
    return (np.ascontiguousarray(u).astype(np.uint32) << np.uint32(16)).view(np.float32)


def bf16_round(x):
    """fp32 -> nearest bf16 value, returned as fp32."""
    return bits_f32(bf16_bits(x)).reshape(np.shape(x))
