"""Weight-gradient GEMM dW = x^T dy on the CPU. Test infrastructure only.

Restates `_gemm_dW` / `_gemm_dW_acc` (ancora/kernels/fused.py:190-219): bf16 inputs, products
accumulated over the token axis, fp32 result, optionally added onto an existing dW. The checker
is the reference's own (tests/kernels/test_gemm_bwd.py:40-44): the fp64 matrix product of the
bf16-rounded inputs, `x.T.astype(float64) @ dy.astype(float64)` -- a library routine; products of
bf16 values are exact in fp32, so only the accumulation order separates a device result from it.
The reference's bar is max |err| / max |ref| < 2 % (test_gemm_bwd.py:41-43); the build's tests
use 2e-5 relative Frobenius, which an fp32 accumulation over a few thousand tokens meets and a
bf16 accumulation, a dropped token block or a transposed operand do not.
"""
import numpy as np


def _f(bits):
    return (np.ascontiguousarray(bits).astype(np.uint32) << np.uint32(16)).view(np.float32)


def gemm_dw(x_bits, dy_bits, dW_prev=None):
    """x_bits (T, K), dy_bits (T, N) uint16 bf16 bits -> (K, N) float64 (+ dW_prev)."""
    x = _f(x_bits).astype(np.float64)
    dy = _f(dy_bits).astype(np.float64)
    out = x.T @ dy
    if dW_prev is not None:
        out = out + np.asarray(dW_prev, dtype=np.float64)
    return out
