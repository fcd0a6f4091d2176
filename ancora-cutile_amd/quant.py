"""MXFP8 weight re-quantisation after the optimizer step, on the MI355X.

Mirror of the device side of ancora/kernels/quant.py: `_quant_mxfp8_w` (:60-73) and
`_quant_mxfp8_w_cm` (:84-100), with the same constants B = 32 (scale block along K) and
QWN = 128 (column granularity), and of the dirty-flag protocol around them: the step marks the
fp8 copies of the bf16 weights stale (ancora/model/resident_train.py:354-357) and the next
forward re-quantises every weight once (:190-199). `Mxfp8WeightCache` holds the fp8 bytes and
E8M0 scale bytes per weight and does exactly that; the arithmetic runs in one HIP kernel per
weight (`anc_quant_mxfp8_w`), all-integer on the bf16 bit patterns.
"""
import numpy as np

from . import _lib
from ._lib import api
from .devbuf import DevBuf

B = 32          # MXFP8 scale block (ancora/kernels/quant.py:19)
QWN = 128       # column granularity of the weight kernels (quant.py:22)


def quant_mxfp8_w(w16, fp8_out, scale_out, K, N, si, E=1, col_major=False):
    """bf16 bits (E*K, N) -> fp8_out (E*K, N) u8 + scale_out (E*K//32, N) u8; col_major=True
    writes the transposed layout fp8_out (E*N, K) + scale_out (E*N, K//32) that a GEMM taking the
    weight as (N, K) row-major reads. Asynchronous on stream `si`."""
    if K % 128 or N % QWN:
        raise ValueError(f"quant_mxfp8_w: K={K} and N={N} must be multiples of 128")
    api.anc_quant_mxfp8_w(w16.ptr, fp8_out.ptr, scale_out.ptr, int(E), int(K), int(N), int(bool(col_major)),
                          int(si))


class Mxfp8WeightCache:
    """fp8 + scale copies of a set of bf16 weights, refreshed lazily.

    weights: {name: dict(p16=DevBuf of bf16 bits, K=int, N=int, E=int (optional, stacked
    experts))}. `mark_dirty()` is what an optimizer step does; `refresh(si)` is what the forward
    does before it reads the fp8 weights: one kernel per weight if anything is stale."""

    def __init__(self, weights, col_major=False):
        _lib.init()
        self.col_major = bool(col_major)
        self.w = {}
        for name, s in weights.items():
            E, K, N = int(s.get("E", 1)), int(s["K"]), int(s["N"])
            if K % 128 or N % QWN:
                raise ValueError(f"Mxfp8WeightCache: {name} ({K},{N}) is not a multiple of 128")
            shp8 = (E * N, K) if self.col_major else (E * K, N)
            shps = (E * N, K // B) if self.col_major else (E * K // B, N)
            self.w[name] = dict(p16=s["p16"], E=E, K=K, N=N, fp8=DevBuf.zeros(shp8, np.uint8),
                                scale=DevBuf.zeros(shps, np.uint8))
        self.dirty = True

    def mark_dirty(self):
        self.dirty = True

    def refresh(self, si=0):
        """Re-quantise every weight if a step has run since the last call. Returns True if it did."""
        if not self.dirty:
            return False
        for s in self.w.values():
            quant_mxfp8_w(s["p16"], s["fp8"], s["scale"], s["K"], s["N"], si, E=s["E"],
                          col_major=self.col_major)
        self.dirty = False
        return True

    def fp8(self, name):
        return self.w[name]["fp8"]

    def scale(self, name):
        return self.w[name]["scale"]

    def nbytes(self):
        return sum(s["fp8"].nbytes + s["scale"].nbytes for s in self.w.values())

    def free(self):
        for s in self.w.values():
            s["fp8"].free()
            s["scale"].free()
        self.w = {}
