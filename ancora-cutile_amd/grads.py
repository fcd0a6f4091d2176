"""Weight-gradient GEMM dW (+)= x^T dy on the MI355X: the producer of the gradients the optimizer
step reads.

Mirror of `ResidentLayerTrain._dW` (ancora/model/resident_train.py:285-287), which launches
`_gemm_dW` or, with gradient accumulation, `_gemm_dW_acc` (ancora/kernels/fused.py:190-219) once
per weight: x (T, K) and dy (T, N) bf16 bits, dW (K, N) fp32. Here up to 4 weights go into one
call (`gemm_dW`), the activations are passed transposed (`transpose_acts`, once per group of
weights that share them), and the call can also leave the bf16 copy of the finished gradient,
which is what `HybridOptimizer(grad_dtype=np.uint16)` reads.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import api, DwProblem
from .devbuf import DevBuf

MAX_PER_CALL = 4


def dw_workspace_bytes(T, K, N):
    n = api.anc_gemm_dw_workspace_bytes(int(T), int(K), int(N))
    if n < 0:
        raise _lib.AncoraError(_lib._lib.anc_last_error().decode())
    return int(n)


def dw_info(T, K, N):
    """(FLOPs, token segments) of one problem."""
    fl, seg = ctypes.c_double(0), ctypes.c_int32(0)
    api.anc_gemm_dw_info(int(T), int(K), int(N), ctypes.byref(fl), ctypes.byref(seg))
    return fl.value, int(seg.value)


def transpose_acts(x, xT, T, K, si=0):
    """x (T, K) bf16 bits -> xT (K, T): the layout `gemm_dW` takes. T and K multiples of 64."""
    api.anc_transpose_bf16(x.ptr, xT.ptr, 1, int(T), int(K), int(si))


class DwWorkspace:
    """Partial-tile scratch of one weight's gradient GEMM, sized on first use and kept."""

    def __init__(self):
        self.buf = None

    def ensure(self, nbytes):
        if self.buf is None or self.buf.nbytes < nbytes:
            if self.buf is not None:
                self.buf.free()
            self.buf = DevBuf.empty(((nbytes + 3) // 4,), np.float32)
        return self.buf

    def free(self):
        if self.buf is not None:
            self.buf.free()
            self.buf = None


def gemm_dW(problems, si=0):
    """problems: list of dicts {xT, dy, dW: DevBuf; T, K, N: int; workspace: DwWorkspace;
    g16: DevBuf or None; accumulate: bool; gn_partials: int device address or None (where the
    grad-norm partial sums of this gradient go, `StepGuard.partials_ptr`)}. dW (+)= x^T dy for
    each, 4 per launch. Asynchronous on stream `si`."""
    _lib.init()
    for i0 in range(0, len(problems), MAX_PER_CALL):
        group = problems[i0:i0 + MAX_PER_CALL]
        arr = (DwProblem * len(group))()
        for k, p in enumerate(group):
            T, K, N = int(p["T"]), int(p["K"]), int(p["N"])
            nb = dw_workspace_bytes(T, K, N)
            ws = p["workspace"].ensure(nb)
            g16 = p.get("g16")
            arr[k] = DwProblem(p["xT"].ptr, p["dy"].ptr, p["dW"].ptr, 0 if g16 is None else g16.ptr, ws.ptr,
                               T, K, N, ws.nbytes, int(bool(p.get("accumulate", False))), 0,
                               int(p.get("gn_partials") or 0))
        api.anc_gemm_dw_multi(arr, len(group), int(si))
