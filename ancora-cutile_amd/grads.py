"""Weight-gradient GEMM dW (+)= x^T dy on the MI355X: the producer of the gradients the optimizer
step reads.

Mirror of `ResidentLayerTrain._dW` (ancora/model/resident_train.py:285-287), which launches
`_gemm_dW` or, with gradient accumulation, `_gemm_dW_acc` (ancora/kernels/fused.py:190-219) once
per weight: x (T, K) and dy (T, N) bf16 bits, dW (K, N) fp32. Here up to 8 weights go into one
call (`gemm_dW`), the activations are passed as they lie (`x`) or transposed (`xT`, for a caller
that keeps them so), and the call can also leave the bf16 copy of the finished gradient, which is
what `HybridOptimizer(grad_dtype=np.uint16)` reads.

By default the token axis is not cut (fixed tiles, no split-K): a gradient's bits do not depend on
how the caller groups its calls. A call fills the GPU when it carries about 500 tiles of 128x256
outputs, which the 7 weights of a layer handed over in one call do (480 at Qwen3-0.6B shapes); a
caller that must launch weight by weight can opt into `segments` (an int, "shape" or "fill"), a
deterministic split of the token axis whose number of pieces then enters the bits.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import api, DwProblem
from .devbuf import DevBuf

MAX_PER_CALL = 8


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


def gemm_dW(problems, si=0, segments=None):
    """problems: list of dicts {x (T, K) or xT (K, T), dy, dW: DevBuf; T, K, N: int; workspace: DwWorkspace;
    g16: DevBuf or None; accumulate: bool; gn_partials: int device address or None (where the
    grad-norm partial sums of this gradient go, `StepGuard.partials_ptr`); segments: int, optional}.
    dW (+)= x^T dy for each, 8 per launch. `segments` (argument, or per problem) fixes the number
    of token segments: None / 1 = none (the default); "shape" = the library's rule (a function of
    T, K, N alone); "fill" = per launch, the largest power of two that keeps the launch within the
    512 workgroups the GPU runs at once (so it depends on what shares the call). The result's bits
    depend on the number of segments and on nothing else. Asynchronous on stream `si`."""
    _lib.init()
    runs, cur = [], []
    for p in problems:                       # a native call takes one activation layout
        if cur and ((p.get("x") is None) != (cur[0].get("x") is None) or len(cur) == MAX_PER_CALL):
            runs.append(cur)
            cur = []
        cur.append(p)
    if cur:
        runs.append(cur)
    for group in runs:
        fill = 0
        if segments == "fill":
            tiles = sum((int(p["K"]) // 128) * (int(p["N"]) // 256) for p in group)
            tmin = min(int(p["T"]) for p in group)
            fill = 1
            while tiles * fill * 2 <= 512 and all(int(p["T"]) % (fill * 2 * 32) == 0 for p in group) \
                    and tmin // (fill * 2) >= 256:
                fill *= 2
        arr = (DwProblem * len(group))()
        for k, p in enumerate(group):
            T, K, N = int(p["T"]), int(p["K"]), int(p["N"])
            S = p.get("segments") or fill or (None if segments == "fill" else segments) or 1
            if S == "shape":
                S = dw_info(T, K, N)[1]
            S = int(S)
            gn = int(p.get("gn_partials") or 0)
            if S == 1 and gn == 0:                 # finished by the GEMM's epilogue: no partial tiles
                ws_ptr = ws_bytes = 0
            else:
                ws = p["workspace"].ensure(S * K * N * 4)
                ws_ptr, ws_bytes = ws.ptr, ws.nbytes
            g16 = p.get("g16")
            x = p.get("x")
            arr[k] = DwProblem((p["xT"] if x is None else x).ptr, p["dy"].ptr, p["dW"].ptr,
                               0 if g16 is None else g16.ptr, ws_ptr, T, K, N, ws_bytes,
                               int(bool(p.get("accumulate", False))), S, gn, 0 if x is None else 1, 0)
        api.anc_gemm_dw_multi(arr, len(group), int(si))
