"""Global gradient norm, clip scale and non-finite guard, resident on the device.

No counterpart in the reference (it has no grad-norm, clipping or NaN guard; its
nearest patterns are the fixed-order reductions of ancora/kernels/muon_ns.py:156-165
and ancora/model/resident_train.py:295-298). `StepGuard.compute` runs the two-stage
deterministic reduction over every gradient of the step and leaves
{sumsq, norm, clip_scale, skip} in a 32-byte device block that the AdamW and Muon
kernels read directly: no host round trip between the norm and the update.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import api, GnDesc, StepCtl, F32, BF16
from .devbuf import DevBuf, upload_table


def _dtype_code(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return F32
    if dtype == np.uint16:
        return BF16
    raise TypeError(f"gradient dtype {dtype}: expected float32 or uint16 (bf16 bits)")


class StepGuard:
    """max_norm: clip threshold (None or <= 0 disables clipping; the non-finite guard stays on)."""

    def __init__(self, max_norm=1.0, eps=1e-6):
        _lib.init()
        self.max_norm = 0.0 if max_norm is None else float(max_norm)
        self.eps = float(eps)
        self.ctl = DevBuf.zeros((8,), np.uint32)
        self._partials = None
        self._table = None
        self._key = None

    @property
    def ptr(self):
        return self.ctl.ptr

    def compute(self, grads, stream=0):
        """grads: list of DevBuf (float32 or uint16/bf16), in a fixed order. Asynchronous."""
        key = tuple((g.ptr, g.size, g.dtype.str) for g in grads)
        if key != self._key:
            self._free_tables()
            descs, chunk0 = [], 0
            for g in grads:
                nch = api.anc_gradnorm_num_partials(g.size)
                descs.append(GnDesc(g.ptr, g.size, chunk0, chunk0, _dtype_code(g.dtype), 0))
                chunk0 += nch
            self._n_partials = chunk0
            self._n_tensors = len(descs)
            self._table = upload_table(descs)
            self._partials = DevBuf.empty((chunk0,), np.float64)
            self._key = key
        api.anc_gradnorm_partials_multi(self._table.ptr, self._n_tensors, self._n_partials,
                                        self._partials.ptr, int(stream))
        api.anc_gradnorm_finalize(self._partials.ptr, self._n_partials, self.max_norm, self.eps,
                                  self.ctl.ptr, int(stream))

    def read(self, stream=0):
        """Synchronise and return the control block as a dict."""
        raw = self.ctl.to_numpy(stream)
        c = StepCtl.from_buffer_copy(raw.tobytes())
        return {"sumsq": c.sumsq, "norm": c.norm, "clip_scale": c.clip_scale, "skip": bool(c.skip)}

    def _free_tables(self):
        for b in (self._partials, self._table):
            if b is not None:
                b.free()
        self._partials = self._table = None

    def free(self):
        self._free_tables()
        self.ctl.free()
