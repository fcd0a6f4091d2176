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
        self._tables = {}
        self._part0 = []
        self._key = None

    @property
    def ptr(self):
        return self.ctl.ptr

    def plan(self, grads):
        """Lay out the partial sums for this list of gradients (fixed order) without computing
        anything: afterwards `partials_ptr(i)` is where tensor i's partials live, so that a
        producer of the gradients can write them itself (`gemm_dW(..., gn_partials=...)`)."""
        key = tuple((g.ptr, g.size, g.dtype.str) for g in grads)
        if key != self._key:
            self._free_tables()
            self._part0, chunk0 = [], 0
            for g in grads:
                self._part0.append(chunk0)
                chunk0 += api.anc_gradnorm_num_partials(g.size)
            self._n_partials = chunk0
            self._partials = DevBuf.empty((chunk0,), np.float64)
            self._tables = {}
            self._key = key

    def partials_ptr(self, i):
        return self._partials.ptr + 8 * self._part0[i]

    def set_t(self, t, stream=0):
        """Set the device step count (a fresh optimizer starts at 0; a resumed one at its saved
        count). The rest of the block is rewritten by the next `compute`."""
        raw = np.zeros(8, np.uint32)
        raw[5] = np.uint32(int(t))
        self.ctl.upload(raw, stream)

    def compute(self, grads, stream=0, produced=(), count_step=False):
        """grads: list of DevBuf (float32 or uint16/bf16), in a fixed order. `produced`: indices
        of gradients whose partial sums are already in place (written by their producer since the
        last call). The result is the same bits either way. `count_step`: advance the block's step
        count `t` unless the step is skipped (for update kernels that take their per-step scalars
        from it). Asynchronous."""
        self.plan(grads)
        produced = tuple(sorted(set(int(i) for i in produced)))
        if produced not in self._tables:
            descs, chunk0 = [], 0
            for i, g in enumerate(grads):
                if i in produced:
                    continue
                descs.append(GnDesc(g.ptr, g.size, chunk0, self._part0[i], _dtype_code(g.dtype), 0))
                chunk0 += api.anc_gradnorm_num_partials(g.size)
            self._tables[produced] = (upload_table(descs) if descs else None, len(descs), chunk0)
        table, n_tensors, n_chunks = self._tables[produced]
        if table is not None:
            api.anc_gradnorm_partials_multi(table.ptr, n_tensors, n_chunks, self._partials.ptr, int(stream))
        api.anc_gradnorm_finalize(self._partials.ptr, self._n_partials, self.max_norm, self.eps,
                                  int(bool(count_step)), self.ctl.ptr, int(stream))

    def read(self, stream=0):
        """Synchronise and return the control block as a dict."""
        raw = self.ctl.to_numpy(stream)
        c = StepCtl.from_buffer_copy(raw.tobytes())
        return {"sumsq": c.sumsq, "norm": c.norm, "clip_scale": c.clip_scale, "skip": bool(c.skip),
                "t": int(c.t)}

    def _free_tables(self):
        for b in [self._partials] + [t[0] for t in self._tables.values()]:
            if b is not None:
                b.free()
        self._partials = None
        self._tables = {}

    def free(self):
        self._free_tables()
        self.ctl.free()
