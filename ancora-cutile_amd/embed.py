"""Input-embedding gradient by sorted scatter, and a row-sparse AdamW with dense results.

Mirror of `build_id_groups` and the `_embed_dw_scatter` launch (ancora/kernels/fused.py:387-424,
used at ancora/model/resident_moe_model.py:262-271, 333-334). `RowSparseAdamW` has no counterpart
in the reference, whose AdamW sweeps the whole embedding every step (ancora/optim/adamw.py:92-97):
it updates only the rows a step's tokens touch and replays the steps a row missed when the row is
next needed, so that every row it hands out is bit-identical to the dense optimizer's.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import api, AdamWHyper, FORM_DIV, FORM_IBC
from .adamw import sr_seed_base
from .devbuf import DevBuf


def build_id_groups(ids_flat):
    """Stable-sort token ids into groups (ancora/kernels/fused.py:411-424). Returns
    (srt, start, cnt, gid), each (M, 1) int32: srt the stable argsort; for group g (one per
    distinct id, ascending) start[g] its first position in srt, cnt[g] its size, gid[g] its id;
    groups beyond the last are padding with cnt = 0."""
    ids = np.asarray(ids_flat).reshape(-1)
    M = ids.size
    order = np.argsort(ids, kind="stable").astype(np.int32)
    uniq, first, counts = np.unique(ids[order], return_index=True, return_counts=True)
    U = uniq.size
    out = [order.reshape(M, 1)]
    for col in (first, counts, uniq):
        a = np.zeros((M, 1), np.int32)
        a[:U, 0] = col
        out.append(a)
    return tuple(out)


class IdGroups:
    """The four group arrays on the device, plus the number of distinct ids."""

    def __init__(self, ids_flat):
        srt, start, cnt, gid = build_id_groups(ids_flat)
        self.M = srt.shape[0]
        self.n_groups = int(np.count_nonzero(cnt))
        self.host = (srt, start, cnt, gid)
        self.srt, self.start, self.cnt, self.gid = (DevBuf(a) for a in (srt, start, cnt, gid))

    def free(self):
        for b in (self.srt, self.start, self.cnt, self.gid):
            b.free()


def embed_dw_scatter(groups, dy, si, out=None, compact=None, V=None):
    """dy: (M, H) bf16 DevBuf. out: (V, H) fp32 DevBuf, added onto in place (the reference's
    launch); or compact: (M, H) fp32 DevBuf that receives one summed row per group."""
    M, H = dy.shape
    if out is not None:
        V = out.shape[0] if V is None else V
    api.anc_embed_dw_scatter(groups.cnt.ptr, groups.start.ptr, groups.gid.ptr, groups.srt.ptr, dy.ptr,
                             0 if out is None else out.ptr, 0 if compact is None else compact.ptr,
                             M, 0 if V is None else V, H, int(si))


class RowSparseAdamW:
    """AdamW over one (V, H) fp32 tensor that steps only the rows named per step.

        opt = RowSparseAdamW(W, lr=3e-4, ...)
        opt.catch_up(row_ids, si)          # before the forward gathers these rows: p32/p16 current
        opt.step(groups.gid, n_groups, compact_grads, si, guard)   # after the backward
        opt.flush(si)                      # every row current (before a checkpoint / evaluation)

    State after `flush` equals the dense `AdamW` run on gradients that are zero outside the touched
    rows, bit for bit (stochastic rounding included). `lr` may change between steps."""

    def __init__(self, W, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.01, form="div", sr=False, seed=0,
                 tensor_seed=0, max_steps=1 << 16):
        _lib.init()
        W = np.ascontiguousarray(W, dtype=np.float32)
        if W.ndim != 2 or W.shape[1] % 64:
            raise ValueError(f"RowSparseAdamW: (V, H) tensor with H % 64 == 0 expected, got {W.shape}")
        self.V, self.H = W.shape
        self.lr, (self.b1, self.b2), self.eps, self.wd = lr, betas, eps, wd
        self.form, self.sr, self.seed, self.tensor_seed = form, bool(sr), int(seed), int(tensor_seed)
        self.t = 0
        self.p32 = DevBuf(W)
        self.p16 = DevBuf.zeros(W.shape, np.uint16)
        self.m = DevBuf.zeros(W.shape, np.float32)
        self.v = DevBuf.zeros(W.shape, np.float32)
        self.last = DevBuf.zeros((self.V,), np.int32)
        self._cap = int(max_steps)
        self.table = DevBuf.zeros((self._cap + 1, 4), np.uint32)
        self._rows_buf = None
        self.last_skipped = False
        self._filled_to = 0          # table entries 1 .. _filled_to hold the scalars of their steps
        self._filled_lr = None       # ... computed with this learning rate

    def _hyper(self):
        return AdamWHyper(beta1=self.b1, beta2=self.b2, omb1=1 - self.b1, omb2=1 - self.b2, eps=self.eps,
                          lr=0.0, bc1=1.0, bc2=1.0, form=FORM_DIV if self.form == "div" else FORM_IBC,
                          sr=int(self.sr), seed_base=0)

    FILL_AHEAD = 256

    def _step_record(self, t, lr):
        bc1, bc2 = 1 - self.b1 ** t, 1 - self.b2 ** t
        if self.form != "div":
            bc1, bc2 = 1.0 / bc1, 1.0 / bc2
        rec = np.zeros(4, np.uint32)
        rec[:3] = np.array([bc1, bc2, lr], np.float32).view(np.uint32)
        rec[3] = sr_seed_base(self.seed, t) if self.sr else 0
        return rec

    def _ensure_step(self, t, si):
        """Table entry t holds step t's scalars at the current learning rate. Entries are written
        FILL_AHEAD steps at a time, so a run at a constant learning rate uploads (and synchronises)
        once per FILL_AHEAD steps instead of at every step; a changed learning rate rewrites from t
        on (earlier entries keep the rate their steps ran with: the replay needs it)."""
        if t <= self._filled_to and self._filled_lr == self.lr:
            return
        hi = min(self._cap, t + self.FILL_AHEAD - 1)
        block = np.stack([self._step_record(s, self.lr) for s in range(t, hi + 1)])
        DevBuf(shape=block.shape, dtype=np.uint32, ptr=self.table.ptr + 16 * t).upload(block, si)
        self._filled_to, self._filled_lr = hi, self.lr

    def _rows(self, rows, si):
        rows = np.ascontiguousarray(rows, dtype=np.int32).reshape(-1)
        if self._rows_buf is None or self._rows_buf.size < rows.size:
            if self._rows_buf is not None:
                _lib.stream_sync(si)
                self._rows_buf.free()
            self._rows_buf = DevBuf.empty((max(rows.size, 1024),), np.int32)
        self._rows_buf.upload(rows, si)
        return self._rows_buf, rows.size

    def _launch(self, rows_ptr, n_rows, grads_ptr, t_now, ctl, si):
        h = self._hyper()
        api.anc_adamw_rows(rows_ptr, n_rows, grads_ptr, self.m.ptr, self.v.ptr, self.p32.ptr, self.p16.ptr,
                           self.last.ptr, self.V, self.H, self.table.ptr, int(t_now), ctypes.byref(h),
                           float(self.wd), self.tensor_seed, int(ctl), int(si))

    def catch_up(self, row_ids, si):
        """Replay, on the distinct rows in `row_ids` (host integers), the steps they missed."""
        if self.t == 0:
            return
        buf, n = self._rows(np.unique(np.asarray(row_ids).reshape(-1)), si)
        self._launch(buf.ptr, n, 0, self.t, 0, si)

    def step(self, gid, n_groups, grads, si, guard=None):
        """gid: device int32 array of distinct row ids (e.g. `IdGroups.gid`), the first n_groups
        valid; grads: (>= n_groups, H) fp32 DevBuf, row i the gradient of gid[i]."""
        if self.t + 1 > self._cap:             # before the counter moves: t always matches the table
            raise RuntimeError(f"RowSparseAdamW: step table holds {self._cap} steps; raise max_steps")
        self._ensure_step(self.t + 1, si)
        self.t += 1
        if n_groups > 0:
            self._launch(gid.ptr, int(n_groups), grads.ptr, self.t, 0 if guard is None else guard.ptr, si)
        self.last_skipped = False
        if guard is not None:
            _lib.stream_sync(si)
            if guard.read(si)["skip"]:
                self.t -= 1
                self.last_skipped = True

    def flush(self, si):
        """Bring every row up to date."""
        if self.t:
            self._launch(0, self.V, 0, self.t, 0, si)

    def master(self):
        return self.p32.to_numpy()

    def free(self):
        for b in (self.p32, self.p16, self.m, self.v, self.last, self.table, self._rows_buf):
            if b is not None:
                b.free()
