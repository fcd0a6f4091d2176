"""AdamW with fp32 master weights, fp32 m/v and a bf16 working copy, on the MI355X.

Mirror of ancora/optim/adamw.py: the same `AdamW` class (constructor, `step`,
`weights`, `master`, `free`, the per-name state dict `st` and the step counter `t`),
the same low-level launch tuple `_adamw(g, m, v, p32, p16, OTM, beta1, beta2, eps, lr,
wd, ibc1, ibc2)` with `_pick_otm` and `C`, and the host RNE helpers. The cuda-tile
kernel is replaced by `anc_adamw` / `anc_adamw_multi` (one launch for the whole
parameter group instead of one per tensor).

Arithmetic: by default the class evaluates the *divide* form of the reference's numpy
test oracle (tests/optim/test_adamw.py:37-41) with every scalar rounded to fp32 once on
the host, so master weights and moments are bit-identical to that oracle;
`form="ibc"` selects the reference kernel's multiply-by-reciprocal form
(ancora/optim/adamw.py:34-37), which is what the low-level `_adamw` tuple carries.

Extensions (all off by default): bf16 gradients (uint16 arrays), gradients already
resident in DevBufs, stochastic-rounded bf16 downcast (`sr=True`, counter-based hash of
ancora/kernels/fused.py:154-161), and a StepGuard (global clip + skip on non-finite).
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import (api, AdamWHyper, AdamWDesc, AdamWStepEntry, F32, BF16, FORM_DIV, FORM_IBC, SR_ON,
                   SR_STEP_SEED)
from .bf16 import bf16_bits as _bf16_bits, bits_f32 as _bits_f32  # noqa: F401  (re-exported)
from .devbuf import DevBuf, upload_table

C = 64   # every tensor is a flat (numel // 64, 64) view (ancora/optim/adamw.py:20)


def _pick_otm(R):
    """Rows per tile of the reference's launch (ancora/optim/adamw.py:44-48). Kept for callers
    that build the launch tuple; the HIP kernel walks fixed 4096-element blocks instead."""
    for cand in (128, 64, 32, 16, 8, 4, 2):
        if R % cand == 0:
            return cand
    return 1


def _g_code(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return F32
    if dtype == np.uint16:
        return BF16
    raise TypeError(f"gradient dtype {dtype}: expected float32 or uint16 (bf16 bits)")


def sr_seed_base(base_seed, t):
    """Per-step seed of the stochastic downcast; tensor i of a group uses seed_base + i
    (uint32 wrap-around)."""
    return (int(base_seed) + 1000003 * int(t)) & 0xFFFFFFFF


def hyper_div(lr, b1, b2, eps, t, sr=False, seed_base=0):
    """Scalars of the numpy-oracle form, each computed in Python double and rounded to fp32
    once (what numpy's weak-scalar promotion does in tests/optim/test_adamw.py:38-40)."""
    return AdamWHyper(beta1=b1, beta2=b2, omb1=1 - b1, omb2=1 - b2, eps=eps, lr=lr,
                      bc1=1 - b1 ** t, bc2=1 - b2 ** t, form=FORM_DIV, sr=int(bool(sr)),
                      seed_base=seed_base)


def hyper_ibc(lr, b1, b2, eps, ibc1, ibc2, sr=False, seed_base=0):
    """Scalars of the reference kernel form (ancora/optim/adamw.py:34-37, 90-91)."""
    return AdamWHyper(beta1=b1, beta2=b2, omb1=0.0, omb2=0.0, eps=eps, lr=lr, bc1=ibc1, bc2=ibc2,
                      form=FORM_IBC, sr=int(bool(sr)), seed_base=seed_base)


def _adamw(stream_int, g, m, v, p32, p16, OTM, beta1, beta2, eps, lr, wd, ibc1, ibc2, ctl=0):
    """The reference's launch `ct.launch(si, (R//OTM,1,1), _adamw, (g, m, v, p32, p16, OTM, ...))`
    (ancora/optim/adamw.py:94-97; also resident_train.py:350-353, resident_model.py:162-166,
    kernels/moe.py:586-588) as one call. g/m/v/p32/p16 are DevBufs over the same element count;
    OTM is accepted and ignored. g may be float32 or uint16 (bf16 bits)."""
    n = p32.size
    if n % C:
        raise ValueError(f"_adamw: numel {n} is not a multiple of {C}")
    h = hyper_ibc(lr, beta1, beta2, eps, ibc1, ibc2)
    api.anc_adamw(g.ptr, m.ptr, v.ptr, p32.ptr, p16.ptr, n, _g_code(g.dtype), ctypes.byref(h),
                  float(wd), 0, int(ctl), int(stream_int))


class AdamW:
    """fp32-master AdamW. params: {name: fp32 ndarray}. no_decay: names with wd=0 (norm gains /
    biases). step(grads, stream) updates in place; .weights() returns the bf16-valued fp32
    weights for the forward (ancora/optim/adamw.py:69-109)."""

    def __init__(self, params, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.01, no_decay=(),
                 form="div", sr=False, seed=0, grad_dtype=np.float32):
        _lib.init()
        self.lr, (self.b1, self.b2), self.eps, self.wd = lr, betas, eps, wd
        if form not in ("div", "ibc"):
            raise ValueError("form must be 'div' or 'ibc'")
        self.form, self.sr, self.seed = form, bool(sr), int(seed)
        self.t = 0
        self.st = {}
        gdt = np.dtype(grad_dtype)
        _g_code(gdt)
        for name, p in params.items():
            if p.size % C:
                # the reference silently truncates (R = p.size // C, adamw.py:79); refuse instead
                raise ValueError(f"AdamW: '{name}' has {p.size} elements, not a multiple of {C}")
            R = p.size // C
            flat = np.ascontiguousarray(p, dtype=np.float32).reshape(R, C)
            self.st[name] = dict(
                shape=p.shape, R=R, otm=_pick_otm(R), wd=0.0 if name in no_decay else wd,
                g=DevBuf.zeros((R, C), gdt),
                m=DevBuf.zeros((R, C), np.float32), v=DevBuf.zeros((R, C), np.float32),
                p32=DevBuf(flat), p16=DevBuf.zeros((R, C), np.uint16))
        self._table = None
        self._table_key = None
        self.last_skipped = False
        self._steps = None           # device table of per-step bias corrections (steps counted on the device)
        self._steps_cap = 0
        self._steps_saturated = False
        self._steps_old = []

    # -- steps counted on the device: bias corrections by step, filled ahead
    def _bias_corrections(self, t):
        if self.form == "div":
            return 1 - self.b1 ** t, 1 - self.b2 ** t
        return 1.0 / (1.0 - self.b1 ** t), 1.0 / (1.0 - self.b2 ** t)

    def _ensure_step_table(self, t_upper):
        """Device table of anc_adamw_step_t whose entry t holds the bias corrections of step t, the
        same Python-double values rounded to fp32 once that `_hyper` passes per step. It ends where
        both corrections have reached 1.0f (the kernel uses the last entry for every later step);
        while they have not, it is extended ahead of `t_upper`, the largest step the next launch
        can be."""
        if self._steps is not None and (self._steps_saturated or t_upper < self._steps_cap):
            return
        cap = max(1024, 2 * self._steps_cap, 2 * int(t_upper))
        tab = (AdamWStepEntry * (cap + 1))()
        one = np.float32(1.0)
        n, saturated = cap, False
        for t in range(1, cap + 1):
            bc1, bc2 = self._bias_corrections(t)
            tab[t].bc1, tab[t].bc2 = bc1, bc2
            if np.float32(bc1) == one and np.float32(bc2) == one:
                n, saturated = t, True
                break
        if self._steps is not None:
            self._steps_old.append(self._steps)      # a launch in flight may still read it
        self._steps = DevBuf(np.frombuffer(tab, dtype=np.uint32, count=4 * (n + 1)).copy())
        self._steps_cap, self._steps_saturated = n, saturated

    # -- descriptor table: one row per tensor, rebuilt only when a gradient pointer changes
    def _build_table(self, gbufs):
        key = tuple((g.ptr, g.dtype.str) for g in gbufs)
        if key == self._table_key:
            return
        if self._table is not None:
            self._table.free()
        descs, blk0 = [], 0
        for seed, ((name, s), g) in enumerate(zip(self.st.items(), gbufs)):
            n = s["R"] * C
            if g.size != n:
                raise ValueError(f"AdamW: gradient of '{name}' has {g.size} elements, expected {n}")
            descs.append(AdamWDesc(g.ptr, s["m"].ptr, s["v"].ptr, s["p32"].ptr, s["p16"].ptr, n,
                                   blk0, s["wd"], seed, _g_code(g.dtype), 0))
            blk0 += api.anc_adamw_num_blocks(n)
        self._total_blocks = blk0
        self._table = upload_table(descs)
        self._table_key = key

    def _hyper(self):
        sb = sr_seed_base(self.seed, self.t) if self.sr else 0
        if self.form == "div":
            return hyper_div(self.lr, self.b1, self.b2, self.eps, self.t, self.sr, sb)
        ibc1 = 1.0 / (1.0 - self.b1 ** self.t)
        ibc2 = 1.0 / (1.0 - self.b2 ** self.t)
        return hyper_ibc(self.lr, self.b1, self.b2, self.eps, ibc1, ibc2, self.sr, sb)

    def launch(self, grads, stream_int, guard=None, device_steps=False, t_upper=None):
        """Asynchronous part of the step: upload host gradients (DevBuf gradients are used in
        place) and launch the fused kernel once over all tensors. `t` is advanced first, as in
        ancora/optim/adamw.py:89-91; a caller that later finds the step skipped calls `unstep()`.
        With `device_steps` the step count lives in the guard's control block (advanced by
        `guard.compute(..., count_step=True)` unless the step is skipped): the kernel takes the
        bias corrections of that step from a table and forms the rounding seed from the count, `t`
        here is left alone and nothing needs undoing; `t_upper` bounds the count from above."""
        if device_steps:
            if guard is None:
                raise ValueError("AdamW.launch: device_steps needs the guard whose block counts the steps")
            self._ensure_step_table(self.t + 1 if t_upper is None else t_upper)
        else:
            self.t += 1
        gbufs = []
        for name, s in self.st.items():
            g = grads[name]
            if isinstance(g, DevBuf):
                gbufs.append(g)
            else:
                g = np.asarray(g)
                if g.dtype != s["g"].dtype:
                    g = g.astype(np.float32) if s["g"].dtype == np.float32 else g
                    if g.dtype != s["g"].dtype:
                        raise TypeError(f"AdamW: gradient of '{name}' is {g.dtype}, the optimizer "
                                        f"was built for {s['g'].dtype}")
                s["g"].upload(g.reshape(s["R"], C), stream_int)
                gbufs.append(s["g"])
        self._build_table(gbufs)
        if device_steps:
            if self.form == "div":
                h = hyper_div(self.lr, self.b1, self.b2, self.eps, 1, False, self.seed)
            else:
                h = hyper_ibc(self.lr, self.b1, self.b2, self.eps, 1.0, 1.0, False, self.seed)
            h.sr = (SR_ON | SR_STEP_SEED) if self.sr else 0
            h.step_table, h.step_cap = self._steps.ptr, self._steps_cap
        else:
            h = self._hyper()
        api.anc_adamw_multi(self._table.ptr, len(self.st), self._total_blocks, ctypes.byref(h),
                            0 if guard is None else guard.ptr, int(stream_int))

    def unstep(self):
        """Undo the counter advance of a step the guard skipped (state was left untouched)."""
        self.t -= 1

    def step(self, grads, stream_int, guard=None):
        self.launch(grads, stream_int, guard)
        _lib.stream_sync(stream_int)                       # ancora/optim/adamw.py:98
        self.last_skipped = False
        if guard is not None and guard.read(stream_int)["skip"]:
            self.unstep()
            self.last_skipped = True

    def weights(self):
        """bf16-valued fp32 weights (what the forward consumes), per name."""
        return {n: _bits_f32(s["p16"].numpy()).reshape(s["shape"]) for n, s in self.st.items()}

    def state_dict(self):
        """Everything a resumed run needs, as host arrays: per tensor the fp32 master, both
        moments and the bf16 weights, plus the step counter (it enters the bias corrections and
        the stochastic-rounding seed). The reference has no optimizer checkpoint at all."""
        out = {"t": np.int64(self.t)}
        for n, s in self.st.items():
            for k in ("p32", "m", "v", "p16"):
                out[f"{n}/{k}"] = s[k].to_numpy()
        return out

    def load_state_dict(self, sd, stream_int=0):
        for n, s in self.st.items():
            for k in ("p32", "m", "v", "p16"):
                a = np.asarray(sd[f"{n}/{k}"])
                if a.size != s[k].size or a.dtype != s[k].dtype:
                    raise ValueError(f"AdamW.load_state_dict: '{n}/{k}' is {a.dtype}[{a.size}], "
                                     f"expected {s[k].dtype}[{s[k].size}]")
                s[k].upload(a.reshape(s[k].shape), stream_int)
        self.t = int(sd["t"])

    def master(self):
        return {n: s["p32"].numpy().reshape(s["shape"]) for n, s in self.st.items()}

    def moments(self):
        return {n: (s["m"].numpy().reshape(s["shape"]), s["v"].numpy().reshape(s["shape"]))
                for n, s in self.st.items()}

    def free(self):
        for s in self.st.values():
            for k in ("g", "m", "v", "p32", "p16"):
                s[k].free()
        if self._table is not None:
            self._table.free()
            self._table = None
        for b in self._steps_old + ([self._steps] if self._steps is not None else []):
            b.free()
        self._steps, self._steps_old = None, []
