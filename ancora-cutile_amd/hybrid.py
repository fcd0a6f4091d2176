"""Muon + AdamW hybrid optimizer on the MI355X.

Mirror of ancora/optim/hybrid.py: `HybridOptimizer(params, is_muon, no_decay, muon_kw,
adamw_kw, si, muon_device)` with `.step(grads, stream_int)`, `.weights()`, `.routing()`,
`.free()` and the attributes `.muon`, `.adamw`, `.muon_names`, `.adamw_names`; the routing
predicate `default_is_muon`. Muon takes the 2-D hidden matrices, AdamW everything else
(gains, embedding, head), and `step` runs Muon first, then AdamW (hybrid.py:45-47).

Extensions, all off by default: `max_grad_norm` (one global norm over every gradient of both
groups, clip scale applied to g before the momentum / moment updates), the non-finite guard
that comes with it (a step with an Inf/NaN gradient leaves every state tensor untouched and
does not advance the step counters), stochastic-rounded bf16 weights, bf16 gradients.
"""
import numpy as np

from . import _lib
from .adamw import AdamW
from .devbuf import DevBuf
from .gradnorm import StepGuard
from .muon import Muon
from .muon_ns import NTM

_ADAMW_TOKENS = ("norm", "ln", "embed", "lm_head", "head", "wte", "wpe")


def default_is_muon(name, p):
    """2-D matrix that is not a norm gain / embedding / lm_head -> Muon (hybrid.py:18-25)."""
    if p.ndim != 2:
        return False
    low = name.lower()
    if any(t in low for t in _ADAMW_TOKENS):
        return False
    return True


def resident_is_muon(name, p):
    """Routing of the device-resident models: like `default_is_muon`, but a stacked [E,K,N]
    expert tensor is E Muon matrices (ancora/kernels/moe.py:433-435, 536-548) and a matrix
    that is not 128-aligned -- the (H, E) router -- stays on AdamW (`_ns_ok`,
    ancora/optim/muon.py:37-41)."""
    if p.ndim not in (2, 3):
        return False
    low = name.lower()
    if any(t in low for t in _ADAMW_TOKENS) or "router" in low:
        return False
    return p.shape[-2] % NTM == 0 and p.shape[-1] % NTM == 0


class HybridOptimizer:
    def __init__(self, params, is_muon=default_is_muon, no_decay=None, muon_kw=None,
                 adamw_kw=None, si=None, muon_device=False, max_grad_norm=None, guard=False,
                 grad_dtype=np.float32):
        muon_kw = {**dict(lr=0.02, momentum=0.95, ns_steps=5), **(muon_kw or {})}
        if muon_device:                      # the reference's switch for GPU Newton-Schulz;
            muon_kw.update(device=True, si=si)   # here the GPU path is the only path
        adamw_kw = adamw_kw or dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.01)
        if no_decay is None:
            # don't decay 1-D gains/biases (hybrid.py:35-36), nor a router that the predicate leaves
            # to AdamW: the resident models run it with wd = 0 (ancora/kernels/moe.py:603-604)
            no_decay = lambda n, p: (p.ndim == 1 or "router" in n.lower())          # noqa: E731

        # A 2-D matrix the predicate sends to Muon stays on Muon whatever its dims (lr, momentum,
        # no decay: what the reference trains it with): one whose dims are not multiples of 128, the
        # (H, E) router of a MoE model under `default_is_muon`, runs zero-padded through the same
        # chain (see `Muon`) where the reference falls back to host Newton-Schulz (`_ns_ok`,
        # ancora/optim/muon.py:37-41, 307).
        def _aligned(p):
            return p.shape[-2] % NTM == 0 and p.shape[-1] % NTM == 0
        self.muon_names = [n for n, p in params.items() if is_muon(n, p) and (_aligned(p) or p.ndim == 2)]
        self.muon_padded = [n for n in self.muon_names if not _aligned(params[n])]
        self.adamw_names = [n for n in params if n not in self.muon_names]
        self.muon = Muon({n: params[n] for n in self.muon_names}, grad_dtype=grad_dtype, **muon_kw)
        self.adamw = AdamW({n: params[n] for n in self.adamw_names},
                           no_decay=tuple(n for n in self.adamw_names if no_decay(n, params[n])),
                           grad_dtype=grad_dtype, **adamw_kw)
        self.guard = StepGuard(max_grad_norm) if (max_grad_norm is not None or guard) else None
        self._last_skipped = False
        self._last_ctl = None
        self._pending = None         # stream of an unsynchronised guarded step whose block was not read yet
        self._t_upper = 0            # guarded steps issued: the device's step count cannot exceed it

    # The guarded step counts its steps on the device (the guard's control block), so that a skipped
    # step needs no undo and `step(..., sync=False)` returns without a host synchronisation. The
    # host mirrors (`last_ctl`, `last_skipped`, the optimizers' `t`) are refreshed when the block
    # is read: right away in a synchronous step, on first use after an asynchronous one.
    def _refresh(self):
        if self._pending is None:
            return
        si, self._pending = self._pending, None
        self._last_ctl = self.guard.read(si)              # synchronises stream si
        self._last_skipped = self._last_ctl["skip"]
        self.adamw.t = self._last_ctl["t"]
        if self.muon.engine is not None:
            self.muon.engine.t = self._last_ctl["t"]

    @property
    def last_ctl(self):
        self._refresh()
        return self._last_ctl

    @property
    def last_skipped(self):
        self._refresh()
        return self._last_skipped

    def step_count(self):
        """Steps that passed the guard so far (reads the device block if a step is pending)."""
        self._refresh()
        return self.adamw.t

    def _grad_bufs(self, grads):
        """Gradient DevBufs in the fixed order of the global norm: Muon names, then AdamW names."""
        out = []
        for n in self.muon_names:
            g = grads[n]
            out.append(g if isinstance(g, DevBuf) else self.muon.st[n]["g"])
        for n in self.adamw_names:
            g = grads[n]
            out.append(g if isinstance(g, DevBuf) else self.adamw.st[n]["g"])
        return out

    def gn_partials_ptr(self, grads, name):
        """Device address where the grad-norm partial sums of gradient `name` live for this set of
        gradient buffers: a producer (`gemm_dW(..., gn_partials=...)`) that writes them there can be
        named in `step(..., produced=[...])`, and the norm then skips its pass over that tensor."""
        bufs = self._grad_bufs(grads)
        self.guard.plan(bufs)
        return self.guard.partials_ptr((self.muon_names + self.adamw_names).index(name))

    def step(self, grads, stream_int, produced=(), sync=True):
        """`produced`: names of resident gradients whose grad-norm partial sums their producer has
        already written (see `gn_partials_ptr`); same result bits with or without. `sync=False`
        (guarded steps with resident gradients): return as soon as the step is queued on
        `stream_int`, as the reference's resident step does (ancora/model/resident_train.py:338-339);
        `last_ctl` / `last_skipped` then read the device block when first asked."""
        if self.guard is None:
            self.muon.step({n: grads[n] for n in self.muon_names}, stream_int)
            self.adamw.step({n: grads[n] for n in self.adamw_names}, stream_int)
            return
        # guarded step: every gradient must be resident before the norm, so upload first
        for opt, names in ((self.muon, self.muon_names), (self.adamw, self.adamw_names)):
            for n in names:
                g = grads[n]
                if not isinstance(g, DevBuf):
                    s = opt.st[n]
                    if opt is self.muon:
                        g = self.muon.host_grad(n, g)
                    else:
                        g = np.asarray(g)
                        if g.dtype != s["g"].dtype and s["g"].dtype == np.float32:
                            g = g.astype(np.float32)
                    s["g"].upload(g.reshape(s["g"].shape), stream_int)
        resident = {}
        for opt, names in ((self.muon, self.muon_names), (self.adamw, self.adamw_names)):
            for n in names:
                g = grads[n]
                resident[n] = g if isinstance(g, DevBuf) else opt.st[n]["g"]
        order = self.muon_names + self.adamw_names
        if self._pending is not None and self._pending != stream_int:
            self._refresh()                # the block is reused: an unread step on another stream first
        self._t_upper += 1
        self.guard.compute(self._grad_bufs(grads), stream_int, produced=[order.index(n) for n in produced],
                           count_step=True)
        # Muon's per-shape chains fork onto their own streams; AdamW runs beside them
        self.muon.launch({n: resident[n] for n in self.muon_names}, stream_int, self.guard,
                         defer_join=True, device_steps=True)
        self.adamw.launch({n: resident[n] for n in self.adamw_names}, stream_int, self.guard,
                          device_steps=True, t_upper=self._t_upper)
        self.muon.join(stream_int)
        self._pending = stream_int
        if sync:
            self._refresh()

    def state_dict(self):
        """Optimizer state of both groups as one flat {key: ndarray} mapping."""
        self._refresh()
        out = {f"muon/{k}": v for k, v in self.muon.state_dict().items()}
        out.update({f"adamw/{k}": v for k, v in self.adamw.state_dict().items()})
        return out

    def load_state_dict(self, sd, stream_int=0):
        self.muon.load_state_dict({k[5:]: v for k, v in sd.items() if k.startswith("muon/")}, stream_int)
        self.adamw.load_state_dict({k[6:]: v for k, v in sd.items() if k.startswith("adamw/")}, stream_int)
        self._pending = None
        if self.guard is not None:
            self.guard.set_t(self.adamw.t, stream_int)
            self._t_upper = self.adamw.t
        _lib.stream_sync(stream_int)

    def save(self, path):
        """Checkpoint to one uncompressed .npz (plain arrays, no pickle): a run resumed with
        `load` continues bit for bit. The reference keeps optimizer state in memory only."""
        np.savez(self._npz(path), **self.state_dict())

    @staticmethod
    def _npz(path):
        """np.savez appends '.npz' to a name without it; `load` must look for the same file."""
        path = str(path)
        return path if path.endswith(".npz") else path + ".npz"

    def load(self, path, stream_int=0):
        with np.load(self._npz(path), allow_pickle=False) as z:
            self.load_state_dict({k: z[k] for k in z.files}, stream_int)

    def weights(self):
        return {**self.muon.weights(), **self.adamw.weights()}

    def routing(self):
        return {"muon": list(self.muon_names), "adamw": list(self.adamw_names)}

    def free(self):
        self.muon.free()
        self.adamw.free()
        if self.guard is not None:
            self.guard.free()
