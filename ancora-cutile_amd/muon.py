"""Muon (momentum orthogonalised by Newton-Schulz) on the MI355X.

Mirror of ancora/optim/muon.py: the host-API class `Muon`, the device-resident classes
`DeviceMuon`, `MuonScratch`, `ResidentMuon`, `BatchedProjMuon`, and `newton_schulz5`.
In the reference the host class runs Newton-Schulz in numpy on the CPU and the
resident classes chain cuda-tile kernels one weight (or one chunk of 8) at a time;
here every class drives the same engine: all weights of one Newton-Schulz shape
(M = min(K,N), Nn = max(K,N)) form one packed fp32 batch, and a step is three
launches per batch -- momentum for every weight, the whole NS chain, update + bf16
refresh for every weight. Tall weights (K > N) enter and leave the batch transposed
inside those elementwise kernels (ancora/optim/muon.py:72-74, 264-274).

    buf = mu*buf + g;  u = g + mu*buf (Nesterov);  O = NS(u);  W -= lr*sqrt(max(1,K/N))*O

Batching is bitwise neutral: a weight's result does not depend on which other weights
share its batch, on `chunk` or on `scope` (tests/training/test_batched_proj_muon.py:74).
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import api, MuonDesc, F32, BF16, MUON_MAX_SCALES, SR_ON, SR_STEP_SEED
from .bf16 import bf16_bits, bits_f32, bf16_round as _bf        # noqa: F401
from .devbuf import DevBuf, upload_table
from . import muon_ns
from .muon_ns import NTM, _KELLER, NsWorkspace


def _g_code(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return F32
    if dtype == np.uint16:
        return BF16
    raise TypeError(f"gradient dtype {dtype}: expected float32 or uint16 (bf16 bits)")


def _check_aligned(K, N, what="Muon weight"):
    # same alignment rule as the reference's asserts (ancora/optim/muon.py:98,172,233)
    if K % NTM or N % NTM:
        raise ValueError(f"{what} ({K},{N}) tile-misaligned: both dims must be multiples of {NTM}")


def _f32bf_trunc(x):
    """Truncating fp32 -> bf16 bits: the reference's *initial* p16 (`f32_to_bf16_bits`,
    ancora/kernels/loss.py:273-274, used at ancora/optim/muon.py:105). After the first step p16
    is the RNE of p32."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


class _Batch:
    """One packed Newton-Schulz batch: weights of one (M, Nn) shape, its descriptor table."""

    def __init__(self, M, Nn, weights):
        self.M, self.Nn, self.weights = M, Nn, weights
        self.E = len(weights)
        self.table = None
        self.key = None
        self.total_blocks = 0
        self.fro = None              # per-block sums of u*u left by the pair momentum kernel

    def build(self, U, scale_index):
        key = tuple((w["G"].ptr, w["G"].dtype.str, w["p32"].ptr, w["p16"].ptr if w["p16"] is not None else 0,
                     w["buf"].ptr, w["p16T"].ptr if w.get("p16T") is not None else 0)
                    for w in self.weights) + (U.ptr,)
        if key == self.key:
            return
        if self.table is not None:
            self.table.free()
        descs, blk0 = [], 0
        for i, w in enumerate(self.weights):
            K, N = w["K"], w["N"]
            descs.append(MuonDesc(w["buf"].ptr, w["G"].ptr, w["p32"].ptr,
                                  w["p16"].ptr if w["p16"] is not None else 0,
                                  U.ptr + i * self.M * self.Nn * 4, K, N, int(K > N),
                                  _g_code(w["G"].dtype), scale_index[w["scale"]], w["seed"], blk0,
                                  w["p16T"].ptr if w.get("p16T") is not None else 0))
            blk0 += (K * N) // 4096
        self.total_blocks = blk0
        self.table = upload_table(descs)
        self.key = key

    def free(self):
        if self.table is not None:
            self.table.free()
            self.table = None
        if self.fro is not None:
            self.fro.free()
            self.fro = None


class MuonEngine:
    """Shape-grouped, batched Muon over device-resident weights.

    weights: list of dicts {buf, p32, p16, G: DevBuf; K, N: int; lid: int (optional)} -- the
    record of ancora/optim/muon.py:220; an optional `p16T` DevBuf (N,K) is a transposed bf16
    copy that the update refreshes in the same pass. `chunk` caps the matrices per batch (None = the whole
    shape group, which is what 288 GB of HBM is for); `scope=k` sub-groups by lid // k
    (ancora/optim/muon.py:221-222,235). Neither changes any result bit."""

    MAX_STREAMS = 4      # batches are dealt round-robin onto at most this many streams

    def __init__(self, weights, momentum=0.95, ns_steps=5, nesterov=True, chunk=None, scope=None,
                 mode="bf16", sr=False, seed=0, workspace=None, concurrent=True):
        _lib.init()
        self.mom, self.ns, self.nesterov = float(momentum), int(ns_steps), bool(nesterov)
        self.mode, self.sr, self.seed = mode, bool(sr), int(seed)
        self.t = 0
        # Fused prologue: the momentum kernel writes the chain's bf16-pair input and the partial
        # sums of the Frobenius norm, and the first Newton-Schulz step applies the scale, so the
        # norm and scaling passes over the batch do not exist. Needs a bf16 mode and >= 2 steps
        # (the fp32 result overlays the pair); otherwise the fp32 hand-off is used.
        self.fused_prologue = mode != "fp32" and self.ns >= 2
        # Grouped launches: the chains of up to 4 shape groups advance together, each product of
        # each Newton-Schulz step being one launch over all of them (no partly filled last wave
        # of workgroups per group). Needs the fused prologue, private buffers per batch and
        # dims that are multiples of 256; other batches run one by one.
        self.grouped = True
        # Fused update: the epilogue of the chain's last product applies W -= lr*O itself (grouped
        # path only; a weight with a transposed bf16 copy to refresh keeps the separate kernel).
        self.fused_update = True
        groups = {}
        scales = []
        for idx, w in enumerate(weights):
            K, N = int(w["K"]), int(w["N"])
            _check_aligned(K, N)
            w["tr"] = K > N
            w["M"], w["Nn"] = (N, K) if w["tr"] else (K, N)
            if "scale" not in w:                                  # (a zero-padded weight brings its own)
                w["scale"] = max(1.0, K / N) ** 0.5              # ancora/optim/muon.py:232
            w.setdefault("seed", idx)
            if w["scale"] not in scales:
                scales.append(w["scale"])
            key = (w["M"], w["Nn"]) if scope is None else (w["M"], w["Nn"], w.get("lid", 0) // scope)
            groups.setdefault(key, []).append(w)
        if len(scales) > MUON_MAX_SCALES:
            raise ValueError(f"more than {MUON_MAX_SCALES} distinct K/N ratios in one Muon group")
        self.scales = scales
        self.scale_index = {s: i for i, s in enumerate(scales)}
        self.batches = []
        for key, ws in groups.items():
            c = len(ws) if chunk is None else max(1, min(int(chunk), len(ws)))
            for i0 in range(0, len(ws), c):
                self.batches.append(_Batch(key[0], key[1], ws[i0:i0 + c]))
        self.groups = groups
        self._own_ws = workspace is None
        # With its own scratch the engine gives every batch a private packed buffer, workspace
        # and stream: the chains of different shape groups are independent, so they run
        # concurrently and fill each other's tails and memory-bound epilogues. A caller-owned
        # (shared) workspace means one chain at a time on the caller's stream.
        self.concurrent = bool(concurrent) and self._own_ws and len(self.batches) > 1
        self.serial = False          # True: keep the private buffers but launch everything on `si`
        self._forked = False
        self._n_forked = 0
        self._streams, self._fork, self._join = [], None, []
        if self.concurrent:
            for b in self.batches:
                b.U = DevBuf.empty((b.E * b.M * b.Nn,), np.float32)
                b.ws = NsWorkspace()
                b.ws.ensure(muon_ns.ns_workspace_bytes(b.E, b.M, b.Nn, mode))
                if len(self._streams) < self.MAX_STREAMS:
                    self._streams.append(_lib.stream_create())
                self._join.append(_lib.Event())
            self._fork = _lib.Event()
            self.ws = None
            self.U = None
        else:
            self.ws = NsWorkspace() if workspace is None else workspace
            self.U = None
            umax = max(b.E * b.M * b.Nn for b in self.batches) if self.batches else 0
            wmax = max(muon_ns.ns_workspace_bytes(b.E, b.M, b.Nn, mode) for b in self.batches) \
                if self.batches else 0
            if umax:
                self.U = DevBuf.empty((umax,), np.float32)
                self.ws.ensure(wmax)
            for b in self.batches:
                b.U, b.ws = self.U, self.ws

    def nbytes(self):
        if self.concurrent:
            return sum(b.U.nbytes + b.ws.nbytes() for b in self.batches)
        return (self.U.nbytes if self.U is not None else 0) + self.ws.nbytes()

    def step(self, si, lr=0.02, schedule=_KELLER, guard=None, defer_join=False, device_steps=False):
        """One Muon step over every weight. Asynchronous on stream `si`: the work is ordered
        after everything already queued on `si`, and (unless defer_join) `si` waits for it.
        `device_steps`: the step count lives in the guard's control block (see `AdamW.launch`); the
        kernels form the rounding seed from it and `t` here is left alone."""
        schedule = muon_ns._resolve(schedule)
        ctl = 0 if guard is None else guard.ptr
        lr_scales = (ctypes.c_float * MUON_MAX_SCALES)(*[lr * s for s in self.scales])
        if device_steps:
            if guard is None:
                raise ValueError("MuonEngine.step: device_steps needs the guard whose block counts the steps")
            self._sr_arg = (SR_ON | SR_STEP_SEED) if self.sr else 0
            seed_base = self.seed & 0xFFFFFFFF
        else:
            self.t += 1
            self._sr_arg = int(self.sr)
            seed_base = ((self.seed + 1000003 * self.t) & 0xFFFFFFFF) if self.sr else 0
        coef = muon_ns.coef_array(schedule, self.ns)
        self._run_mode = muon_ns.effective_mode(self.mode, schedule)
        together = [b for b in self.batches
                    if self.grouped and self.fused_prologue and b.M % 256 == 0 and b.Nn % 256 == 0]
        if not self.concurrent and len(self.batches) > 1:
            # shared packed buffer and workspace: one batch per call, and only if that buys the
            # fused update
            per_call = 1
            if not self.fused_update:
                together = []
        else:
            per_call = 4
            if len(together) < 2 and not self.fused_update:
                together = []
        alone = [b for b in self.batches if b not in together]
        for i0 in range(0, len(together), per_call):
            self._step_grouped(together[i0:i0 + per_call], si, ctl, coef, lr_scales, seed_base)
        forked = self.concurrent and not self.serial and len(alone) > 1
        if forked:
            self._fork.record(si)
        for i, b in enumerate(alone):
            st = si
            if forked:
                st = self._streams[i % len(self._streams)]
                if i < len(self._streams):
                    self._fork.wait_on(st)
            b.build(b.U, self.scale_index)
            buf = b.ws.ensure(muon_ns.ns_workspace_bytes(b.E, b.M, b.Nn, self._run_mode))
            if self.fused_prologue:
                self._momentum_pair(b, ctl, st)
                n_el = b.E * b.M * b.Nn
                api.anc_ns_batched_pair(b.U.ptr, b.U.ptr + n_el * 2, b.fro.ptr,
                                        b.total_blocks // b.E, b.U.ptr, b.E, b.M, b.Nn, self.ns, coef,
                                        1e-7, muon_ns.MODES[self._run_mode], buf.ptr, buf.nbytes, int(st))
            else:
                api.anc_muon_momentum_multi(b.table.ptr, b.E, b.total_blocks, self.mom,
                                            int(self.nesterov), F32, ctl, int(st))
                api.anc_ns_batched(b.U.ptr, b.E, b.M, b.Nn, self.ns, coef, 1e-7,
                                   muon_ns.MODES[self._run_mode], buf.ptr, buf.nbytes, int(st))
            api.anc_muon_update_multi(b.table.ptr, b.E, b.total_blocks, lr_scales, F32,
                                      self._sr_arg, seed_base, ctl, int(st))
            if forked:
                self._join[i].record(st)
        self._forked = forked
        self._n_forked = len(alone) if forked else 0
        if forked and not defer_join:
            self.join(si)

    def _momentum_pair(self, b, ctl, st):
        if b.fro is None:
            b.fro = DevBuf.empty((b.total_blocks,), np.float64)
        api.anc_muon_momentum_multi_pair(b.table.ptr, b.E, b.total_blocks, self.mom, int(self.nesterov),
                                         b.U.ptr, b.E * b.M * b.Nn * 2, b.fro.ptr, ctl, int(st))

    def _step_grouped(self, group, si, ctl, coef, lr_scales, seed_base):
        probs = (_lib.NsProblem * len(group))()
        for k, b in enumerate(group):
            b.build(b.U, self.scale_index)
            buf = b.ws.ensure(muon_ns.ns_workspace_bytes(b.E, b.M, b.Nn, self._run_mode))
            self._momentum_pair(b, ctl, si)
            n_el = b.E * b.M * b.Nn
            probs[k] = _lib.NsProblem(b.U.ptr, b.U.ptr + n_el * 2, b.fro.ptr, b.U.ptr, buf.ptr,
                                      b.total_blocks // b.E, b.E, b.M, b.Nn, buf.nbytes)
        if self.fused_update and not any(w.get("p16T") is not None for b in group for w in b.weights):
            tables = (ctypes.c_uint64 * len(group))(*[b.table.ptr for b in group])
            api.anc_muon_ns_update_multi(probs, len(group), tables, self.ns, coef, 1e-7,
                                         muon_ns.MODES[self._run_mode], lr_scales, self._sr_arg, seed_base, ctl,
                                         int(si))
            return
        api.anc_ns_batched_pair_multi(probs, len(group), self.ns, coef, 1e-7, muon_ns.MODES[self._run_mode],
                                      int(si))
        for b in group:
            api.anc_muon_update_multi(b.table.ptr, b.E, b.total_blocks, lr_scales, F32,
                                      self._sr_arg, seed_base, ctl, int(si))

    def join(self, si):
        """Make stream `si` wait for the per-batch streams of the last step."""
        if self._forked:
            for ev in self._join[:self._n_forked]:
                ev.wait_on(si)

    def unstep(self):
        self.t -= 1

    def free(self):
        _lib.api.anc_device_sync()
        for b in self.batches:
            b.free()
        if self.concurrent:
            for b in self.batches:
                b.U.free()
                b.ws.free()
            for st in self._streams:
                api.anc_stream_destroy(st)
            for ev in self._join + [self._fork]:
                ev.free()
            self._streams = []
            return
        if self.U is not None:
            self.U.free()
            self.U = None
        if self._own_ws:
            self.ws.free()


def newton_schulz5(G, steps=5, eps=1e-7, schedule=None, mode="bf16", si=0):
    """Orthogonalise one host matrix on the device (the reference's host function,
    ancora/optim/muon.py:67-80, runs this in numpy; Keller coefficients by default as there).
    Returns an fp32 ndarray of the same shape. Both dims must be multiples of 128."""
    G = np.asarray(G, dtype=np.float32)
    K, N = G.shape
    _check_aligned(K, N, "newton_schulz5 input")
    X = np.ascontiguousarray(G.T) if K > N else G
    M, Nn = X.shape
    d = DevBuf(X)
    try:
        muon_ns.ns_batched(d, 1, M, Nn, si, steps=steps, eps=eps, schedule=schedule, mode=mode)
        out = d.to_numpy(si)
    finally:
        d.free()
    return np.ascontiguousarray(out.T) if K > N else out


class MuonScratch:
    """Shared transient Newton-Schulz scratch for per-weight resident Muon
    (ancora/optim/muon.py:138-159): sized for the largest weight, one for the whole model."""

    def __init__(self, shapes, mode="bf16"):
        self.mode = mode
        self.ws = NsWorkspace()
        kn = max(int(K) * int(N) for K, N in shapes)
        need = max(muon_ns.ns_workspace_bytes(1, min(K, N), max(K, N), mode) for K, N in shapes)
        self.ws.ensure(need)
        self.u = DevBuf.empty((kn,), np.float32)

    def nbytes(self):
        return self.ws.nbytes() + self.u.nbytes

    def free(self):
        self.ws.free()
        self.u.free()


class ResidentMuon:
    """Per-2D-weight Muon over the layer's existing buffers (p32 master + the p16 the GEMM reads)
    with a shared MuonScratch; the only persistent state is the momentum buffer
    (ancora/optim/muon.py:162-204)."""

    def __init__(self, p32, p16, K, N, scratch, momentum=0.95, ns_steps=5, mode=None):
        _check_aligned(K, N)
        self.p32, self.p16, self.K, self.N, self.sc = p32, p16, K, N, scratch
        self.tr = K > N
        self.M, self.Nn = (N, K) if self.tr else (K, N)
        self.shape_scale = max(1.0, K / N) ** 0.5
        self.mom, self.ns = momentum, ns_steps
        self.mode = scratch.mode if mode is None else mode
        self.buf = DevBuf.zeros((K, N), np.float32)

    def step(self, g_dev, si, lr=0.02, schedule=_KELLER, guard=None):
        """g_dev: (K,N) device weight-gradient (float32, or uint16 bf16 bits)."""
        K, N, sc = self.K, self.N, self.sc
        ctl = 0 if guard is None else guard.ptr
        api.anc_muon_momentum(self.buf.ptr, g_dev.ptr, sc.u.ptr, K, N, float(self.mom), 1,
                              int(self.tr), _g_code(g_dev.dtype), F32, ctl, int(si))
        muon_ns.ns_batched(sc.u, 1, self.M, self.Nn, si, steps=self.ns, schedule=schedule,
                           mode=self.mode, workspace=sc.ws)
        api.anc_muon_update(self.p32.ptr, self.p16.ptr, sc.u.ptr, K, N,
                            float(lr * self.shape_scale), int(self.tr), F32, 0, 0, ctl, int(si))

    def free(self):
        self.buf.free()


class DeviceMuon:
    """Device-resident Muon over one 2-D weight with its own state and scratch
    (ancora/optim/muon.py:88-135)."""

    def __init__(self, W, lr=0.02, momentum=0.95, ns_steps=5, mode="bf16"):
        K, N = W.shape
        _check_aligned(K, N)
        self.K, self.N = K, N
        self.lr = lr
        self.p32 = DevBuf(np.ascontiguousarray(W, dtype=np.float32))
        self.p16 = DevBuf(_f32bf_trunc(W))
        self._scratch = MuonScratch([(K, N)], mode)
        self._rm = ResidentMuon(self.p32, self.p16, K, N, self._scratch, momentum, ns_steps)
        self.buf = self._rm.buf

    def step(self, g_dev, si, schedule=_KELLER):
        self._rm.step(g_dev, si, self.lr, schedule)

    def master(self):
        return self.p32.to_numpy()

    def free(self):
        self._rm.free()
        self._scratch.free()
        self.p32.free()
        self.p16.free()


class BatchedProjMuon:
    """Model-level batched Muon over all 2-D projection weights across layers
    (ancora/optim/muon.py:207-284). weights: list of {buf, p32, p16, G, K, N, lid}."""

    def __init__(self, weights, momentum=0.95, ns_steps=5, chunk=8, scope=None, mode="bf16",
                 sr=False, seed=0):
        self.mom, self.ns = momentum, ns_steps
        self.engine = MuonEngine(weights, momentum, ns_steps, True, chunk, scope, mode, sr, seed)
        self.groups = self.engine.groups

    def step(self, si, lr=0.02, schedule=_KELLER, guard=None):
        self.engine.step(si, lr, schedule, guard)

    def free(self):
        self.engine.free()


def _ceil_tile(n):
    return (int(n) + NTM - 1) // NTM * NTM


class Muon:
    """fp32-master Muon for 2-D matrix params (ancora/optim/muon.py:287-318). params:
    {name: (R,C) fp32 ndarray}; a 3-D [E,R,C] entry is E independent slices. The reference's host
    class runs Newton-Schulz on the CPU unless `device=True`; this one always runs on the GPU, so
    `device` and `si` are accepted and only `si` is used (as the default stream). `schedule`
    defaults to the process-wide setting of `set_polar_express` (Keller unless switched).

    A 2-D matrix whose dims are not multiples of 128 (the (H, E) router of a MoE model under the
    default routing predicate) cannot enter the tiled chain as it is; the reference runs its
    Newton-Schulz on the host for those (`_ns_ok`, ancora/optim/muon.py:37-41, 307). Here its
    state lives zero-padded to the next multiples of 128: the padding rows and columns of the
    iterate stay exactly zero through the chain (A = X X^T has zero rows there, B X as well), the
    Frobenius norm does not see them, so the result is the Newton-Schulz of the matrix itself,
    padded; the shape factor sqrt(max(1, rows/cols)) is that of the original dims. Such a matrix
    takes host gradients (or a DevBuf already padded); accessors return the original shape."""

    def __init__(self, params, lr=0.02, momentum=0.95, nesterov=True, ns_steps=5, device=False,
                 si=None, schedule=_KELLER, mode="bf16", chunk=None, sr=False, seed=0,
                 grad_dtype=np.float32):
        _lib.init()
        self.lr, self.mom, self.nesterov, self.ns = lr, momentum, nesterov, ns_steps
        self.device, self.si, self.schedule = device, si, schedule
        self.st = {}
        recs = []
        gdt = np.dtype(grad_dtype)
        for n, p in params.items():
            assert p.ndim in (2, 3), f"Muon is for 2D matrices, {n} is {p.shape}"
            K0, N0 = p.shape[-2], p.shape[-1]
            K, N = _ceil_tile(K0), _ceil_tile(N0)
            pad = (K0, N0) if (K, N) != (K0, N0) else None
            if pad is not None and p.ndim != 2:
                _check_aligned(K0, N0, f"stacked Muon weight '{n}'")
            E = 1 if p.ndim == 2 else p.shape[0]
            s = dict(shape=p.shape, E=E, K=K, N=N, pad=pad)
            s.update(p32=DevBuf(self._padded(s, np.ascontiguousarray(p, dtype=np.float32)).reshape(E * K, N)),
                     p16=DevBuf.zeros((E * K, N), np.uint16),
                     buf=DevBuf.zeros((E * K, N), np.float32),
                     g=DevBuf.zeros((E * K, N), gdt))
            self.st[n] = s
            for e in range(E):
                r = dict(buf=s["buf"].at_pos(e * K), p32=s["p32"].at_pos(e * K),
                         p16=s["p16"].at_pos(e * K), G=s["g"].at_pos(e * K), K=K, N=N,
                         name=n, e=e)
                if pad is not None:
                    r["scale"] = max(1.0, K0 / N0) ** 0.5      # ancora/optim/muon.py:308, original dims
                recs.append(r)
        self._recs = recs
        self._recs_of = {}
        for r in recs:
            self._recs_of.setdefault(r["name"], []).append(r)
        self._gptr = {}                       # name -> pointer of the resident gradient last bound
        self.engine = MuonEngine(recs, momentum, ns_steps, nesterov, chunk, None, mode, sr, seed) \
            if recs else None
        self.last_skipped = False

    @staticmethod
    def _padded(s, a):
        """Host array `a` of the parameter's own shape, zero-padded to the stored (K, N)."""
        if s["pad"] is None:
            return a
        out = np.zeros((s["K"], s["N"]), a.dtype)
        out[:s["pad"][0], :s["pad"][1]] = a.reshape(s["pad"])
        return out

    @staticmethod
    def _unpadded(s, a):
        a = a.reshape(s["E"] * s["K"], s["N"])
        if s["pad"] is not None:
            a = np.ascontiguousarray(a[:s["pad"][0], :s["pad"][1]])
        return a.reshape(s["shape"])

    def host_grad(self, n, g):
        """A host gradient of parameter `n` as the array its device buffer takes: the buffer's
        dtype, zero-padded where the state is."""
        s = self.st[n]
        g = np.asarray(g)
        if g.dtype != s["g"].dtype:
            if s["g"].dtype == np.float32:
                g = g.astype(np.float32)
            else:
                raise TypeError(f"Muon: gradient of '{n}' is {g.dtype}, the optimizer was "
                                f"built for {s['g'].dtype}")
        return self._padded(s, g).reshape(s["E"] * s["K"], s["N"])

    def launch(self, grads, stream_int=None, guard=None, defer_join=False, device_steps=False):
        si = stream_int if stream_int is not None else (self.si or 0)
        for n, s in self.st.items():
            g = grads[n]
            if isinstance(g, DevBuf):
                if g.size != s["E"] * s["K"] * s["N"]:
                    raise TypeError(f"Muon: the resident gradient of '{n}' has {g.size} elements; its state is "
                                    f"stored as {(s['E'] * s['K'], s['N'])} (zero-padded to multiples of {NTM}): "
                                    "pass a host gradient or a DevBuf padded the same way")
                if self._gptr.get(n) != (g.ptr, g.dtype.str):
                    gv = g.view((s["E"] * s["K"], s["N"]))
                    for r in self._recs_of[n]:
                        r["G"] = gv.at_pos(r["e"] * s["K"])
                    self._gptr[n] = (g.ptr, g.dtype.str)
            else:
                if n in self._gptr:               # back to the optimizer's own gradient buffer
                    for r in self._recs_of[n]:
                        r["G"] = s["g"].at_pos(r["e"] * s["K"])
                    del self._gptr[n]
                s["g"].upload(self.host_grad(n, g), si)
        if self.engine is not None:
            self.engine.step(si, self.lr, self.schedule, guard, defer_join, device_steps)
        return si

    def join(self, si):
        if self.engine is not None:
            self.engine.join(si)

    def unstep(self):
        if self.engine is not None:
            self.engine.unstep()

    def step(self, grads, stream_int=None, guard=None):
        si = self.launch(grads, stream_int, guard)
        _lib.stream_sync(si)
        self.last_skipped = False
        if guard is not None and guard.read(si)["skip"]:
            self.unstep()
            self.last_skipped = True

    def state_dict(self):
        """Host arrays for a resumed run: per weight the fp32 master, the momentum buffer and the
        bf16 weights, plus the step counter (it seeds the stochastic rounding)."""
        out = {"t": np.int64(self.engine.t if self.engine is not None else 0)}
        for n, s in self.st.items():
            for k in ("p32", "buf", "p16"):
                out[f"{n}/{k}"] = s[k].to_numpy()
        return out

    def load_state_dict(self, sd, stream_int=0):
        for n, s in self.st.items():
            for k in ("p32", "buf", "p16"):
                a = np.asarray(sd[f"{n}/{k}"])
                if a.size != s[k].size or a.dtype != s[k].dtype:
                    raise ValueError(f"Muon.load_state_dict: '{n}/{k}' is {a.dtype}[{a.size}], "
                                     f"expected {s[k].dtype}[{s[k].size}]")
                s[k].upload(a.reshape(s[k].shape), stream_int)
        if self.engine is not None:
            self.engine.t = int(sd["t"])

    def weights(self):
        """bf16-valued fp32 weights for the forward (ancora/optim/muon.py:311-312)."""
        return {n: _bf(self._unpadded(s, s["p32"].to_numpy())) for n, s in self.st.items()}

    def weights16(self):
        """The device-maintained bf16 copy (RNE or SR of the master), as fp32 values."""
        return {n: bits_f32(self._unpadded(s, s["p16"].to_numpy())) for n, s in self.st.items()}

    def master(self):
        return {n: self._unpadded(s, s["p32"].to_numpy()) for n, s in self.st.items()}

    def momentum_buffers(self):
        return {n: self._unpadded(s, s["buf"].to_numpy()) for n, s in self.st.items()}

    def free(self):
        if self.engine is not None:
            self.engine.free()
        for s in self.st.values():
            for k in ("p32", "p16", "buf", "g"):
                s[k].free()
