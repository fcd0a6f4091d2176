"""Optimizer for stacked MoE expert tensors and the router on the MI355X.

Mirror of the optimizer part of ancora/kernels/moe.py: `ExpertMuonScratch` (:404-421) and
`GroupedMoEFFN.init_adamw` / `.step` (:525-609), lifted out of the FFN class (whose forward
and backward are not part of this package) into `ExpertOptimizer`. Expert tensors are
stacked [E, K, N]; with optimizer="muon" every expert slice is one matrix of a batched
Newton-Schulz chain (fp32 master + one momentum buffer, no second moment), otherwise the
flat tensor goes through AdamW. The router stays on AdamW (wd = 0, :603-604). The transposed
copies the backward reads (`_transpose_e`, :370-377, 593-597) are refreshed by the Muon update
kernel in the same pass; the AdamW variant runs the transpose kernel after the step.
"""
import numpy as np

from . import _lib
from ._lib import api
from .adamw import _adamw, _pick_otm, C as AC
from .devbuf import DevBuf
from .muon import MuonEngine
from .muon_ns import NsWorkspace, ns_workspace_bytes, _KELLER


class ExpertMuonScratch:
    """Shared batched-NS scratch for Muon over the experts of every MoE layer and of the three
    weight tensors, which run sequentially on one stream (ancora/kernels/moe.py:404-421)."""

    def __init__(self, E, M, mode="bf16"):
        self.ws = NsWorkspace()
        self.ws.ensure(ns_workspace_bytes(E, M, M, mode))

    def nbytes(self):
        return self.ws.nbytes()

    def free(self):
        self.ws.free()


class ExpertOptimizer:
    """weights: {"gate_proj": [E,H,Ie], "up_proj": [E,H,Ie], "down_proj": [E,Ie,H]} fp32 masters;
    router: (H,E) fp32 or None. Gradients are DevBufs of the same shapes (float32, or uint16 bf16
    bits), passed to step()."""

    NAMES = ("gate_proj", "up_proj", "down_proj")

    def __init__(self, weights, router=None, optimizer="muon", betas=(0.9, 0.999), eps=1e-8,
                 wd=0.0, momentum=0.95, ns_steps=5, muon_scratch=None, mode="bf16"):
        _lib.init()
        self.optimizer, self._betas, self._eps, self._wd, self._t = optimizer, betas, eps, wd, 0
        self.st = {}
        for name in self.NAMES:
            W = np.ascontiguousarray(weights[name], dtype=np.float32)
            E, K, N = W.shape
            s = dict(E=E, K=K, N=N, p32=DevBuf(W.reshape(E * K, N)),
                     p16=DevBuf.zeros((E * K, N), np.uint16), p16T=DevBuf.zeros((E * N, K), np.uint16))
            if optimizer == "muon":
                s["buf"] = DevBuf.zeros((E * K, N), np.float32)
            else:
                s["m"] = DevBuf.zeros((E * K, N), np.float32)
                s["v"] = DevBuf.zeros((E * K, N), np.float32)
            self.st[name] = s
        self._engine = None
        self._engine_key = None
        self._scratch = muon_scratch
        self._mom, self._ns, self._mode = momentum, ns_steps, mode
        self.router = None
        if router is not None:
            r = np.ascontiguousarray(router, dtype=np.float32)
            if r.size % AC:
                raise ValueError(f"router has {r.size} elements, not a multiple of {AC}")
            R = r.size // AC
            self.router = dict(shape=r.shape, R=R, otm=_pick_otm(R), p32=DevBuf(r.reshape(R, AC)),
                               m=DevBuf.zeros((R, AC), np.float32), v=DevBuf.zeros((R, AC), np.float32),
                               p16=DevBuf.zeros((R, AC), np.uint16))

    def _muon_engine(self, grads):
        key = tuple(grads[n].ptr for n in self.NAMES)
        if key != self._engine_key:
            if self._engine is not None:
                self._engine.free()
            recs = []
            for name in self.NAMES:
                s, g = self.st[name], grads[name]
                g2 = g.view((s["E"] * s["K"], s["N"]))
                for e in range(s["E"]):
                    recs.append(dict(buf=s["buf"].at_pos(e * s["K"]), p32=s["p32"].at_pos(e * s["K"]),
                                     p16=s["p16"].at_pos(e * s["K"]), G=g2.at_pos(e * s["K"]),
                                     p16T=s["p16T"].at_pos(e * s["N"]), K=s["K"], N=s["N"]))
            ws = None if self._scratch is None else self._scratch.ws
            self._engine = MuonEngine(recs, self._mom, self._ns, True, None, None, self._mode,
                                      workspace=ws)
            self._engine_key = key
        return self._engine

    def step(self, grads, si, lr=1e-3, muon_lr=0.02, router_grad=None, schedule=_KELLER, guard=None):
        """One optimizer step (ancora/kernels/moe.py:567-609): experts (batched Muon at muon_lr, or
        AdamW at lr), transposed-weight refresh, router AdamW with wd = 0."""
        self._t += 1
        b1, b2 = self._betas
        ibc1 = 1.0 / (1.0 - b1 ** self._t)
        ibc2 = 1.0 / (1.0 - b2 ** self._t)
        ctl = 0 if guard is None else guard.ptr
        if self.optimizer == "muon":
            self._muon_engine(grads).step(si, muon_lr, schedule, guard)
        else:
            for name in self.NAMES:
                s = self.st[name]
                _adamw(si, grads[name], s["m"], s["v"], s["p32"], s["p16"], 0, b1, b2, self._eps, lr,
                       self._wd, ibc1, ibc2, ctl)
        if self.optimizer != "muon":                 # Muon's update kernel refreshes p16T itself
            for name in self.NAMES:                  # the transposed backward weights
                s = self.st[name]
                api.anc_transpose_bf16(s["p16"].ptr, s["p16T"].ptr, s["E"], s["K"], s["N"], int(si))
        if self.router is not None and router_grad is not None:
            r = self.router
            _adamw(si, router_grad, r["m"], r["v"], r["p32"], r["p16"], r["otm"], b1, b2, self._eps,
                   lr, 0.0, ibc1, ibc2, ctl)

    def master(self):
        out = {n: s["p32"].to_numpy().reshape(s["E"], s["K"], s["N"]) for n, s in self.st.items()}
        if self.router is not None:
            out["router"] = self.router["p32"].to_numpy().reshape(self.router["shape"])
        return out

    def free(self):
        if self._engine is not None:
            self._engine.free()
        for s in self.st.values():
            for k in ("p32", "p16", "p16T", "buf", "m", "v"):
                if k in s:
                    s[k].free()
        if self.router is not None:
            for k in ("p32", "m", "v", "p16"):
                self.router[k].free()


class GroupedMoEFFNOptim:
    """The optimizer half of `GroupedMoEFFN` under its own method names, `init_adamw(si, ...)` and
    `step(si, lr, muon_lr)` (ancora/kernels/moe.py:525-609), as a mixin for the class that owns the
    layer's forward and backward. It works on the attributes that class already has and allocates
    only optimizer state:

        E, H, Ie            experts, hidden width, expert width
        optimizer           "muon" (batched Newton-Schulz per expert slice, square experts) or "adamw"
        w                   {"gate_proj", "up_proj", "down_proj": [E,K,N] fp32; "router": (H,E) fp32}
        Wg, Wu, Wd          packed bf16 forward weights, DevBuf (E*K, N): they ARE the optimizer's
                            p16 and are updated in place (moe.py:526-528)
        WgT, WuT, WdT       their transposes for the backward, DevBuf (E*N, K), refreshed by the step
        dWg, dWu, dWd       fp32 gradients, DevBuf (E*K, N), read on the step's stream
        device_route        True: router AdamW on the device over Wr_dev (H*E fp32 DevBuf, the master
                            the gating reads) with the gradient restored from Gr_acc into
                            G_router_dev; False: host AdamW on w["router"] with G_router (ndarray)
        _muon_lr, _muon_scr optional: default Muon learning rate, shared ExpertMuonScratch

    Sets `_wq_dirty_mx = True` after every step, as the reference does for its fp8 weight cache."""

    def init_adamw(self, si, betas=(0.9, 0.999), eps=1e-8, wd=0.0):
        _lib.init()
        self._AC, self._betas, self._eps, self._wd, self._t = AC, betas, eps, wd, 0
        E, H, Ie = self.E, self.H, self.Ie
        names = (("Wg", "gate_proj", H, Ie), ("Wu", "up_proj", H, Ie), ("Wd", "down_proj", Ie, H))
        self._eopt, self._muon, self._engine = {}, {}, None
        if self.optimizer == "muon":
            if Ie != H:
                raise ValueError(f"expert Muon assumes square experts (Ie={Ie}, H={H}), moe.py:539")
            recs = []
            for attr, key, K, N in names:
                master = np.ascontiguousarray(self.w[key], dtype=np.float32).reshape(E * K, N)
                s = dict(p32=DevBuf(master), buf=DevBuf.zeros((E * K, N), np.float32), p16=getattr(self, attr))
                self._muon[attr] = s
                g, pT = getattr(self, "d" + attr).view((E * K, N), np.float32), getattr(self, attr + "T")
                for e in range(E):
                    recs.append(dict(buf=s["buf"].at_pos(e * K), p32=s["p32"].at_pos(e * K),
                                     p16=s["p16"].view((E * K, N)).at_pos(e * K), G=g.at_pos(e * K),
                                     p16T=pT.view((E * N, K)).at_pos(e * N), K=K, N=N))
            scr = getattr(self, "_muon_scr", None)
            self._engine = MuonEngine(recs, 0.95, 5, True, None, None, "bf16",
                                      workspace=None if scr is None else scr.ws)
        else:
            for attr, key, K, N in names:
                flat = np.ascontiguousarray(self.w[key], dtype=np.float32).reshape(-1)
                R = flat.size // AC
                self._eopt[attr] = dict(R=R, otm=_pick_otm(R), p32=DevBuf(flat.reshape(R, AC)),
                                        m=DevBuf.zeros((R, AC), np.float32), v=DevBuf.zeros((R, AC), np.float32),
                                        p16=getattr(self, attr).view((R, AC), np.uint16), K=K, N=N)
        if getattr(self, "device_route", False):
            Rr = (H * E) // AC
            self._ropt = dict(R=Rr, otm=_pick_otm(Rr), p32=self.Wr_dev.view((Rr, AC), np.float32),
                              m=DevBuf.zeros((Rr, AC), np.float32), v=DevBuf.zeros((Rr, AC), np.float32),
                              p16=DevBuf.zeros((Rr, AC), np.uint16))
            self._router_dev_adam = True
        else:
            self._rm = np.zeros_like(self.w["router"], np.float32)
            self._rv = np.zeros_like(self.w["router"], np.float32)

    def step(self, si, lr=1e-3, muon_lr=None):
        self._t += 1
        b1, b2 = self._betas
        eps, wd = self._eps, self._wd
        ibc1 = 1.0 / (1.0 - b1 ** self._t)
        ibc2 = 1.0 / (1.0 - b2 ** self._t)
        E, H, Ie = self.E, self.H, self.Ie
        if self.optimizer == "muon":
            mlr = getattr(self, "_muon_lr", 0.02) if muon_lr is None else muon_lr
            self._engine.step(si, mlr)            # momentum, chain, update, bf16 and transposed bf16 refresh
        else:
            for attr, s in self._eopt.items():
                g = getattr(self, "d" + attr).view((s["R"], AC), np.float32)
                _adamw(si, g, s["m"], s["v"], s["p32"], s["p16"], s["otm"], b1, b2, eps, lr, wd, ibc1, ibc2)
            api.anc_transpose_bf16(self.Wg.ptr, self.WgT.ptr, E, H, Ie, int(si))
            api.anc_transpose_bf16(self.Wu.ptr, self.WuT.ptr, E, H, Ie, int(si))
            api.anc_transpose_bf16(self.Wd.ptr, self.WdT.ptr, E, Ie, H, int(si))
        self._wq_dirty_mx = True
        if getattr(self, "_router_dev_adam", False):
            self.G_router_dev.copy_from(self.Gr_acc, si)
            s = self._ropt
            gr = self.G_router_dev.view((s["R"], AC), np.float32)
            _adamw(si, gr, s["m"], s["v"], s["p32"], s["p16"], s["otm"], b1, b2, eps, lr, 0.0, ibc1, ibc2)
        else:
            g = np.asarray(self.G_router)
            self._rm = b1 * self._rm + (1 - b1) * g
            self._rv = b2 * self._rv + (1 - b2) * g * g
            upd = (self._rm * ibc1) / (np.sqrt(self._rv * ibc2) + eps) + wd * self.w["router"]
            self.w["router"] = self.w["router"].astype(np.float32) - lr * upd

    def free_optim(self):
        if self._engine is not None:
            self._engine.free()
        for d in list(self._muon.values()) + list(self._eopt.values()):
            for k in ("p32", "buf", "m", "v"):
                if k in d:
                    d[k].free()
        if getattr(self, "_router_dev_adam", False):
            for k in ("m", "v", "p16"):
                self._ropt[k].free()
