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
import ctypes

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
