"""Writes tests/golden/*.npz: small input/output vectors of the optimizer path, produced by the
numpy oracle (oracle/) on the inputs the reference's own tests describe (none of them ships
vectors: they draw from np.random.default_rng(seed), tests/optim/test_adamw.py:19-31,
tests/kernels/_probe_sr_ops.py:41-47, tests/kernels/_probe_polar_express_device.py:60-66). The
reference itself is not imported or run. The files pin the oracle against drift (tests/test_golden.py
re-derives them) and give the GPU parity tests a committed leg.

    python tests/golden/make_golden.py        (from the repository root)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.adamw_ref import AdamWRef                                   # noqa: E402
from oracle.bf16_ref import bf16_rne_bits, bf16_sr_bits, sr_dither      # noqa: E402
from oracle.gradnorm_ref import gradnorm_fixed, gradnorm_f64, control   # noqa: E402
from oracle.muon_ref import muon_momentum, muon_update, host_ns, PE_SCHEDULE  # noqa: E402
from oracle.quant_ref import quant_mxfp8_w                              # noqa: E402


def adamw_case():
    """tests/optim/test_adamw.py:19-43: seed 0, (256,64)*0.1 and (64,) ~ 1, grads *0.5, 5 steps."""
    rng = np.random.default_rng(0)
    p_w = (rng.standard_normal((256, 64)) * 0.1).astype(np.float32)
    p_n = (1.0 + rng.standard_normal(64) * 0.05).astype(np.float32)
    opt = AdamWRef({"w": p_w, "n": p_n}, 0.01, (0.9, 0.999), 1e-8, 0.01, ("n",), form="div")
    gw, gn = [], []
    for _ in range(5):
        g = {"w": (rng.standard_normal((256, 64)) * 0.5).astype(np.float32),
             "n": (rng.standard_normal(64) * 0.5).astype(np.float32)}
        gw.append(g["w"]); gn.append(g["n"])
        opt.step(g)
    # inputs are re-drawn from the seed by the tests, as the reference does; outputs only
    return dict(out_w=opt.st["w"]["p"], out_n=opt.st["n"]["p"], m_n=opt.st["n"]["m"], v_n=opt.st["n"]["v"],
                w16=bf16_rne_bits(opt.st["w"]["p"]).reshape(256, 64))


def sr_case():
    """tests/kernels/_probe_sr_ops.py:41-47: x = 1 + 0.4 * 2**-8 under many seeds, plus a grid of
    dither values and a random tensor at one seed."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal(4096).astype(np.float32)
    return dict(dither=sr_dither(np.arange(64)[:, None], np.arange(64)[None, :], 12345).astype(np.uint32),
                x=x, x_bits_seed7=bf16_sr_bits(x, 7),
                probe_bits=np.array([bf16_sr_bits(np.full(64, 1.0 + 0.4 * 2.0 ** -8, np.float32), s) for s in range(40)]))


def gradnorm_case():
    rng = np.random.default_rng(6)
    gs = [bf16_rne_bits((1e-3 * rng.standard_normal(n)).astype(np.float32)) for n in (8192 * 3 + 17, 64, 100000)]
    s = gradnorm_fixed(gs)
    c = control(s, 1.0, 1e-6)
    return dict(sumsq=np.float64(s), sumsq_f64=np.float64(gradnorm_f64(gs)),
                norm=np.float32(c["norm"]), clip=np.float32(c["clip_scale"]))


def muon_case():
    """One Muon step on a wide and a tall weight: momentum, 5 Polar-Express iterations in fp32 on
    the host (tolerance-level: BLAS summation order is not fixed), update."""
    rng = np.random.default_rng(7)
    out = {}
    for tag, (K, N) in (("wide", (128, 256)), ("tall", (256, 128))):
        W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
        g = rng.standard_normal((K, N)).astype(np.float32)
        buf, u = muon_momentum(np.zeros((K, N), np.float32), g, 0.95, True)
        X = u.T if K > N else u
        O = host_ns(X, PE_SCHEDULE, 5)
        O = O.T if K > N else O
        # every 8th row of the results; inputs are re-drawn from the seed by the tests
        out.update({f"{tag}_u": np.ascontiguousarray(u[::8]), f"{tag}_O": np.ascontiguousarray(O[::8]),
                    f"{tag}_Wnew": np.ascontiguousarray(muon_update(W, O, 0.02)[::8])})
    return out


def quant_case():
    rng = np.random.default_rng(8)
    w = (0.05 * rng.standard_normal((256, 128))).astype(np.float32)
    w[::9, ::7] *= 1e-4
    w[:32, :4] = 0
    wb = bf16_rne_bits(w).reshape(256, 128)
    f, s = quant_mxfp8_w(wb)
    return dict(fp8=f, scale=s)


CASES = {"adamw_seed0": adamw_case, "sr_hash": sr_case, "gradnorm": gradnorm_case, "muon_step": muon_case,
         "quant_mxfp8": quant_case}

if __name__ == "__main__":
    for name, fn in CASES.items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **fn())
        print(name, os.path.getsize(path), "bytes")
