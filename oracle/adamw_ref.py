"""AdamW step in numpy fp32. Test infrastructure only."""
import numpy as np

f32 = np.float32


def adamw_step_div(p, m, v, g, lr, b1, b2, eps, wd, t, clip=1.0):
    """One step in the form of the reference's numpy test oracle
    (tests/optim/test_adamw.py:37-41): fp32 arrays, Python-double scalars (numpy rounds each
    to fp32 once):
        m = b1*m + (1-b1)*g;  v = b2*v + (1-b2)*g*g
        mh = m/(1-b1**t);     vh = v/(1-b2**t)
        p = p - lr*(mh/(sqrt(vh)+eps) + wd*p)
    `clip` (build extension) multiplies g first; clip == 1 leaves g bit-identical.
    Returns (p, m, v)."""
    p, m, v = (np.asarray(a, dtype=f32) for a in (p, m, v))
    g = np.asarray(g, dtype=f32) * f32(clip)
    m = b1 * m + (1 - b1) * g
    v = b2 * v + (1 - b2) * g * g
    mh = m / (1 - b1 ** t)
    vh = v / (1 - b2 ** t)
    p = p - lr * (mh / (np.sqrt(vh) + eps) + wd * p)
    assert p.dtype == f32 and m.dtype == f32 and v.dtype == f32
    return p, m, v


def adamw_step_ibc(p, m, v, g, lr, b1, b2, eps, wd, ibc1, ibc2, clip=1.0):
    """One step in the form of the reference kernel (ancora/optim/adamw.py:34-37): every
    scalar is an fp32 kernel argument, (1.0 - beta) is formed in fp32 inside the kernel,
    and the bias corrections arrive as reciprocals ibc = 1/(1-beta**t) (adamw.py:90-91):
        mn = b1*m + (1-b1)*g;  vn = b2*v + (1-b2)*g*g
        upd = (mn*ibc1)/(sqrt(vn*ibc2)+eps) + wd*p;  pn = p - lr*upd"""
    p, m, v = (np.asarray(a, dtype=f32) for a in (p, m, v))
    g = np.asarray(g, dtype=f32) * f32(clip)
    b1, b2, eps, lr, wd, ibc1, ibc2 = (f32(s) for s in (b1, b2, eps, lr, wd, ibc1, ibc2))
    o1, o2 = f32(1.0) - b1, f32(1.0) - b2
    m = b1 * m + o1 * g
    v = b2 * v + o2 * g * g
    upd = (m * ibc1) / (np.sqrt(v * ibc2) + eps) + wd * p
    p = p - lr * upd
    assert p.dtype == f32
    return p, m, v


class AdamWRef:
    """Host restatement of the `AdamW` class bookkeeping (ancora/optim/adamw.py:69-109):
    per-name state, `t` incremented before the bias correction (:89-91), wd = 0 for no_decay
    names (:80), bf16 weights = RNE(master) (:41, 100-102)."""

    def __init__(self, params, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.01, no_decay=(),
                 form="div"):
        self.lr, (self.b1, self.b2), self.eps, self.wd, self.form = lr, betas, eps, wd, form
        self.t = 0
        self.st = {n: dict(p=np.asarray(p, dtype=f32).copy(), m=np.zeros(p.shape, f32),
                           v=np.zeros(p.shape, f32), wd=0.0 if n in no_decay else wd)
                   for n, p in params.items()}

    def step(self, grads, clip=1.0):
        self.t += 1
        for n, s in self.st.items():
            g = np.asarray(grads[n], dtype=f32)
            if self.form == "div":
                s["p"], s["m"], s["v"] = adamw_step_div(s["p"], s["m"], s["v"], g, self.lr, self.b1,
                                                        self.b2, self.eps, s["wd"], self.t, clip)
            else:
                ibc1 = 1.0 / (1.0 - self.b1 ** self.t)
                ibc2 = 1.0 / (1.0 - self.b2 ** self.t)
                s["p"], s["m"], s["v"] = adamw_step_ibc(s["p"], s["m"], s["v"], g, self.lr, self.b1,
                                                        self.b2, self.eps, s["wd"], ibc1, ibc2, clip)

    def master(self):
        return {n: s["p"].copy() for n, s in self.st.items()}
