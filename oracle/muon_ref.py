"""Muon step and the Newton-Schulz / Polar-Express iteration in numpy fp32.
Test infrastructure only."""
import numpy as np

from .bf16_ref import bf16_round

f32 = np.float32

# Keller Jordan quintic coefficients (ancora/kernels/muon_ns.py:21; ancora/optim/muon.py:70)
A_COEF, B_COEF, C_COEF = 3.4445, -4.7750, 2.0315
# Polar-Express per-iteration coefficients (ancora/kernels/muon_ns.py:30-34)
PE_SCHEDULE = [(4.0848, -6.8946, 2.9270),
               (3.9505, -6.3029, 2.6377),
               (3.7418, -5.5913, 2.3037),
               (2.8769, -3.1427, 1.2046),
               (2.8366, -3.0525, 1.2012)]


def coef_at(schedule, k):
    """(a, b, c) of iteration k: Keller when schedule is None, else schedule[k] with the last
    triple repeated past the end (ancora/kernels/muon_ns.py:37-42)."""
    if schedule is None:
        return A_COEF, B_COEF, C_COEF
    return schedule[k] if k < len(schedule) else schedule[-1]


def newton_schulz5(G, steps=5, eps=1e-7):
    """Keller quintic Newton-Schulz in fp32 (ancora/optim/muon.py:67-80): transpose when tall,
    X = X/(||X||_F + eps), then steps x {A = X X^T; B = b A + c A A; X = a X + B X}."""
    a, b, c = A_COEF, B_COEF, C_COEF
    X = np.asarray(G).astype(f32)
    transposed = X.shape[0] > X.shape[1]
    if transposed:
        X = X.T
    X = X / (np.linalg.norm(X) + eps)
    for _ in range(steps):
        A = X @ X.T
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    return X.T if transposed else X


def host_ns(X, sched, n, eps=1e-7):
    """fp32 Newton-Schulz with a per-iteration schedule
    (tests/kernels/_probe_polar_express_device.py:27-34). No transposition: the caller passes
    M <= N. sched=None means Keller for every iteration."""
    X = np.asarray(X).astype(f32)
    X = X / (np.linalg.norm(X) + eps)
    for k in range(n):
        a, b, c = coef_at(sched, k)
        A = X @ X.T
        X = a * X + (b * A + c * (A @ A)) @ X
    return X


def ns_any_shape(G, sched, n=5, eps=1e-7):
    """host_ns with the transposition rule of ancora/optim/muon.py:72-74,80 for tall inputs."""
    G = np.asarray(G).astype(f32)
    if G.shape[0] > G.shape[1]:
        return host_ns(G.T, sched, n, eps).T
    return host_ns(G, sched, n, eps)


def ortho_err(Y):
    """||Y Y^T - I||_F / sqrt(M) (tests/kernels/_probe_polar_express_device.py:37-39)."""
    M = Y.shape[0]
    return float(np.linalg.norm(Y @ Y.T - np.eye(M, dtype=Y.dtype)) / np.sqrt(M))


def ns_reference_device_model(X, sched, n=5, eps=1e-7):
    """Model of the reference's *device* numerics (its default fused chain,
    ancora/kernels/muon_ns.py:259-276): X, A, B and the new X are each stored as bf16 (RNE),
    products accumulate in fp32, X is multiplied by the reciprocal norm. Not a pass/fail
    target: it shows how far the reference's own rounding points sit from host_ns."""
    X = bf16_round(np.asarray(X).astype(f32))
    recip = f32(1.0) / (np.sqrt(np.sum(X.astype(np.float64) ** 2)).astype(f32) + f32(eps))
    X = bf16_round(X * recip)
    for k in range(n):
        a, b, c = (f32(t) for t in coef_at(sched, k))
        A = bf16_round(X @ X.T)
        B = bf16_round(b * A + c * (A @ A))
        X = bf16_round(a * X + B @ X)
    return X


def muon_momentum(buf, g, mom=0.95, nesterov=True, clip=1.0):
    """buf = mom*buf + g; u = g + mom*buf (Nesterov) or buf (ancora/optim/muon.py:303-305;
    device form ancora/kernels/muon_ns.py:183-186). `clip` (build extension) scales g first.
    Returns (buf, u), both fp32."""
    g = np.asarray(g, dtype=f32) * f32(clip)
    buf = np.asarray(buf, dtype=f32) * f32(mom)
    buf = buf + g
    u = g + f32(mom) * buf if nesterov else buf
    return buf, u


def shape_scale(K, N):
    """sqrt(max(1, rows/cols)) (ancora/optim/muon.py:308)."""
    return max(1.0, K / N) ** 0.5


def muon_update(W, O, lr, K=None, N=None):
    """W -= lr*scale*O (ancora/optim/muon.py:308-309): the product lr*scale is formed in Python
    double, then applied in fp32 (numpy's weak-scalar promotion); the device form does the same
    with lr_scale as an fp32 kernel argument (ancora/kernels/muon_ns.py:189-195)."""
    W = np.asarray(W, dtype=f32)
    K = W.shape[0] if K is None else K
    N = W.shape[1] if N is None else N
    return W - (lr * shape_scale(K, N)) * np.asarray(O, dtype=f32)


class MuonRef:
    """Host restatement of `Muon` (ancora/optim/muon.py:287-318) with an explicit schedule:
    sched=None is Keller (what the reference's host class always uses), PE_SCHEDULE is the
    Polar-Express variant of the device chain."""

    def __init__(self, params, lr=0.02, momentum=0.95, nesterov=True, ns_steps=5, sched=None):
        self.lr, self.mom, self.nesterov, self.ns, self.sched = lr, momentum, nesterov, ns_steps, sched
        self.w = {n: np.asarray(p, dtype=f32).copy() for n, p in params.items()}
        self.buf = {n: np.zeros_like(w) for n, w in self.w.items()}

    def step(self, grads, clip=1.0):
        for n, W in self.w.items():
            self.buf[n], u = muon_momentum(self.buf[n], grads[n], self.mom, self.nesterov, clip)
            o = ns_any_shape(u, self.sched, self.ns)
            self.w[n] = muon_update(W, o, self.lr)

    def weights(self):
        return {n: bf16_round(W) for n, W in self.w.items()}     # ancora/optim/muon.py:311-312

    def master(self):
        return {n: W.copy() for n, W in self.w.items()}


def default_is_muon(name, p):
    """Routing predicate (ancora/optim/hybrid.py:18-25): 2-D and the lower-cased name contains
    none of norm, ln, embed, lm_head, head, wte, wpe."""
    if p.ndim != 2:
        return False
    low = name.lower()
    return not any(t in low for t in ("norm", "ln", "embed", "lm_head", "head", "wte", "wpe"))
