"""Numpy model of the library's bf16 Newton-Schulz chain. Test infrastructure only.

`oracle/muon_ref.py:host_ns` restates the reference's fp32 host chain (ancora/optim/muon.py:67-80,
tests/kernels/_probe_polar_express_device.py:27-34): that is the parity target. This file models
something else: the arithmetic of the HIP chain itself (csrc/ns.hip, csrc/ns_gemm_big.hip) -- where
it rounds to bf16, which products carry residual terms, which statistic sends a matrix through
which gate -- so that the plan and its thresholds can be examined on the CPU: how far the chain's
rounding points put a given input from `host_ns`, and on which side of a threshold an input falls.
It is not bit-exact to the GPU (numpy's BLAS accumulates a product in another order than the
matrix cores): errors against `host_ns` agree to about two digits, decisions exactly unless an input
sits on a threshold. `tests/test_gpu_ns_model.py` pins it to the GPU on both counts.

Rounding points modelled (same as the kernels):
  iterate carried as a bf16 pair x = Xh + Xl, Xh = bf16(x), Xl = bf16(x - Xh);
  A = X X^T accumulated in fp32 from bf16 operands: Xh Xh^T, plus Xh Xl^T + Xl Xh^T where the plan
    or a gate says so; diag(A) kept in fp32 (dA), off-diagonal part F rounded to Fh = bf16(F)
    (and Fl = bf16(F - Fh) where needed);
  B = b A + c A A with A A = dA^2 + dA F + F dA + F F: only F F from bf16 operands (Fh Fh, plus
    Fh Fl + Fl Fh where needed); the entries of A in the fp32 terms are the fp32 F where the chain
    keeps the fp32 copy of A and Fh where it does not; diag(B) in fp32 (dB), Boff -> Bh (, Bl);
  X' = (a + dB) (.) x + Boff X from bf16 operands: Bh Xh (+ Bh Xl) (+ Bl Xh);
  where the plan says so (N >= 2M) and no product of the next iteration multiplies it, the low half
    Xl is kept as 8 bits relative to the ulp of Xh instead of a bf16.
"""
import numpy as np

from .bf16_ref import bf16_round

f32 = np.float32

TAU_HARD, TAU_PLAIN = 2.5, 1.3
TAU_WIDE_LO, TAU_WIDE_HI, TAU_WIDE_NEAR = 2.5, 40.0, 1.5
COLC_FRAC, BULK_SHARE = 0.85, 3e-3
TAU_WIDE_NEAR_2M, NEAR_DIFF_2M = 1.15, 0.15
COL_BLOCK, COL_ROW_STEP = 64, 4


class Plan:
    """`split_plan` of csrc/ns.hip for (M, N, mode, steps); mode in bf16, bf16_fast, bf16_x3, bf16_late3."""

    def __init__(self, M, N, mode="bf16", steps=5):
        self.x_from = self.fb_from = steps
        self.gate_tau = {}
        self.gate_bx = set()
        self.gate_hi = {}            # upper bounds of the A = X X^T gates (absent: none)
        self.gate_bx_hi = None       # upper bound of the X = a X + B X gates
        self.wide = False
        self.wide_near = TAU_WIDE_LO
        self.wide_near_diff = 0.0    # > 0: the near range flags on proxy - colc > this instead of the ratio rule
        self.wide_from = 1
        self.drop_a32 = False
        self.low8 = False            # low halves of the iterate as 8 bits where no product multiplies them
        if mode == "bf16_x3":
            self.x_from = self.fb_from = 0
            return
        if mode == "bf16_late3" and M >= 1024:
            self.x_from = self.fb_from = 2 if steps >= 5 else (steps - 3 if steps > 3 else 0)
            if steps >= 5:
                self.fb_from = self.x_from + 1
            if self.x_from > 1:
                self.wide, self.wide_near = True, (TAU_WIDE_NEAR if N < 2 * M else TAU_WIDE_LO)
            return
        if mode not in ("bf16", "bf16_late3"):
            return
        if M >= 1024:
            self.drop_a32 = mode == "bf16" and N >= 2 * M
            self.low8 = self.drop_a32
            if steps >= 2:
                self.wide, self.wide_near = True, (TAU_WIDE_NEAR if N < 2 * M else TAU_WIDE_LO)
                if mode == "bf16" and N >= 2 * M:
                    self.wide_near, self.wide_near_diff = TAU_WIDE_NEAR_2M, NEAR_DIFF_2M
            if N < 2 * M:
                self.x_from = min(steps - 2, 3)
                self.gate_tau = {1: TAU_HARD, 2: TAU_HARD}
                if steps == 5:
                    self.gate_tau = {1: TAU_HARD, 2: TAU_PLAIN, 3: TAU_PLAIN}
                    self.gate_bx = {2, 3}
                    self.x_from = 4
            else:
                self.gate_tau = {2: TAU_HARD}
                if steps < 5:
                    self.gate_tau[1] = TAU_HARD
        else:
            start = 0 if M < 256 else 1
            self.x_from = self.fb_from = min(steps - 3, start)
        self.x_from, self.fb_from = max(self.x_from, 0), max(self.fb_from, 0)


def statistics(Xh, Fh0):
    """(proxy, colc, bulk) as the kernels compute them: the proxy N * ||Fh||_F^2 from the first
    iteration's bf16 off-diagonal A (k_ns_cond), the column concentration and the share of the mass
    in the lightest block of 64 columns from every fourth row of the input's high half
    (k_ns_colstat, k_ns_classify)."""
    M, N = Xh.shape
    proxy = float(N) * float(np.sum(Fh0.astype(np.float64) ** 2))
    c2 = np.sum(Xh[::COL_ROW_STEP].astype(np.float64) ** 2, axis=0)
    parts = (N + COL_BLOCK - 1) // COL_BLOCK
    pad = np.zeros(parts * COL_BLOCK)
    pad[:N] = c2
    blocks = pad.reshape(parts, COL_BLOCK).sum(axis=1)
    s2, s4 = float(c2.sum()), float(np.sum(c2 * c2))
    colc = N * s4 / (s2 * s2) if s2 > 0 else 1.0
    bulk = parts * float(blocks.min()) / s2 if s2 > 0 else 1.0
    return proxy, colc, bulk


def wide_flag(plan, proxy, colc, bulk):
    """k_ns_classify's decision."""
    if not plan.wide:
        return False
    if TAU_WIDE_LO < proxy < TAU_WIDE_HI:
        return True
    if proxy >= TAU_WIDE_HI:
        return colc < COLC_FRAC * proxy or bulk < BULK_SHARE
    if plan.wide_near < proxy <= TAU_WIDE_LO:
        if plan.wide_near_diff > 0:
            return proxy - colc > plan.wide_near_diff
        return colc < COLC_FRAC * proxy
    return False


def low8(y, Xh):
    """anc_low8_encode / _decode (csrc/ns_common.h): the low half of y next to Xh = bf16(y) as 8 bits
    in the integer space of the fp32 bit patterns: d = bits(y) - bits(Xh) in -0x8000 .. 0x8000,
    q = min(d + 0x80, 0x7FFF) >> 8, read back as the float with bits(Xh) + (q << 8) (y to 24 bits).
    Returns that float minus Xh (exact in fp32)."""
    yb, hb = np.ascontiguousarray(y, dtype=f32).view(np.uint32), np.ascontiguousarray(Xh, dtype=f32).view(np.uint32)
    d = (yb - hb).astype(np.int32) + np.int32(0x80)
    q = np.minimum(d, np.int32(0x7FFF)) >> 8
    x = (hb + (q.astype(np.uint32) << np.uint32(8))).view(f32)
    return (x - Xh).astype(f32)


def chain(X, sched, steps=5, mode="bf16", eps=1e-7, info=None, overrides=None):
    """The chain's result for one (M, N) fp32 matrix, M <= N, through the fp32-input entry
    (normalise, then the pair). `info`, if a dict, receives the statistics and decisions.
    `overrides`: {"wide": bool} forces the wide gate's decision (to look at both sides of it);
    {"gram3": iterations, "bx_l": iterations, "f3": iterations} add the residual of X to A = X X^T,
    the residual of X to X = a X + B X, the residuals of F and Boff to their products in those
    iterations on top of the plan (to price a candidate gate)."""
    from .muon_ref import coef_at
    X = np.asarray(X, dtype=f32)
    M, N = X.shape
    plan = Plan(M, N, mode, steps)
    rc = f32(1.0) / (f32(np.sqrt(np.sum(X.astype(np.float64) ** 2))) + f32(eps))
    x = X * rc
    Xh = bf16_round(x)
    Xl = bf16_round(x - Xh)
    idx = np.arange(M)
    proxy = colc = bulk = None
    flagged = False
    for k in range(steps):
        a, b, c = (f32(t) for t in coef_at(sched, k))
        split, split_fb = k >= plan.x_from, k >= plan.fb_from
        over = (not split) and k in plan.gate_tau and proxy is not None and proxy > plan.gate_tau[k]
        gated = over and (k not in plan.gate_hi or proxy <= plan.gate_hi[k])
        gated_bx = over and k in plan.gate_bx and (plan.gate_bx_hi is None or proxy <= plan.gate_bx_hi)
        wide_k = flagged and k >= plan.wide_from
        ov = overrides or {}
        gram3 = split or gated or (wide_k and (k < plan.x_from or k < plan.fb_from)) or k in ov.get("gram3", ())
        f3 = split_fb or (wide_k and k < plan.fb_from) or k in ov.get("f3", ())
        G = Xh @ Xh.T
        if gram3:
            P = Xh @ Xl.T
            G = G + P + P.T
        d = G[idx, idx].copy()
        F = G.copy()
        F[idx, idx] = 0
        Fh = bf16_round(F)
        if k == 0:
            proxy, colc, bulk = statistics(Xh, Fh)
            flagged = wide_flag(plan, proxy, colc, bulk)
            if overrides and "wide" in overrides:
                flagged = bool(overrides["wide"]) and plan.wide
        FF = Fh @ Fh
        if f3:
            Fl = bf16_round(F - Fh)
            P = Fh @ Fl
            FF = FF + P + P.T
        has_a32 = (not plan.drop_a32) or (k > 0 and flagged)
        Au = F if has_a32 else Fh
        a2 = FF + (d[:, None] * Au + Au * d[None, :])
        Boff = b * Au + c * a2
        Boff[idx, idx] = 0
        dB = b * d + c * (FF[idx, idx] + d * d)
        Bh = bf16_round(Boff)
        Y = Bh @ Xh
        bx_l = (split or (gated_bx and not split_fb) or (wide_k and k < plan.fb_from)
                or k in ov.get("bx_l", ()))
        if bx_l:
            Y = Y + Bh @ Xl
        if f3:
            Y = Y + bf16_round(Boff - Bh) @ Xh
        y = (a + dB)[:, None] * (Xh + Xl) + Y
        Xh = bf16_round(y)
        # 8-bit low half where no product of the next iteration multiplies it
        nk = k + 1
        if (plan.low8 and nk < steps and plan.gate_tau and not flagged and nk < plan.x_from
                and not (nk in plan.gate_tau and proxy > plan.gate_tau[nk])
                and not any(nk in ov.get(key, ()) for key in ("gram3", "bx_l"))):
            Xl = low8(y, Xh)
        else:
            Xl = bf16_round(y - Xh)
    if info is not None:
        info.update(proxy=proxy, colc=colc, bulk=bulk, wide=flagged, plan=plan)
    return y


def chain_any_shape(G, sched, steps=5, mode="bf16", **kw):
    """`chain` with the reference's transposition rule for tall matrices (ancora/optim/muon.py:72-74)."""
    G = np.asarray(G, dtype=f32)
    if G.shape[0] > G.shape[1]:
        return chain(np.ascontiguousarray(G.T), sched, steps, mode, **kw).T
    return chain(G, sched, steps, mode, **kw)
