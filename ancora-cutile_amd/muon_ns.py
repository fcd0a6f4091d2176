"""Resident Newton-Schulz / Polar-Express drivers on the MI355X.

Mirror of ancora/kernels/muon_ns.py: `newton_schulz_resident`, `newton_schulz_resident_e`,
`PE_SCHEDULE`, the Keller coefficients, the process-wide `set_polar_express` toggle with
its `_KELLER` sentinel, and the tile constants `NTM, NTN, NTK`. The 25 cuda-tile kernels
and the 28-launch chain behind those drivers are replaced by one C entry point,
`anc_ns_batched`, which runs the whole chain for a batch of same-shape matrices.

The library carries the iterate in fp32 (operands are rounded to bf16 only at the
matrix-core input), so its native driver `ns_batched` takes and returns fp32. The two
reference-shaped drivers keep the reference's bf16 in / bf16 out contract on `gX`: they
widen into a workspace, run the chain and round the result back (RNE). Their scratch
arguments (gA, gA2, gB, gBX, grecip) are accepted for call compatibility and not touched.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import api, NS_BF16, NS_FP32, NS_BF16_FAST, NS_BF16_X3, NS_BF16_LATE3
from .devbuf import DevBuf

NTM, NTN, NTK = 128, 128, 64                       # ancora/kernels/muon_ns.py:20
A_COEF, B_COEF, C_COEF = 3.4445, -4.7750, 2.0315   # ancora/kernels/muon_ns.py:21

# Polar-Express per-iteration coefficients (ancora/kernels/muon_ns.py:30-34)
PE_SCHEDULE = [(4.0848, -6.8946, 2.9270),
               (3.9505, -6.3029, 2.6377),
               (3.7418, -5.5913, 2.3037),
               (2.8769, -3.1427, 1.2046),
               (2.8366, -3.0525, 1.2012)]

MODES = {"bf16": NS_BF16, "bf16_fast": NS_BF16_FAST, "bf16_x3": NS_BF16_X3, "fp32": NS_FP32,
         "bf16_late3": NS_BF16_LATE3,
         # the gated plan whatever the schedule ("bf16" turns into "bf16_late3" under Keller's
         # coefficients, see effective_mode)
         "bf16_gated": NS_BF16,
         # same arithmetic forced onto the 128x128-tile kernel (ANC_NS_TILE128), for tests
         "bf16_tile128": NS_BF16 | 0x100, "bf16_fast_tile128": NS_BF16_FAST | 0x100,
         "bf16_late3_tile128": NS_BF16_LATE3 | 0x100}


def _coef_at(schedule, k):
    """(a,b,c) of iteration k: Keller if schedule is None, else schedule[k] with the last triple
    repeated once the schedule is exhausted (ancora/kernels/muon_ns.py:37-42)."""
    if schedule is None:
        return A_COEF, B_COEF, C_COEF
    return schedule[k] if k < len(schedule) else schedule[-1]


# Process-wide default: None = Keller (ancora/kernels/muon_ns.py:44-65). `schedule=None` passed
# explicitly still means Keller; the sentinel means "caller said nothing, use the default".
_KELLER = object()
_DEFAULT_SCHEDULE = None


def set_polar_express(on: bool):
    """Select Polar Express (on) or Keller (off) for every NS call that does not pass an explicit
    schedule. Returns the previous setting."""
    global _DEFAULT_SCHEDULE
    prev = _DEFAULT_SCHEDULE
    _DEFAULT_SCHEDULE = PE_SCHEDULE if on else None
    return prev


def _resolve(schedule):
    return _DEFAULT_SCHEDULE if schedule is _KELLER else schedule


def is_keller(schedule):
    """True for a resolved schedule that applies Keller's triple in every iteration."""
    return schedule is None or all(tuple(t) == (A_COEF, B_COEF, C_COEF) for t in schedule)


def effective_mode(mode, schedule):
    """The mode a chain call runs in. Keller's quintic does not drive the singular values to 1
    (they end in 0.7 .. 1.2), so the off-diagonal of A = X X^T never becomes small and the bf16
    rounding of every operand stays a first-order error up to the last iteration: the gated plan
    of "bf16", tuned on Polar Express, reaches 3e-3 .. 5e-3 there. Under Keller "bf16" therefore
    runs as "bf16_late3" (the residual of X from iteration 2 on, those of F and Boff from
    iteration 3 on: 2.05 times the matrix-core work, 9e-4 at worst); "bf16_gated" keeps the gated plan. `schedule` is
    the resolved one (None = Keller)."""
    if mode == "bf16" and is_keller(schedule):
        return "bf16_late3"
    return mode


def coef_array(schedule, steps):
    flat = []
    for k in range(steps):
        flat.extend(_coef_at(schedule, k))
    return (ctypes.c_float * max(1, len(flat)))(*flat)


class NsWorkspace:
    """Device scratch of the chain; grows on demand, never shrinks. The chain keeps nothing in it
    between calls, so one workspace serves every group that runs sequentially on a stream
    (the role of MuonScratch / ExpertMuonScratch, ancora/optim/muon.py:138-159)."""

    def __init__(self):
        self.buf = None

    def ensure(self, nbytes):
        if self.buf is None or self.buf.nbytes < nbytes:
            if self.buf is not None:
                _lib.api.anc_device_sync()
                self.buf.free()
            self.buf = DevBuf.empty((int(nbytes),), np.uint8)
        return self.buf

    def nbytes(self):
        return 0 if self.buf is None else self.buf.nbytes

    def free(self):
        if self.buf is not None:
            self.buf.free()
            self.buf = None


_SHARED_WS = NsWorkspace()


def ns_workspace_bytes(E, M, N, mode="bf16"):
    _lib.load()
    n = api.anc_ns_workspace_bytes(E, M, N, MODES[mode])
    if n < 0:
        raise _lib.AncoraError(_lib._lib.anc_last_error().decode())
    return int(n)


def _acct_mode(mode, schedule):
    """Mode of the accounting helpers: `schedule` is the schedule the chain ran under (resolved as
    the drivers resolve it), so that mode="bf16" counts the plan it really ran; the default sentinel
    leaves `mode` as given (pass "bf16_late3" etc. yourself)."""
    return mode if schedule is _ASIS else effective_mode(mode, _resolve(schedule))


_ASIS = object()


def ns_flops(E, M, N, steps=5, mode="bf16", schedule=_ASIS):
    """(executed, dense) matrix-core FLOPs of one chain call over E (M,N) matrices."""
    _lib.load()
    ex, de = ctypes.c_double(0), ctypes.c_double(0)
    api.anc_ns_flops(E, M, N, int(steps), MODES[_acct_mode(mode, schedule)], ctypes.byref(ex), ctypes.byref(de))
    return ex.value, de.value


def ns_hard_info(workspace_ptr, E, M, N, steps=5, mode="bf16", si=0, schedule=_ASIS):
    """(n_gated, extra_flops) of the last chain call that used this workspace: how many of its E
    matrices took extra terms through a conditioning gate, and the matrix-core work they add,
    all together, to `ns_flops`' executed count. Synchronises stream `si`. `mode` (with `schedule`)
    must name the mode that call ran in: the workspace layout depends on it."""
    n, ex = ctypes.c_int32(0), ctypes.c_double(0)
    api.anc_ns_hard_info(int(workspace_ptr), int(E), int(M), int(N), MODES[_acct_mode(mode, schedule)], int(steps),
                         ctypes.byref(n), ctypes.byref(ex), int(si))
    return n.value, ex.value


def ns_product_flops(E, M, N, k, product, steps=5, mode="bf16", schedule=_ASIS):
    """Executed matrix-core FLOPs of product 0 (A = X X^T), 1 (B = b A + c A A) or 2
    (X = a X + B X) of iteration k of a chain call."""
    ex = ctypes.c_double(0)
    api.anc_ns_product_flops(int(E), int(M), int(N), int(steps), MODES[_acct_mode(mode, schedule)], int(k),
                             int(product), ctypes.byref(ex))
    return ex.value


def ns_batched(X32, E, M, N, si, steps=5, eps=1e-7, schedule=_KELLER, mode="bf16", workspace=None):
    """Native driver: X32 is a DevBuf of E packed (M,N) fp32 matrices, M <= N, both multiples of
    128; overwritten with the orthogonalised result."""
    schedule = _resolve(schedule)
    if X32.dtype != np.float32 or X32.size < E * M * N:
        raise ValueError(f"ns_batched: X32 must hold {E}x{M}x{N} float32, has {X32.size} {X32.dtype}")
    mode = effective_mode(mode, schedule)
    ws = _SHARED_WS if workspace is None else workspace
    need = ns_workspace_bytes(E, M, N, mode)
    buf = ws.ensure(need)
    coef = coef_array(schedule, steps)
    api.anc_ns_batched(X32.ptr, E, M, N, int(steps), coef, float(eps), MODES[mode], buf.ptr,
                       buf.nbytes, int(si))


ns_fp32_batched = ns_batched


def ns_batched_pair(U, fro_partials, n_partials, E, M, N, si, steps=5, eps=1e-7, schedule=_KELLER,
                    mode="bf16", workspace=None):
    """The chain on what `anc_muon_momentum_multi_pair` leaves in the packed buffer U (an
    E*M*N fp32-sized DevBuf holding the bf16 pair of the unnormalised input: hi in its first
    half, lo in its second) and the per-block sums of squares in `fro_partials`; U is
    overwritten with the fp32 result. No norm pass, no scaling pass."""
    schedule = _resolve(schedule)
    if U.dtype != np.float32 or U.size < E * M * N:
        raise ValueError(f"ns_batched_pair: U must hold {E}x{M}x{N} float32, has {U.size} {U.dtype}")
    if mode == "fp32" or steps < 2:
        raise ValueError("ns_batched_pair: bf16 modes and steps >= 2 only")
    mode = effective_mode(mode, schedule)
    ws = _SHARED_WS if workspace is None else workspace
    buf = ws.ensure(ns_workspace_bytes(E, M, N, mode))
    coef = coef_array(schedule, steps)
    api.anc_ns_batched_pair(U.ptr, U.ptr + E * M * N * 2, fro_partials.ptr, int(n_partials), U.ptr,
                            E, M, N, int(steps), coef, float(eps), MODES[mode], buf.ptr, buf.nbytes,
                            int(si))


def _run_bf16(gX, E, M, N, si, steps, eps, schedule, mode, workspace):
    if gX.dtype != np.uint16 or gX.size < E * M * N:
        raise ValueError("newton_schulz_resident: gX must hold the packed bf16 (uint16) batch")
    if M % NTM or N % NTN or M > N:
        raise ValueError(f"newton_schulz_resident: (M,N)=({M},{N}) must be 128-aligned with M <= N")
    mode = effective_mode(mode, schedule)
    ws = _SHARED_WS if workspace is None else workspace
    n = E * M * N
    need = ns_workspace_bytes(E, M, N, mode)
    xbytes = (n * 4 + 255) // 256 * 256
    buf = ws.ensure(need + xbytes)
    x32 = DevBuf(shape=(E * M, N), dtype=np.float32, ptr=buf.ptr)
    api.anc_bf16_to_f32(gX.ptr, x32.ptr, n, int(si))
    coef = coef_array(schedule, steps)
    api.anc_ns_batched(x32.ptr, E, M, N, int(steps), coef, float(eps), MODES[mode],
                       buf.ptr + xbytes, buf.nbytes - xbytes, int(si))
    api.anc_f32_to_bf16(x32.ptr, gX.ptr, n, int(si))


def newton_schulz_resident(gX, gA, gA2, gB, gBX, grecip, M, N, si, steps=5, eps=1e-7,
                           schedule=_KELLER, fused=True, mode="bf16", workspace=None):
    """Resident NS on one (M,N) bf16 matrix, overwritten in place
    (ancora/kernels/muon_ns.py:245-283). `fused` selected between two launch chains of the
    reference with slightly different rounding; here there is one chain and the flag is ignored."""
    _run_bf16(gX, 1, M, N, si, steps, eps, _resolve(schedule), mode, workspace)


def newton_schulz_resident_e(gX, gA, gA2, gB, gBX, grecip, E, M, N, si, steps=5, eps=1e-7,
                             schedule=_KELLER, fused=True, mode="bf16", workspace=None):
    """Batched resident NS over E (M,N) bf16 matrices packed (E*M, N)
    (ancora/kernels/muon_ns.py:430-468). Each matrix's result is independent of E."""
    _run_bf16(gX, E, M, N, si, steps, eps, _resolve(schedule), mode, workspace)
