"""The numpy model of the bf16 Newton-Schulz chain (oracle/ns_chain_model.py) on the CPU: its plan
mirrors the library's, and every threshold of the gates is walked from both sides with an input
family whose knob moves a matrix across it: the chain's rounding points must stay inside the 2e-3
bar on either side, so that a threshold edit that opens a hole fails here, before it costs a GPU
minute. (tests/test_gpu_ns_model.py pins the model itself to the GPU.)"""
import ctypes

import numpy as np
import pytest

from oracle import ns_inputs as I
from oracle.bf16_ref import bf16_round
from oracle.muon_ref import PE_SCHEDULE, host_ns
from oracle.ns_chain_model import (Plan, chain, statistics, TAU_PLAIN, TAU_HARD, TAU_WIDE_NEAR, TAU_WIDE_HI, COLC_FRAC,
                                   BULK_SHARE, NEAR_DIFF_2M)

BAR = 2e-3


def rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b) / np.linalg.norm(b))


def run(X):
    info = {}
    y = chain(X, PE_SCHEDULE, 5, "bf16", info=info)
    return rel(y, host_ns(X, PE_SCHEDULE, 5)), info


def stats(X):
    x = (X / np.linalg.norm(X)).astype(np.float32)
    Xh = bf16_round(x)
    G = Xh @ Xh.T
    np.fill_diagonal(G, 0)
    return statistics(Xh, bf16_round(G))


def test_plan_mirrors_the_library():
    """The executed matrix-core work the library reports for a chain (anc_ns_flops: host code, no
    GPU needed) equals what the model's plan multiplies, over shapes, modes and chain lengths."""
    from ancora_cutile_amd import _lib
    _lib.load()
    modes = {"bf16": _lib.NS_BF16, "bf16_fast": _lib.NS_BF16_FAST, "bf16_x3": _lib.NS_BF16_X3, "bf16_late3": _lib.NS_BF16_LATE3}
    for (M, N) in ((128, 128), (256, 512), (512, 1536), (1024, 1024), (1024, 1536), (1024, 2048), (1024, 3072), (2048, 4096)):
        for mode, code in modes.items():
            for steps in (2, 3, 4, 5, 6, 8):
                ex, de = ctypes.c_double(0), ctypes.c_double(0)
                _lib.api.anc_ns_flops(1, M, N, steps, code, ctypes.byref(ex), ctypes.byref(de))
                p = Plan(M, N, mode, steps)
                ts = 256.0 if M % 256 == 0 and N % 256 == 0 else 128.0
                t = M / ts
                sym = t * (t + 1) / 2 * 2.0 * ts * ts
                want = 0.0
                for k in range(steps):
                    sx, sfb = k >= p.x_from, k >= p.fb_from
                    want += sym * (3 if sx else 1) * N + sym * (3 if sfb else 1) * M + 2.0 * M * N * M * (1 + sx + sfb)
                assert ex.value == want, (M, N, mode, steps, p.x_from, p.fb_from)


def test_low_half_as_eight_bits():
    """The 8-bit low half of the iterate (csrc/ns_common.h anc_low8_encode / _decode, restated in
    the model): high half + low half reproduce the value to 24 bits (2^-16 relative, 2^-15 where the
    cap at 127 bites), without bias, exactly where the value has 16 significant bits, across binade
    borders in both directions and for zeros; what comes back is exactly representable next to the
    high half (the chain adds the two in fp32)."""
    from oracle.ns_chain_model import low8
    rng = np.random.default_rng(1)
    y = (rng.standard_normal(1 << 20) * np.exp(rng.uniform(-30, 10, 1 << 20))).astype(np.float32)
    special = np.array([0.0, -0.0, 1.0, -1.0, 2.0 - 2.0 ** -17, -(2.0 - 2.0 ** -17), 1.0 + 2.0 ** -9, 1.0 + 2.0 ** -8 + 2.0 ** -16,
                        3.0 * 2.0 ** -100, 1.0078125 - 2.0 ** -23], np.float32)
    y[:special.size] = special
    h = bf16_round(y)
    lo = low8(y, h)
    x = (h + lo).astype(np.float32)
    assert np.array_equal((x - h).astype(np.float32), lo)                   # exact next to the high half
    err = (x.astype(np.float64) - y) / np.where(y == 0, 1.0, y)
    assert np.abs(err).max() <= 2.0 ** -15 and np.percentile(np.abs(err), 99) <= 2.0 ** -16
    assert abs(err.mean()) < 1e-7                                           # rounded, not truncated
    nz = y != 0                                                             # (h + lo loses the sign of -0)
    q = (x.view(np.uint32).astype(np.int64) - h.view(np.uint32).astype(np.int64))[nz] / 256
    assert np.array_equal(q, np.rint(q)) and q.min() >= -128 and q.max() <= 127   # a whole byte
    # values that sit k / 256 of a bf16 step next to a bf16 number, |k| <= 127, come back exactly
    k = rng.integers(-127, 128, y.size).astype(np.int64)
    hb = h.view(np.uint32).astype(np.int64)
    ok = (hb & 0x7F800000 > 0x10000000) & (hb & 0x7F800000 < 0x7F000000)
    exact = ((hb + (k << 8)) & 0xFFFFFFFF).astype(np.uint32).view(np.float32)[ok]
    he = bf16_round(exact)
    assert np.array_equal(he, h[ok]) and np.array_equal((he + low8(exact, he)).astype(np.float32), exact)
    assert x[0] == 0 and x[2] == 1 and x[3] == -1


@pytest.mark.parametrize("M,N", [(1024, 1024)])
def test_low_gate_from_both_sides(M, N):
    """Scaled columns just below and just above the low gate (proxy 1.3, N < 2M)."""
    for target in (TAU_PLAIN - 0.05, TAU_PLAIN + 0.05):
        s = I.solve_knob(lambda v: I.scaled_columns(M, N, v), target, 0.0, 1.0)
        err, info = run(I.scaled_columns(M, N, s))
        assert abs(info["proxy"] - target) < 0.01 and not info["wide"]
        assert err < BAR, (target, err)


@pytest.mark.parametrize("M,N", [(1024, 1024), (1024, 1536)])
def test_near_range_from_both_sides(M, N):
    """A gap in the spectrum with flat column norms (a fraction of near-duplicate rows) just below
    and just above the start of the wide gate's near range; scaled columns with the same proxy
    (column norms explain it) stay with the low gate on both sides."""
    for target, wide in ((TAU_WIDE_NEAR - 0.05, False), (TAU_WIDE_NEAR + 0.05, True), (2.3, True)):
        f = I.solve_knob(lambda v: I.duplicated_rows(M, N, v), target, 0.0, 1.0)
        err, info = run(I.duplicated_rows(M, N, f))
        assert info["wide"] == wide and info["colc"] < COLC_FRAC * info["proxy"]
        assert err < BAR, ("duplicated rows", target, err)
        s = I.solve_knob(lambda v: I.scaled_columns(M, N, v), target, 0.0, 1.5)
        err, info = run(I.scaled_columns(M, N, s))
        assert not info["wide"] and info["colc"] > COLC_FRAC * info["proxy"]
        assert err < BAR, ("scaled columns", target, err)


@pytest.mark.parametrize("M,N", [(1024, 2048), (1024, 3072)])
def test_near_range_of_wide_shapes_from_both_sides(M, N):
    """N >= 2M has no residual term in its plan and no low gate: a gap in the spectrum with flat
    column norms (a fraction of near-duplicate rows) would leave the bar from proxy 1.25 on. Its near
    range takes a matrix whose proxy exceeds its column concentration by more than NEAR_DIFF_2M:
    either side of that, the same with the columns scaled on top (the part of the proxy the columns
    explain does not count: a ratio rule would miss the scaled case), and the top of the range."""
    for sigma in (0.0, 0.4):
        for target, wide in ((NEAR_DIFF_2M - 0.03, False), (NEAR_DIFF_2M + 0.03, True), (0.3, True)):
            f = I.solve_knob(lambda v: I.gap_scaled_columns(M, N, v, sigma), target, 0.0, 0.5, stat=I.unexplained_proxy)
            err, info = run(I.gap_scaled_columns(M, N, f, sigma))
            assert info["wide"] == wide, (sigma, target, info["proxy"], info["colc"])
            assert err < (BAR if not wide else 1e-4), (sigma, target, err)
    f = I.solve_knob(lambda v: I.duplicated_rows(M, N, v), 2.3, 0.0, 1.0)
    err, info = run(I.duplicated_rows(M, N, f))
    assert info["wide"] and err < 1e-4
    # what the plan alone would leave there (the price list of the gate)
    X = I.duplicated_rows(M, N, f)
    assert rel(chain(X, PE_SCHEDULE, 5, "bf16", overrides={"wide": False}), host_ns(X, PE_SCHEDULE, 5)) > 3e-3
    # scaled columns with a proxy inside the range: the columns explain it, no gate, inside the bar
    s = I.solve_knob(lambda v: I.scaled_columns(M, N, v), 2.0, 0.0, 1.0)
    err, info = run(I.scaled_columns(M, N, s))
    assert not info["wide"] and abs(info["proxy"] - info["colc"]) < 0.05 and err < BAR


@pytest.mark.parametrize("M,N", [(1024, 1024), (1024, 3072)])
def test_band_edges_from_both_sides(M, N):
    """The wide gate's band: a log-uniform spectrum at proxy 2.4 / 2.6 (its lower edge, which is also
    the outlier-column gate's threshold), outlier columns at proxy 38 / 42 (its upper edge, where
    the column statistic takes over and finds columns: cheap gates)."""
    for target in (TAU_HARD - 0.1, TAU_HARD + 0.1):
        d = I.solve_knob(lambda v: I.log_spectrum(M, N, v), target, 0.0, 3.0)
        err, info = run(I.log_spectrum(M, N, d))
        near = info["colc"] < COLC_FRAC * info["proxy"] if N < 2 * M else info["proxy"] - info["colc"] > NEAR_DIFF_2M
        assert info["wide"] == (target > TAU_HARD or near)
        assert err < BAR, ("log spectrum", target, err)
    r = N // 50
    for target, wide in ((TAU_WIDE_HI - 2, True), (TAU_WIDE_HI + 2, False)):
        k = I.solve_knob(lambda v: I.outlier_columns(M, N, r, v), target, 1.0, 100.0)
        err, info = run(I.outlier_columns(M, N, r, k))
        assert info["wide"] == wide
        assert err < BAR, ("outlier columns", target, err)


@pytest.mark.parametrize("M,N,rank", [(1024, 1024, 16), (1024, 3072, 32)])
def test_column_statistic_from_both_sides(M, N, rank):
    """Above the band. A low-rank signal with outlier columns: the column concentration explains a
    fifth to a half of the proxy, the matrix takes the wide gate (with the cheap gates such mixtures
    sit at 3e-3 .. 7e-3 at 1024x3072). Pure outlier columns x100: concentration = proxy, cheap
    gates. Outlier columns with 2e-3 / 4e-3 of the mass outside them: either side of the bulk
    threshold."""
    def ratio(X):
        p, c, _ = stats(X)
        return c / p
    for target in (0.225, 0.5):
        k = I.solve_knob(lambda v: I.low_rank_plus_columns(M, N, rank, 0.1, N // 100, v), target, 1.0, 300.0, stat=ratio)
        err, info = run(I.low_rank_plus_columns(M, N, rank, 0.1, N // 100, k))
        assert info["proxy"] > TAU_WIDE_HI and info["wide"]
        assert err < BAR / 2, ("low rank + columns", target, err)
    err, info = run(I.outlier_columns(M, N, N // 100, 100.0))
    assert info["proxy"] > TAU_WIDE_HI and not info["wide"] and info["colc"] > 0.95 * info["proxy"]
    assert err < BAR, ("pure outlier columns", err)
    r = N // 100
    for share, wide in ((BULK_SHARE - 1e-3, True), (BULK_SHARE + 1e-3, False)):
        k = np.sqrt((N - r) * (1 - share) / (share * r))
        err, info = run(I.outlier_columns(M, N, r, k))
        assert info["wide"] == wide
        assert err < BAR, ("outlier columns, bulk share", share, err)


def test_known_limit_low_rank_bulk_behind_independent_outlier_columns():
    """What the classifier cannot see: a rank-32 bulk (10 % noise) whose outlier columns carry
    independent entries. The column norms explain the proxy (colc / proxy 0.97), so the matrix
    keeps the cheap gates and lands above the bar; the wide gate's terms would fix it. Stated in the
    header as a known limit of ANC_NS_BF16; this test keeps the number honest."""
    M, N = 1024, 3072
    rng = np.random.default_rng(0)
    g = rng.standard_normal((M, N)).astype(np.float32)
    x = ((rng.standard_normal((M, 32)) @ rng.standard_normal((32, N))) / np.sqrt(32)).astype(np.float32) + np.float32(0.1) * g
    cols = rng.choice(N, N // 100, replace=False)
    x[:, cols] = np.float32(23.5) * rng.standard_normal((M, cols.size)).astype(np.float32)
    ref = host_ns(x, PE_SCHEDULE, 5)
    info = {}
    cheap = rel(chain(x, PE_SCHEDULE, 5, "bf16", info=info), ref)
    assert not info["wide"] and info["colc"] > 0.9 * info["proxy"]
    assert 2e-3 < cheap < 3.5e-3
    assert rel(chain(x, PE_SCHEDULE, 5, "bf16", overrides={"wide": True}), ref) < 1e-4
    assert rel(chain(x, PE_SCHEDULE, 5, "bf16_x3"), ref) < 1e-4
