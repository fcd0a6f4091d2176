"""Pins the numpy AdamW / bf16 / SR oracle against what the reference's own tests and the
mathematics fix (no GPU)."""
import math

import numpy as np

from oracle.adamw_ref import AdamWRef, adamw_step_div, adamw_step_ibc
from oracle.bf16_ref import bf16_rne_bits, bits_to_f32, bf16_sr_bits, sr_dither
from util import max_ulp


def test_reference_case_two_forms_agree_to_reference_bar():
    """tests/optim/test_adamw.py:19-43: seed 0, 5 steps; the kernel form and the numpy form agree
    to the reference's own bar rel < 1e-5 (they are NOT bit-identical: see the cancellation test)."""
    rng = np.random.default_rng(0)
    lr, b1, b2, eps, wd = 0.01, 0.9, 0.999, 1e-8, 0.01
    p_w = (rng.standard_normal((256, 64)) * 0.1).astype(np.float32)
    p_n = (1.0 + rng.standard_normal(64) * 0.05).astype(np.float32)
    a = AdamWRef({"w": p_w, "n": p_n}, lr, (b1, b2), eps, wd, ("n",), form="div")
    b = AdamWRef({"w": p_w, "n": p_n}, lr, (b1, b2), eps, wd, ("n",), form="ibc")
    for _ in range(5):
        grads = {"w": (rng.standard_normal((256, 64)) * 0.5).astype(np.float32),
                 "n": (rng.standard_normal(64) * 0.5).astype(np.float32)}
        a.step(grads); b.step(grads)
        for n in ("w", "n"):
            e = np.abs(a.st[n]["p"] - b.st[n]["p"]).max() / (np.abs(a.st[n]["p"]).max() + 1e-9)
            assert e < 1e-5
    assert a.t == 5


def test_first_step_closed_form():
    """t = 1 from zero moments: m_hat = g, v_hat = g*g, so dp = -lr*(g/(|g|+eps) + wd*p)."""
    rng = np.random.default_rng(1)
    p = rng.standard_normal(4096).astype(np.float32)
    g = (rng.standard_normal(4096) * 1e-3).astype(np.float32)
    lr, wd = 3e-4, 0.1
    pn, m, v = adamw_step_div(p, np.zeros_like(p), np.zeros_like(p), g, lr, 0.9, 0.95, 1e-8, wd, 1)
    g64, p64 = g.astype(np.float64), p.astype(np.float64)
    want = p64 - lr * (g64 / (np.abs(g64) + 1e-8) + wd * p64)
    assert np.max(np.abs(pn - want)) < 2e-6 * np.max(np.abs(want))
    assert np.allclose(m, 0.1 * g64, rtol=1e-6) and np.allclose(v, 0.05 * g64 * g64, rtol=1e-6)
    # a dropped weight-decay term or a sign error shows up at once
    assert np.max(np.abs(pn - (p64 + lr * (g64 / (np.abs(g64) + 1e-8) + wd * p64)))) > 1e-4


def test_zero_gradient_decays_moments_only_and_wd_zero_names():
    p = np.linspace(-1, 1, 128).astype(np.float32)
    m0 = np.full(128, 0.5, np.float32)
    v0 = np.full(128, 0.25, np.float32)
    pn, m, v = adamw_step_div(p, m0, v0, np.zeros(128, np.float32), 1e-3, 0.9, 0.95, 1e-8, 0.0, 10)
    assert np.all(m == np.float32(0.9) * m0) and np.all(v == np.float32(0.95) * v0)
    mh = 0.45 / (1 - 0.9 ** 10)
    vh = 0.2375 / (1 - 0.95 ** 10)
    assert np.allclose(p - pn, 1e-3 * mh / (math.sqrt(vh) + 1e-8), rtol=0, atol=2e-7)


def test_fp64_evaluation_agrees():
    rng = np.random.default_rng(2)
    n = 10000
    p, m, g = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
    v = rng.random(n).astype(np.float32)
    lr, b1, b2, eps, wd, t = 1e-2, 0.9, 0.999, 1e-8, 0.01, 4
    pn, mn, vn = adamw_step_div(p, m, v, g, lr, b1, b2, eps, wd, t)
    P, M, V, G = (x.astype(np.float64) for x in (p, m, v, g))
    M2 = b1 * M + (1 - b1) * G
    V2 = b2 * V + (1 - b2) * G * G
    P2 = P - lr * ((M2 / (1 - b1 ** t)) / (np.sqrt(V2 / (1 - b2 ** t)) + eps) + wd * P)
    assert np.max(np.abs(pn - P2)) < 1e-6 and np.max(np.abs(mn - M2)) < 1e-6


def test_forms_differ_at_cancellation_points():
    """The multiply-by-reciprocal kernel form is not within 1 ulp of the divide form everywhere
    (why the device evaluates the divide form): some elements differ by more than 1 ulp."""
    rng = np.random.default_rng(0)
    p = (0.02 * rng.standard_normal(1 << 18)).astype(np.float32)
    g = bits_to_f32(bf16_rne_bits((1e-3 * rng.standard_normal(1 << 18)).astype(np.float32)))
    z = np.zeros_like(p)
    a = adamw_step_div(p, z, z, g, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1)[0]
    b = adamw_step_ibc(p, z, z, g, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1 / (1 - 0.9), 1 / (1 - 0.95))[0]
    assert max_ulp(a, b) > 1
    assert np.max(np.abs(a - b)) < 1e-8


def test_bf16_rne_is_nearest_even_by_brute_force():
    """Value-level definition: among the two neighbouring bf16 values pick the nearer, ties to
    the even mantissa -- checked against a search that does not use the bit trick."""
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(2000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 2000),
                        np.array([1.0, 1.00390625, 1.01171875, 1.005859375, -1.00390625, 0.0,
                                  3.3895314e38], np.float32)]).astype(np.float32)
    got = bits_to_f32(bf16_rne_bits(x)).astype(np.float64)
    u = x.view(np.uint32)
    lo = bits_to_f32((u >> 16).astype(np.uint16)).astype(np.float64)          # truncation
    hi = bits_to_f32(((u >> 16) + 1).astype(np.uint16)).astype(np.float64)    # next in magnitude
    x64 = x.astype(np.float64)
    dl, dh = np.abs(x64 - lo), np.abs(hi - x64)
    even_lo = ((u >> 16) & 1) == 0
    want = np.where(dl < dh, lo, np.where(dh < dl, hi, np.where(even_lo, lo, hi)))
    finite = np.isfinite(hi)
    assert np.array_equal(got[finite], want[finite])
    assert bf16_rne_bits(np.float32(1.00390625)) == 0x3F80         # 1 + 2^-8: tie -> even (down)
    assert bf16_rne_bits(np.float32(1.01171875)) == 0x3F82         # 1 + 3*2^-8: tie -> even (up)
    assert bf16_rne_bits(np.float32(1.005859375)) == 0x3F81        # 1 + 3*2^-9: nearest


def test_sr_hash_hand_computed_and_invariants():
    # one value worked by hand with Python integers
    row, col, seed = 12345, 37, 99
    key = ((row * 73856093) & 0xFFFFFFFF) ^ ((col * 19349663) & 0xFFFFFFFF) ^ seed
    h = (key * 0x9E3779B1) & 0xFFFFFFFF
    h ^= h >> 16
    h = (h * 0x85EBCA6B) & 0xFFFFFFFF
    h ^= h >> 13
    assert int(sr_dither(row, col, seed)) == h & 0xFFFF
    # exact bf16 values are unchanged whatever the seed (tests/kernels/_probe_sr_ops.py:62-66)
    x = bits_to_f32(bf16_rne_bits(np.random.default_rng(0).standard_normal(4096).astype(np.float32)))
    for s in (0, 7, 123456):
        assert np.array_equal(bits_to_f32(bf16_sr_bits(x, s)), x)
    # unbiased: mean over 400 seeds within 10% of one bf16 ulp (tests/kernels/_probe_sr_ops.py:44-61)
    v = np.full((64, 128), 1.0 + 0.4 / 256.0, np.float32)
    acc = np.zeros(v.shape, np.float64)
    for s in range(400):
        acc += bits_to_f32(bf16_sr_bits(v, s)).reshape(v.shape)
    assert abs(acc.mean() / 400 - float(v[0, 0])) / (1 / 128.0) < 0.1
    # results are either neighbour, never anything else
    out = bits_to_f32(bf16_sr_bits(v, 5))
    assert set(np.unique(out)) <= {np.float32(1.0), np.float32(1.0078125)}
    # non-finite values pass through
    bad = np.array([np.inf, -np.inf, np.nan], np.float32)
    b = bf16_sr_bits(bad, 1)
    assert b[0] == 0x7F80 and b[1] == 0xFF80 and (b[2] & 0x7F80) == 0x7F80 and (b[2] & 0x7F) != 0
