"""GPU parity of the deterministic global grad-norm, clip scale and skip guard."""
import numpy as np
import pytest

from oracle import gradnorm_ref as gn
from oracle.adamw_ref import AdamWRef
from util import max_ulp, bits_equal, bf16_grad

pytestmark = pytest.mark.gpu


def _bufs(arrs):
    from ancora_cutile_amd import DevBuf
    return [DevBuf(a) for a in arrs]


def _ctl(arrs, max_norm=1.0):
    from ancora_cutile_amd import StepGuard
    g = StepGuard(max_norm)
    bufs = _bufs(arrs)
    g.compute(bufs, 0)
    out = g.read(0)
    for b in bufs:
        b.free()
    g.free()
    return out


@pytest.mark.parametrize("sizes", [(64,), (8192,), (8193,), (5,), (100000, 77, 8192 * 3 + 1)])
def test_matches_fixed_order_oracle_bitwise_and_f64_within_one_ulp(gpu, sizes):
    rng = np.random.default_rng(sum(sizes))
    arrs = []
    for i, n in enumerate(sizes):
        if i % 2 == 0:
            arrs.append(bf16_grad(rng, (n,), 1e-3)[0])
        else:
            arrs.append(rng.standard_normal(n).astype(np.float32))
    c = _ctl(arrs)
    fixed = gn.gradnorm_fixed(arrs)
    assert c["sumsq"] == fixed                                   # same bits as the restated order
    want = gn.control(gn.gradnorm_f64(arrs), 1.0)
    assert max_ulp(np.float32(c["norm"]), np.float32(want["norm"])) <= 1
    mine = gn.control(fixed, 1.0)
    assert np.float32(c["norm"]) == np.float32(mine["norm"])
    assert np.float32(c["clip_scale"]) == np.float32(mine["clip_scale"])
    assert not c["skip"]


def test_closed_forms(gpu):
    """3-4-5 and a constant vector: exact answers."""
    a = np.zeros(64, np.float32); a[0] = 3.0
    b = np.zeros(9000, np.float32); b[-1] = 4.0
    c = _ctl([a, b], max_norm=1.0)
    assert c["sumsq"] == 25.0 and c["norm"] == 5.0
    assert np.float32(c["clip_scale"]) == np.float32(1.0) / (np.float32(5.0) + np.float32(1e-6))
    ones = np.full(1 << 16, 0.5, np.float32)
    assert _ctl([ones], max_norm=None)["sumsq"] == (1 << 16) * 0.25
    assert _ctl([ones], max_norm=None)["clip_scale"] == 1.0


def test_independent_of_launch_grouping_and_repeatable(gpu):
    """One multi-tensor launch, per-tensor launches into the same partial array, and a second
    run all give the same bits."""
    import ctypes
    from ancora_cutile_amd import DevBuf, StepGuard, _lib
    from ancora_cutile_amd._lib import api
    rng = np.random.default_rng(5)
    arrs = [bf16_grad(rng, (n,), 1e-3)[0] for n in (70000, 64, 8192 * 2, 123456)]
    a = _ctl(arrs)["sumsq"]
    assert _ctl(arrs)["sumsq"] == a
    bufs = _bufs(arrs)
    nparts = [api.anc_gradnorm_num_partials(b.size) for b in bufs]
    parts = DevBuf.zeros((sum(nparts),), np.float64)
    ctl = DevBuf.zeros((8,), np.uint32)
    off = 0
    for b, k in zip(bufs, nparts):
        api.anc_gradnorm_partials(b.ptr, b.size, _lib.BF16, parts.ptr, off, 0)
        off += k
    api.anc_gradnorm_finalize(parts.ptr, sum(nparts), 1.0, 1e-6, 0, ctl.ptr, 0)
    raw = ctl.to_numpy()
    assert raw.view(np.float64)[0] == a
    for b in bufs + [parts, ctl]:
        b.free()


@pytest.mark.parametrize("bad", [np.inf, -np.inf, np.nan])
def test_non_finite_gradient_skips_the_step(gpu, bad):
    """A single Inf/NaN anywhere sets skip; AdamW then leaves m, v, p32, p16 untouched and the
    step counter does not advance."""
    from ancora_cutile_amd import AdamW, StepGuard, DevBuf
    rng = np.random.default_rng(1)
    p = rng.standard_normal((300, 64)).astype(np.float32)
    g = rng.standard_normal((300, 64)).astype(np.float32)
    opt = AdamW({"x": p})
    guard = StepGuard(1.0)
    opt.step({"x": g}, 0)                      # one clean step so the state is non-trivial
    before = (opt.master()["x"], *opt.moments()["x"], opt.st["x"]["p16"].to_numpy())
    g2 = g.copy(); g2[123, 7] = bad
    gb = DevBuf(g2)
    guard.compute([gb], 0)
    opt.step({"x": gb}, 0, guard=guard)
    assert guard.read(0)["skip"] and opt.last_skipped and opt.t == 1
    after = (opt.master()["x"], *opt.moments()["x"], opt.st["x"]["p16"].to_numpy())
    for x, y in zip(before, after):
        assert bits_equal(x, y)
    gb.free(); guard.free(); opt.free()


def test_clip_scale_feeds_adamw(gpu):
    """Clip active (norm > 1): AdamW with the device-computed scale equals the oracle evaluated
    with that same scale, bit for bit."""
    from ancora_cutile_amd import AdamW, StepGuard, DevBuf
    rng = np.random.default_rng(2)
    p = (0.02 * rng.standard_normal((512, 64))).astype(np.float32)
    gb_bits, g = bf16_grad(rng, (512, 64), 1e-3)
    rows = rng.choice(512, 5, replace=False)
    g[rows] *= 100
    from oracle.bf16_ref import bf16_rne_bits, bits_to_f32
    gb_bits = bf16_rne_bits(g); g = bits_to_f32(gb_bits).reshape(512, 64)
    opt = AdamW({"x": p}, wd=0.1, grad_dtype=np.uint16)
    ref = AdamWRef({"x": p}, wd=0.1)
    guard = StepGuard(0.05)
    gdev = DevBuf(gb_bits)
    guard.compute([gdev], 0)
    opt.step({"x": gdev}, 0, guard=guard)
    c = guard.read(0)
    assert 0 < c["clip_scale"] < 1
    want = gn.control(gn.gradnorm_fixed([gb_bits]), 0.05)
    assert np.float32(c["clip_scale"]) == np.float32(want["clip_scale"])
    ref.step({"x": g}, clip=c["clip_scale"])
    assert max_ulp(opt.master()["x"], ref.st["x"]["p"]) == 0
    gdev.free(); guard.free(); opt.free()
