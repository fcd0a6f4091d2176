"""GPU parity of the fused AdamW kernel against the numpy oracle, through the C ABI.
Bar: m, v, p32 within 1 ulp of the oracle (0 ulp expected), bf16 copies bit-exact."""
import ctypes

import numpy as np
import pytest

from oracle.adamw_ref import AdamWRef, adamw_step_div, adamw_step_ibc
from oracle.bf16_ref import bf16_rne_bits, bf16_sr_bits, bits_to_f32
from util import max_ulp, bits_equal, bf16_grad

pytestmark = pytest.mark.gpu
ULP_TOL = 1   # fp32 ulps, before the bf16 downcast


def test_reference_case_five_steps(gpu):
    """The reference's own case (tests/optim/test_adamw.py:19-53): seed 0, (256,64)*0.1 and (64,),
    grads*0.5, 5 steps, lr=.01, betas=(.9,.999), wd=.01, no_decay=('n',)."""
    from ancora_cutile_amd import AdamW
    rng = np.random.default_rng(0)
    lr, b1, b2, eps, wd = 0.01, 0.9, 0.999, 1e-8, 0.01
    p_w = (rng.standard_normal((256, 64)) * 0.1).astype(np.float32)
    p_n = (1.0 + rng.standard_normal(64) * 0.05).astype(np.float32)
    opt = AdamW({"w": p_w.copy(), "n": p_n.copy()}, lr=lr, betas=(b1, b2), eps=eps, wd=wd,
                no_decay=("n",))
    ref = AdamWRef({"w": p_w, "n": p_n}, lr=lr, betas=(b1, b2), eps=eps, wd=wd, no_decay=("n",))
    for t in range(1, 6):
        grads = {"w": (rng.standard_normal((256, 64)) * 0.5).astype(np.float32),
                 "n": (rng.standard_normal(64) * 0.5).astype(np.float32)}
        opt.step(grads, 0)
        ref.step(grads)
        master, mom = opt.master(), opt.moments()
        for name in ("w", "n"):
            assert max_ulp(master[name], ref.st[name]["p"]) <= ULP_TOL, (t, name)
            assert max_ulp(mom[name][0], ref.st[name]["m"]) <= ULP_TOL
            assert max_ulp(mom[name][1], ref.st[name]["v"]) <= ULP_TOL
            # the reference's own bar
            e = np.abs(master[name] - ref.st[name]["p"]).max() / (np.abs(ref.st[name]["p"]).max() + 1e-9)
            assert e < 1e-5
    w16 = opt.weights()["w"]
    assert np.array_equal(w16, bits_to_f32(bf16_rne_bits(opt.master()["w"])).reshape(256, 64))
    assert opt.t == 5
    opt.free()


@pytest.mark.parametrize("t", [1, 1000])
def test_config1_bf16_grads_bit_exact(gpu, t):
    """BASELINE config 1 (AdamW part): 1024x1024 weight + 1024 gain, bf16 grads ~N(0,1e-3),
    lr=3e-4, betas=(0.9,0.95), eps=1e-8, wd=0.1 (gain 0); step 1 from zero moments and
    step 1000 from random moments."""
    from ancora_cutile_amd import AdamW
    rng = np.random.default_rng(0)
    W = (0.02 * rng.standard_normal((1024, 1024))).astype(np.float32)
    gain = (1 + 0.05 * rng.standard_normal(1024)).astype(np.float32)
    gw_bits, gw = bf16_grad(rng, (1024, 1024))
    gg_bits, gg = bf16_grad(rng, (1024,))
    opt = AdamW({"w": W, "g": gain}, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1,
                no_decay=("g",), grad_dtype=np.uint16)
    ref = AdamWRef({"w": W, "g": gain}, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, no_decay=("g",))
    if t > 1:
        for name, shape in (("w", (1024, 1024)), ("g", (1024,))):
            m0 = (1e-3 * rng.standard_normal(shape)).astype(np.float32)
            v0 = (1e-6 * rng.random(shape)).astype(np.float32)
            ref.st[name]["m"], ref.st[name]["v"] = m0.copy(), v0.copy()
            opt.st[name]["m"].upload(m0.reshape(-1, 64))
            opt.st[name]["v"].upload(v0.reshape(-1, 64))
        opt.t = ref.t = t - 1
    opt.step({"w": gw_bits, "g": gg_bits}, 0)
    ref.step({"w": gw, "g": gg})
    master, mom = opt.master(), opt.moments()
    for name in ("w", "g"):
        assert max_ulp(master[name], ref.st[name]["p"]) == 0
        assert max_ulp(mom[name][0], ref.st[name]["m"]) == 0
        assert max_ulp(mom[name][1], ref.st[name]["v"]) == 0
        p16 = opt.st[name]["p16"].to_numpy().reshape(ref.st[name]["p"].shape)
        assert bits_equal(p16, bf16_rne_bits(ref.st[name]["p"]))
    opt.free()


def test_ibc_form_matches_reference_kernel_form(gpu):
    """The low-level `_adamw` tuple evaluates the reference kernel's formula
    (ancora/optim/adamw.py:34-37) with fp32 scalars."""
    from ancora_cutile_amd import DevBuf, _adamw, _pick_otm
    rng = np.random.default_rng(3)
    n = 64 * 130
    p = rng.standard_normal(n).astype(np.float32)
    m = (0.1 * rng.standard_normal(n)).astype(np.float32)
    v = (0.01 * rng.random(n)).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    b1, b2, eps, lr, wd, t = 0.9, 0.999, 1e-8, 1e-2, 0.01, 7
    ibc1, ibc2 = 1 / (1 - b1 ** t), 1 / (1 - b2 ** t)
    d = [DevBuf(x.reshape(-1, 64)) for x in (g, m, v, p)]
    p16 = DevBuf.zeros((n // 64, 64), np.uint16)
    _adamw(0, d[0], d[1], d[2], d[3], p16, _pick_otm(n // 64), b1, b2, eps, lr, wd, ibc1, ibc2)
    pr, mr, vr = adamw_step_ibc(p, m, v, g, lr, b1, b2, eps, wd, ibc1, ibc2)
    assert max_ulp(d[3].to_numpy().ravel(), pr) <= ULP_TOL
    assert max_ulp(d[1].to_numpy().ravel(), mr) <= ULP_TOL
    assert max_ulp(d[2].to_numpy().ravel(), vr) <= ULP_TOL
    assert bits_equal(p16.to_numpy().ravel(), bf16_rne_bits(d[3].to_numpy().ravel()))
    for b in d + [p16]:
        b.free()


@pytest.mark.parametrize("n", [64, 4096, 4096 + 64, 3 * 4096 - 64, 1 << 20])
def test_stochastic_rounding_bit_exact_and_ragged_sizes(gpu, n):
    """SR downcast equals the numpy restatement of the hash bit for bit, on sizes that end
    inside, at and just past a 4096-element block."""
    from ancora_cutile_amd import _lib
    from ancora_cutile_amd._lib import api
    from ancora_cutile_amd.adamw import hyper_div
    from ancora_cutile_amd import DevBuf
    rng = np.random.default_rng(n)
    p = rng.standard_normal(n).astype(np.float32)
    m = (0.1 * rng.standard_normal(n)).astype(np.float32)
    v = (0.01 * rng.random(n)).astype(np.float32)
    gb, g = bf16_grad(rng, (n,), 1.0)
    seed = 0xC0FFEE + n
    h = hyper_div(3e-4, 0.9, 0.95, 1e-8, 3, sr=True, seed_base=seed)
    d = dict(g=DevBuf(gb), m=DevBuf(m), v=DevBuf(v), p=DevBuf(p))
    p16 = DevBuf.zeros((n,), np.uint16)
    guard_words = DevBuf(np.full(64, 0xDEADBEEF, np.uint32))       # canary after nothing: sanity
    api.anc_adamw(d["g"].ptr, d["m"].ptr, d["v"].ptr, d["p"].ptr, p16.ptr, n, _lib.BF16,
                  ctypes.byref(h), 0.1, 5, 0, 0)
    pr, mr, vr = adamw_step_div(p, m, v, g, 3e-4, 0.9, 0.95, 1e-8, 0.1, 3)
    assert max_ulp(d["p"].to_numpy(), pr) == 0
    assert max_ulp(d["m"].to_numpy(), mr) == 0 and max_ulp(d["v"].to_numpy(), vr) == 0
    assert bits_equal(p16.to_numpy(), bf16_sr_bits(pr, (seed + 5) & 0xFFFFFFFF))
    assert np.all(guard_words.to_numpy() == 0xDEADBEEF)
    for b in list(d.values()) + [p16, guard_words]:
        b.free()


def test_multi_tensor_launch_equals_single_launches(gpu):
    """Results do not depend on how tensors are batched into launches."""
    from ancora_cutile_amd import AdamW
    rng = np.random.default_rng(11)
    shapes = {"a": (64,), "b": (1024, 128), "c": (4096 + 64,), "d": (3, 64), "e": (200, 64)}
    params = {k: rng.standard_normal(s).astype(np.float32) for k, s in shapes.items()}
    grads = {k: rng.standard_normal(s).astype(np.float32) for k, s in shapes.items()}
    both = AdamW(params, wd=0.1, sr=True, seed=9)
    both.step(grads, 0)
    got = both.master()
    got16 = {k: s["p16"].to_numpy() for k, s in both.st.items()}
    for i, k in enumerate(shapes):
        one = AdamW({k: params[k]}, wd=0.1, sr=True, seed=9 + i)   # same per-tensor seed
        one.step({k: grads[k]}, 0)
        assert bits_equal(one.master()[k], got[k])
        assert bits_equal(one.st[k]["p16"].to_numpy(), got16[k])
        one.free()
    both.free()


def test_rejects_misaligned_sizes(gpu):
    from ancora_cutile_amd import AdamW
    with pytest.raises(ValueError):
        AdamW({"x": np.zeros(100, np.float32)})


def test_special_values(gpu):
    """g = 0 only decays the moments; exact-zero weights with wd = 0 stay zero; an Inf weight is
    passed through the SR downcast unchanged."""
    from ancora_cutile_amd import AdamW
    n = 128
    p = np.zeros(n, np.float32)
    p[3] = np.inf
    opt = AdamW({"x": p}, wd=0.0, sr=True)
    opt.st["x"]["m"].upload(np.full((2, 64), 0.5, np.float32))
    opt.st["x"]["v"].upload(np.full((2, 64), 0.25, np.float32))
    opt.step({"x": np.zeros(n, np.float32)}, 0)
    m, v = opt.moments()["x"]
    assert np.all(m == np.float32(0.9) * np.float32(0.5)) and np.all(v == np.float32(0.95) * np.float32(0.25))
    w16 = opt.st["x"]["p16"].to_numpy().ravel()
    assert (w16[3] & 0x7F80) == 0x7F80        # Inf * wd(0) is NaN: still non-finite, not wrapped
    opt.free()
