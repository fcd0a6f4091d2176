"""Pins the Muon / Newton-Schulz oracle (no GPU)."""
import numpy as np

from oracle.muon_ref import (newton_schulz5, host_ns, ns_any_shape, ortho_err, PE_SCHEDULE,
                             coef_at, muon_momentum, muon_update, shape_scale, MuonRef,
                             default_is_muon, ns_reference_device_model, A_COEF, B_COEF, C_COEF)
from util import rel_fro


def _poly(s, sched, n):
    for k in range(n):
        a, b, c = coef_at(sched, k)
        s = a * s + b * s ** 3 + c * s ** 5
    return s


def test_svd_cross_check():
    """NS acts on singular values only: U p5(S/||S||) V^T from an fp64 SVD is an independent
    oracle. A transposed operand, a dropped term or a wrong coefficient breaks it."""
    rng = np.random.default_rng(0)
    for shape in ((48, 48), (32, 80)):
        X = rng.standard_normal(shape)
        U, S, Vt = np.linalg.svd(X, full_matrices=False)
        for sched in (None, PE_SCHEDULE):
            want = (U * _poly(S / np.linalg.norm(S), sched, 5)) @ Vt
            assert rel_fro(host_ns(X, sched, 5), want) < 2e-5
        assert rel_fro(newton_schulz5(X, 5), (U * _poly(S / np.linalg.norm(S), None, 5)) @ Vt) < 2e-5


def test_fixed_points_of_the_scalar_map():
    assert abs(_poly(1.0, None, 1) - (A_COEF + B_COEF + C_COEF)) < 1e-12      # 0.7010
    assert abs(sum(PE_SCHEDULE[-1]) - 0.9853) < 1e-4
    assert coef_at(PE_SCHEDULE, 9) == PE_SCHEDULE[-1] and coef_at(None, 3) == (A_COEF, B_COEF, C_COEF)


def test_equivariance_and_invariants():
    rng = np.random.default_rng(1)
    X = rng.standard_normal((64, 128)).astype(np.float32)
    Y = host_ns(X, PE_SCHEDULE, 5)
    assert rel_fro(ns_any_shape(X.T, PE_SCHEDULE), Y.T) < 1e-5          # NS(X^T) = NS(X)^T
    assert rel_fro(host_ns(7.5 * X, PE_SCHEDULE, 5), Y) < 1e-5          # scale invariance
    assert np.all(host_ns(np.zeros((64, 64)), PE_SCHEDULE, 5) == 0)     # zero stays zero
    s = np.linalg.svd(Y, compute_uv=False)
    assert 0.6 < s.min() and s.max() < 1.2
    # Polar Express beats Keller at 5 iterations (tests/kernels/_probe_polar_express_device.py:83)
    assert ortho_err(Y) < ortho_err(host_ns(X, None, 5)) and ortho_err(Y) < 0.1
    # tall input: newton_schulz5 transposes in and out (ancora/optim/muon.py:72-74,80)
    T = rng.standard_normal((96, 32)).astype(np.float32)
    assert newton_schulz5(T).shape == (96, 32)
    assert rel_fro(newton_schulz5(T), newton_schulz5(T.T).T) < 1e-5


def test_reference_rounding_points_sit_far_from_fp32():
    """The reference's own device rounding (bf16 storage of X, A, B) is several 1e-3 away from
    host_ns, which is why the library carries fp32 between GEMMs."""
    rng = np.random.default_rng(2)
    X = rng.standard_normal((256, 256)).astype(np.float32)
    e = rel_fro(ns_reference_device_model(X, PE_SCHEDULE), host_ns(X, PE_SCHEDULE, 5))
    assert 2e-3 < e < 5e-2


def test_momentum_update_and_step():
    rng = np.random.default_rng(3)
    buf0 = rng.standard_normal((8, 8)).astype(np.float32)
    g = rng.standard_normal((8, 8)).astype(np.float32)
    buf, u = muon_momentum(buf0, g, 0.95, True)
    assert np.allclose(buf, 0.95 * buf0 + g, rtol=1e-6) and np.allclose(u, g + 0.95 * buf, rtol=1e-6)
    assert np.array_equal(muon_momentum(buf0, g, 0.95, False)[1], buf)
    assert shape_scale(1024, 1024) == 1 and shape_scale(1024, 3072) == 1
    assert abs(shape_scale(2048, 1024) - 2 ** 0.5) < 1e-12 and abs(shape_scale(3072, 1024) - 3 ** 0.5) < 1e-12
    W = rng.standard_normal((16, 8)).astype(np.float32)
    O = rng.standard_normal((16, 8)).astype(np.float32)
    assert np.allclose(muon_update(W, O, 0.02), W - 0.02 * 2 ** 0.5 * O, rtol=1e-6)
    opt = MuonRef({"w": W}, lr=0.02)
    opt.step({"w": O})
    _, u = muon_momentum(np.zeros_like(W), O)
    assert np.array_equal(opt.w["w"], muon_update(W, newton_schulz5(u), 0.02))


def test_routing_table():
    """ancora/optim/hybrid.py:18-25 over the Qwen3 / MoE name lists (qwen3_model.py:41-46,
    moe_model.py:51-60)."""
    two, one, three = np.zeros((4, 4)), np.zeros(4), np.zeros((2, 4, 4))
    muon = ["layer0.q_proj", "layer3.k_proj", "layer1.v_proj", "layer0.o_proj", "layer2.gate_proj",
            "layer2.up_proj", "layer27.down_proj", "layer1.ffn.router"]
    adam = ["embed", "lm_head", "final_norm", "layer0.input_ln", "layer0.post_ln", "layer0.q_norm",
            "layer0.k_norm", "wte", "wpe"]
    for n in muon:
        assert default_is_muon(n, two)
    for n in adam:
        assert not default_is_muon(n, two)
    assert not default_is_muon("layer0.q_proj", one)
    assert not default_is_muon("layer1.ffn.gate_proj", three)
