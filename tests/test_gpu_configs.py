"""The BASELINE configurations at (or near) their real sizes, checked through the oracle on
samples and through size-independent properties elsewhere."""
import numpy as np
import pytest

from oracle.adamw_ref import adamw_step_div
from oracle.bf16_ref import bf16_rne_bits, bf16_sr_bits, bits_to_f32
from oracle.muon_ref import host_ns, ortho_err, PE_SCHEDULE, muon_momentum, muon_update, ns_any_shape
from oracle import gradnorm_ref as gn
from util import rel_fro, bits_equal, max_ulp, bf16_grad

pytestmark = pytest.mark.gpu


def test_config3_muon_only_stress_full_batches(gpu):
    """Config 3: the 196 matrices of the Qwen3-0.6B set grouped by shape (56 x 1024x1024,
    56 x 1024x2048, 84 x 1024x3072), ~N(0,1), 5 Polar-Express iterations, bf16 mode; a sample of
    each group against the fp32 oracle (2e-3), every matrix through the orthogonality property,
    and the fp32 validation mode on a sample (1e-5)."""
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd.muon_ns import ns_batched
    for (M, N, E) in ((1024, 1024, 56), (1024, 2048, 56), (1024, 3072, 84)):
        rng = np.random.default_rng(M + N)
        base = rng.standard_normal((4, M, N)).astype(np.float32)      # 4 distinct matrices ...
        X = DevBuf.empty((E * M, N), np.float32)
        for e in range(E):                                            # ... scaled per slot (NS is scale
            X.at_pos(e * M).upload(base[e % 4] * np.float32(1 + e))   # invariant; bits differ per slot)
        ns_batched(X, E, M, N, 0, schedule=PE_SCHEDULE, mode="bf16")
        want = [host_ns(base[i], PE_SCHEDULE, 5) for i in range(4)]
        for e in (0, 1, 2, 3, E // 2, E - 1):
            got = X.at_pos(e * M).to_numpy()[:M]
            assert rel_fro(got, want[e % 4]) < 2e-3, (M, N, e)
        for e in range(0, E, 7):
            got = X.at_pos(e * M).to_numpy()[:M]
            assert ortho_err(got) < 0.45 and np.all(np.isfinite(got))   # 5-step PE leaves sigma in ~[0.7,1.2]
            assert abs(ortho_err(got) - ortho_err(want[e % 4])) < 0.01
        X.free()
        Xf = DevBuf(np.ascontiguousarray(base[:2].reshape(2 * M, N)))
        ns_batched(Xf, 2, M, N, 0, schedule=PE_SCHEDULE, mode="fp32")
        for e in range(2):
            assert rel_fro(Xf.at_pos(e * M).to_numpy()[:M], want[e]) < 1e-5
        Xf.free()


def test_config4_moe_family_small(gpu):
    """Config 4 at reduced width: alternating dense / MoE layers, stacked [E,K,N] experts on Muon
    (one matrix per slice), (H,E) routers on AdamW, 1 of 4 experts with zero gradient."""
    from ancora_cutile_amd import HybridOptimizer, resident_is_muon, PE_SCHEDULE as PE
    from ancora_cutile_amd.shapes import moe_shapes
    shapes = moe_shapes(layers=2, hidden=128, dense_ffn=384, experts=4, expert_ffn=128, q_heads=2,
                        kv_heads=1, head_dim=128, vocab=512)
    rng = np.random.default_rng(4)
    params = {n: ((1 + 0.05 * rng.standard_normal(s)) if len(s) == 1 else 0.02 * rng.standard_normal(s))
              .astype(np.float32) for n, s in shapes.items()}
    gb, g = {}, {}
    for n, p in params.items():
        gb[n], g[n] = bf16_grad(rng, p.shape, 1e-3)
        if p.ndim == 3:
            g[n][2] = 0
            gb[n][2] = 0
    opt = HybridOptimizer(params, is_muon=resident_is_muon, muon_kw=dict(schedule=PE),
                          adamw_kw=dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1),
                          max_grad_norm=1.0, grad_dtype=np.uint16)
    r = opt.routing()
    assert "layer1.ffn.router" in r["adamw"] and "layer1.ffn.gate_proj" in r["muon"]
    assert "embed" in r["adamw"] and "layer0.down_proj" in r["muon"]
    opt.step(gb, 0)
    clip = opt.last_ctl["clip_scale"]
    mm, am = opt.muon.master(), opt.adamw.master()
    for n in r["muon"]:
        W = params[n].reshape((-1,) + params[n].shape[-2:])
        G = g[n].reshape(W.shape)
        got = mm[n].reshape(W.shape)
        for e in range(W.shape[0]):
            if not G[e].any():
                assert bits_equal(got[e], W[e])                  # idle expert: zero update at step 1
                continue
            _, u = muon_momentum(np.zeros_like(W[e]), G[e], clip=clip)
            want = muon_update(W[e], ns_any_shape(u, PE_SCHEDULE, 5), 0.02)
            assert rel_fro(W[e] - got[e], W[e] - want) < 2.5e-3, (n, e)
    for n in r["adamw"]:
        wd = 0.0 if params[n].ndim == 1 else 0.1
        want, _, _ = adamw_step_div(params[n], 0 * params[n], 0 * params[n], g[n], 3e-4, 0.9, 0.95, 1e-8,
                                    wd, 1, clip=clip)
        assert max_ulp(am[n], want) == 0, n
    opt.free()


def test_config5_flat_buffer_guard_and_update(gpu):
    """Config 5 at 1/16 size (75M elements; the kernel walks 4096-element blocks independently of
    the total): bf16 gradient with 0.01% Inf/NaN -> the guard skips and every state tensor keeps its
    bits; the clean gradient -> norm, clip, update and SR downcast match the oracle on sampled
    blocks; step counter 1000."""
    from ancora_cutile_amd import AdamW, StepGuard, DevBuf
    n = 75_000_000 // 64 * 64
    rng = np.random.default_rng(5)
    p = rng.standard_normal(n, dtype=np.float32)
    gbits = bf16_rne_bits(1e-3 * rng.standard_normal(n, dtype=np.float32))
    opt = AdamW({"flat": p}, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=True, seed=11,
                grad_dtype=np.uint16)
    m0 = (1e-3 * rng.standard_normal(n, dtype=np.float32)).reshape(-1, 64)
    v0 = (1e-6 * rng.random(n, dtype=np.float32)).reshape(-1, 64)
    opt.st["flat"]["m"].upload(m0)
    opt.st["flat"]["v"].upload(v0)
    opt.t = 999
    guard = StepGuard(1.0)
    bad = gbits.copy()
    idx = rng.choice(n, n // 10000, replace=False)
    bad[idx] = rng.choice(np.array([0x7F80, 0xFF80, 0x7FC0], np.uint16), idx.size)
    gdev = DevBuf(bad)
    guard.compute([gdev], 0)
    opt.step({"flat": gdev}, 0, guard=guard)
    assert guard.read(0)["skip"] and opt.t == 999
    s = opt.st["flat"]
    assert bits_equal(s["p32"].to_numpy().ravel(), p) and bits_equal(s["m"].to_numpy(), m0)
    assert bits_equal(s["v"].to_numpy(), v0) and not s["p16"].to_numpy().any()
    gdev.upload(gbits)
    guard.compute([gdev], 0)
    opt.step({"flat": gdev}, 0, guard=guard)
    c = guard.read(0)
    assert not c["skip"] and opt.t == 1000
    assert c["sumsq"] == gn.gradnorm_fixed([gbits])
    assert max_ulp(np.float32(c["norm"]), np.float32(gn.control(gn.gradnorm_f64([gbits]))["norm"])) <= 1
    P, M_, V = s["p32"].to_numpy().ravel(), s["m"].to_numpy().ravel(), s["v"].to_numpy().ravel()
    P16 = s["p16"].to_numpy().ravel()
    g = bits_to_f32(gbits)
    from ancora_cutile_amd.adamw import sr_seed_base
    for lo in (0, 4096 * 777, n - 4096 * 3, n - 64):
        hi = min(n, lo + 8192)
        pw, mw, vw = adamw_step_div(p[lo:hi], m0.ravel()[lo:hi], v0.ravel()[lo:hi], g[lo:hi], 3e-4, 0.9,
                                    0.95, 1e-8, 0.1, 1000, clip=c["clip_scale"])
        assert max_ulp(P[lo:hi], pw) == 0 and max_ulp(M_[lo:hi], mw) == 0 and max_ulp(V[lo:hi], vw) == 0
        assert bits_equal(P16[lo:hi], bf16_sr_bits(pw, sr_seed_base(11, 1000), first_index=lo))
    gdev.free(); guard.free(); opt.free()
