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
            assert rel_fro(W[e] - got[e], W[e] - want) < 2e-3, (n, e)
    for n in r["adamw"]:
        wd = 0.0 if params[n].ndim == 1 or "router" in n else 0.1    # the router is not decayed (ancora/kernels/moe.py:603-604)
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


def _zero_idle(rng, gb, g, params, idle_per_tensor=4):
    """Config 4's sparsity: `idle_per_tensor` of the experts of every stacked tensor get an all-zero
    gradient. Returns {name: sorted idle expert indices}."""
    idle = {}
    for n, p in params.items():
        if p.ndim == 3:
            idx = np.sort(rng.choice(p.shape[0], idle_per_tensor, replace=False))
            g[n][idx] = 0
            gb[n][idx] = 0
            idle[n] = [int(i) for i in idx]
    return idle


def test_config4_moe_family_real_width(gpu):
    """Config 4 at its real width: one dense layer (FFN 3072) and one MoE layer (16 experts of
    1024x1024 per tensor, stacked [16,1024,1024]; router 1024x16 on AdamW), hidden 1024, 4 of 16
    experts idle. 59 Muon matrices in three Newton-Schulz shape groups, all on the 256x256-tile
    kernels, the (1024,1024) group with its residual-term iterations. Every expert of one stacked
    tensor, three of each other and every 2-D projection against the numpy oracle at 2e-3."""
    from ancora_cutile_amd import HybridOptimizer, resident_is_muon, PE_SCHEDULE as PE
    from ancora_cutile_amd.shapes import moe_shapes
    shapes = moe_shapes(layers=2, hidden=1024, dense_ffn=3072, experts=16, expert_ffn=1024, vocab=2048)
    rng = np.random.default_rng(44)
    params = {n: ((1 + 0.05 * rng.standard_normal(s)) if len(s) == 1 else 0.02 * rng.standard_normal(s))
              .astype(np.float32) for n, s in shapes.items()}
    gb, g = {}, {}
    for n, p in params.items():
        gb[n], g[n] = bf16_grad(rng, p.shape, 1e-3)
    idle = _zero_idle(rng, gb, g, params)
    opt = HybridOptimizer(params, is_muon=resident_is_muon, muon_kw=dict(schedule=PE),
                          adamw_kw=dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1),
                          max_grad_norm=1.0, grad_dtype=np.uint16)
    r = opt.routing()
    assert "layer1.ffn.router" in r["adamw"] and len(r["muon"]) == 7 + 4 + 3
    assert sorted((b.M, b.Nn, b.E) for b in opt.muon.engine.batches) == [(1024, 1024, 52), (1024, 2048, 4), (1024, 3072, 3)]
    opt.step(gb, 0)
    clip = opt.last_ctl["clip_scale"]
    order = opt.muon_names + opt.adamw_names
    assert opt.last_ctl["sumsq"] == gn.gradnorm_fixed([gb[n] for n in order])
    mm, am = opt.muon.master(), opt.adamw.master()
    worst = 0.0
    for n in r["muon"]:
        W = params[n].reshape((-1,) + params[n].shape[-2:])
        G = g[n].reshape(W.shape)
        got = mm[n].reshape(W.shape)
        if W.shape[0] == 1:
            picks = [0]
        elif n.endswith("ffn.down_proj"):
            picks = list(range(W.shape[0]))
        else:
            live = [e for e in range(W.shape[0]) if e not in idle[n]]
            picks = sorted(set(idle[n] + live[:2] + live[-1:]))
        for e in picks:
            if not G[e].any():
                assert e in idle[n] and bits_equal(got[e], W[e])        # idle expert: untouched at step 1
                continue
            _, u = muon_momentum(np.zeros_like(W[e]), G[e], clip=clip)
            want = muon_update(W[e], ns_any_shape(u, PE_SCHEDULE, 5), 0.02)
            err = rel_fro(W[e] - got[e], W[e] - want)
            worst = max(worst, err)
            assert err < 2e-3, (n, e, err)
    print(f"\nconfig 4 at width 1024: worst update-direction error {worst:.3e}")
    for n in r["adamw"]:
        wd = 0.0 if params[n].ndim == 1 or "router" in n else 0.1    # the router is not decayed (ancora/kernels/moe.py:603-604)
        want, _, _ = adamw_step_div(params[n], 0 * params[n], 0 * params[n], g[n], 3e-4, 0.9, 0.95, 1e-8,
                                    wd, 1, clip=clip)
        assert max_ulp(am[n], want) == 0, n
    opt.free()


def test_config4_expert_optimizer_e16_1024(gpu):
    """The reference's expert probe size (tests/kernels/_probe_expert_muon_ns.py:24-54: E=16 of
    1024x1024, distinct experts) through the MoE layer's own optimizer class: three stacked tensors,
    4 idle experts each, Polar-Express. Per expert: cos > 0.99 and rel < 0.05 (the reference's bars:
    no cross-matrix leak) and the 2e-3 bar against the oracle; idle experts untouched; the transposed
    bf16 copy the backward reads equals the transpose of the new bf16 weights; router on AdamW."""
    from ancora_cutile_amd import DevBuf, PE_SCHEDULE as PE
    from ancora_cutile_amd.moe import ExpertOptimizer
    from oracle.adamw_ref import adamw_step_ibc
    E, H = 16, 1024
    rng = np.random.default_rng(45)
    weights = {n: (0.02 * rng.standard_normal((E, H, H))).astype(np.float32) for n in ExpertOptimizer.NAMES}
    router = (0.02 * rng.standard_normal((H, E))).astype(np.float32)
    gb, g = {}, {}
    for n in weights:
        gb[n], g[n] = bf16_grad(rng, (E, H, H), 1e-3)
    idle = _zero_idle(rng, gb, g, weights)
    rgrad = (1e-3 * rng.standard_normal((H, E))).astype(np.float32)
    opt = ExpertOptimizer(weights, router=router, optimizer="muon")
    gdev = {n: DevBuf(gb[n].reshape(E * H, H)) for n in weights}
    rdev = DevBuf(rgrad.reshape(-1, 64))
    opt.step(gdev, 0, lr=1e-3, muon_lr=0.02, router_grad=rdev, schedule=PE)
    gpu.stream_sync(0)
    got = opt.master()
    for n in weights:
        s = opt.st[n]
        p16 = s["p16"].to_numpy().reshape(E, H, H)
        p16T = s["p16T"].to_numpy().reshape(E, H, H)
        for e in range(E):
            assert bits_equal(p16T[e], np.ascontiguousarray(p16[e].T)), (n, e)
            if e in idle[n]:
                assert bits_equal(got[n][e], weights[n][e]), (n, e)
                continue
            if n != "up_proj" and e not in (0, 7, 15):
                continue
            _, u = muon_momentum(np.zeros((H, H), np.float32), g[n][e])
            o_ref = host_ns(u, PE_SCHEDULE, 5)
            o_got = (weights[n][e].astype(np.float64) - got[n][e]) / 0.02
            cos = float(np.sum(o_got * o_ref) / (np.linalg.norm(o_got) * np.linalg.norm(o_ref)))
            assert cos > 0.99 and rel_fro(o_got, o_ref) < 0.05, (n, e)            # reference bars
            assert rel_fro(o_got, o_ref) < 2e-3, (n, e, rel_fro(o_got, o_ref))
    b1, b2 = 0.9, 0.999
    want, _, _ = adamw_step_ibc(router, 0 * router, 0 * router, rgrad, 1e-3, b1, b2, 1e-8, 0.0,
                                1.0 / (1.0 - b1), 1.0 / (1.0 - b2))
    assert max_ulp(got["router"], want) <= 1
    for b in list(gdev.values()) + [rdev]:
        b.free()
    opt.free()


def _tiled(base, n, scale_step):
    """n-element fp32 array made of copies of `base`, copy k scaled by 1 + k*scale_step: cheap to
    build at 1.2e9 elements, different bits in every copy."""
    out = np.empty(n, np.float32)
    B = base.size
    for k, lo in enumerate(range(0, n, B)):
        hi = min(n, lo + B)
        np.multiply(base[:hi - lo], np.float32(1.0 + k * scale_step), out=out[lo:hi])
    return out


def _block(buf, lo, hi):
    """Elements [lo, hi) of a (R, 64) device buffer, lo and hi multiples of 64."""
    return buf.at_pos(lo // 64).view(((hi - lo) // 64, 64)).to_numpy().ravel()


def test_config5_flat_buffer_full_size(gpu):
    """Config 5 at its real size, one flat 1.2e9-element buffer (fp32 master, m, v: 4.8 GB each,
    byte offsets beyond 2^32 from element 2^30 on; bf16 gradient and weights 2.4 GB), step 1000.
    Gradient with 0.01 % Inf/NaN: the guard skips, the master (all of it), the bf16 weights (all)
    and sampled blocks of m and v keep their bits. Clean gradient: sum of squares bit-equal to the
    fixed-order oracle, norm within 1 ulp of the fp64 closed form; m, v, master 0 ulp and stochastic
    bf16 bits equal on blocks at the start, across elements 2^29 and 2^30 (byte offsets 2^31 and
    2^32 of the fp32 arrays), deep in the upper part and at the very end."""
    from ancora_cutile_amd import AdamW, StepGuard, DevBuf
    from ancora_cutile_amd.adamw import sr_seed_base
    n = 1_200_000_000
    B = 1 << 24
    rng = np.random.default_rng(55)
    p = _tiled(rng.standard_normal(B, dtype=np.float32), n, 2.0 ** -12)
    m0 = _tiled(1e-3 * rng.standard_normal(B, dtype=np.float32), n, 2.0 ** -11)
    v0 = _tiled(1e-6 * rng.random(B, dtype=np.float32), n, 2.0 ** -10)
    gbase = bf16_rne_bits(1e-3 * rng.standard_normal(B, dtype=np.float32))
    gbits = np.empty(n, np.uint16)
    for k, lo in enumerate(range(0, n, B)):
        hi = min(n, lo + B)
        gbits[lo:hi] = gbase[:hi - lo] ^ np.uint16(0x8000 if k & 1 else 0)      # alternate the sign per copy
    opt = AdamW({"flat": p}, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=True, seed=11,
                grad_dtype=np.uint16)
    s = opt.st["flat"]
    s["m"].upload(m0.reshape(-1, 64))
    s["v"].upload(v0.reshape(-1, 64))
    opt.t = 999
    guard = StepGuard(1.0)
    spans = [(0, 8192), ((1 << 29) - 4096, (1 << 29) + 4096), ((1 << 30) - 4096, (1 << 30) + 4096),
             (1_150_000_000 // 64 * 64, 1_150_000_000 // 64 * 64 + 8192), (n - 4096 * 3, n), (n - 64, n)]
    # -- 0.01 % non-finite: skipped, nothing written
    idx = rng.choice(n, n // 10000, replace=False)
    saved = gbits[idx].copy()
    gbits[idx] = rng.choice(np.array([0x7F80, 0xFF80, 0x7FC0], np.uint16), idx.size)
    gdev = DevBuf(gbits)
    guard.compute([gdev], 0)
    opt.step({"flat": gdev}, 0, guard=guard)
    assert guard.read(0)["skip"] and opt.t == 999 and opt.last_skipped
    assert bits_equal(s["p32"].to_numpy().ravel(), p) and not s["p16"].to_numpy().any()
    for lo, hi in spans:
        assert bits_equal(_block(s["m"], lo, hi), m0[lo:hi]) and bits_equal(_block(s["v"], lo, hi), v0[lo:hi])
    # -- clean gradient: the update
    gbits[idx] = saved
    gdev.upload(gbits)
    guard.compute([gdev], 0)
    opt.step({"flat": gdev}, 0, guard=guard)
    c = guard.read(0)
    assert not c["skip"] and opt.t == 1000
    parts = np.concatenate([gn.chunk_partials(gbits[lo:lo + B]) for lo in range(0, n, B)])   # B % 8192 == 0
    assert c["sumsq"] == gn.finalize_fixed(parts)
    f64 = sum(gn.gradnorm_f64([gbits[lo:lo + B]]) for lo in range(0, n, B))
    assert max_ulp(np.float32(c["norm"]), np.float32(gn.control(f64)["norm"])) <= 1
    for lo, hi in spans:
        gseg = bits_to_f32(gbits[lo:hi])
        pw, mw, vw = adamw_step_div(p[lo:hi], m0[lo:hi], v0[lo:hi], gseg, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1000,
                                    clip=c["clip_scale"])
        assert max_ulp(_block(s["p32"], lo, hi), pw) == 0, lo
        assert max_ulp(_block(s["m"], lo, hi), mw) == 0 and max_ulp(_block(s["v"], lo, hi), vw) == 0, lo
        assert bits_equal(_block(s["p16"], lo, hi), bf16_sr_bits(pw, sr_seed_base(11, 1000), first_index=lo)), lo
    # every element was updated: the master moved everywhere the gradient or the decay is non-zero
    P = s["p32"].to_numpy().ravel()
    assert np.count_nonzero(P != p) > 0.999 * n
    gdev.free(); guard.free(); opt.free()
