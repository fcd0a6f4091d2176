"""BASELINE config 4 at full size, and the resident MoE model's step call stack.

Config 4: 16 layers alternating dense / MoE at hidden 1024 (dense FFN 3072; MoE layers with 16
experts, gate / up / down each a stacked [16, 1024, 1024] tensor, and a (1024, 16) router), 472 Muon
matrices (416 of them 1024x1024) and 734,565,376 parameters; per MoE layer 4 of the 16 experts have a
zero gradient. One guarded step, built with the benchmark's generator, checked against the oracle.
"""
import numpy as np
import pytest

from oracle import gradnorm_ref as gn
from oracle.adamw_ref import adamw_step_div
from oracle.bf16_ref import bits_to_f32
from oracle.muon_ref import PE_SCHEDULE, muon_momentum, muon_update, ns_any_shape
from util import bits_equal, max_ulp, rel_fro, StubMoELayer

pytestmark = pytest.mark.gpu

LR_MUON, LR_ADAM = 0.02, 3e-4


@pytest.fixture(scope="module")
def c4(gpu):
    import bench
    from ancora_cutile_amd import HybridOptimizer, PE_SCHEDULE as PE
    from ancora_cutile_amd.hybrid import resident_is_muon
    from ancora_cutile_amd.shapes import moe_shapes
    params, grads = bench.synth(moe_shapes(layers=16))
    opt = HybridOptimizer(params, is_muon=resident_is_muon,
                          muon_kw=dict(lr=LR_MUON, momentum=0.95, ns_steps=5, schedule=PE),
                          adamw_kw=dict(lr=LR_ADAM, betas=(0.9, 0.95), eps=1e-8, wd=0.1),
                          max_grad_norm=1.0, grad_dtype=np.uint16)
    opt.step(grads, 0)
    yield dict(params=params, grads=grads, opt=opt, ctl=dict(opt.last_ctl))
    opt.free()


def test_config4_shape_of_the_set_and_norm(c4):
    """472 Muon matrices in three Newton-Schulz shapes, routers and gains on AdamW; one norm over
    every gradient, sum of squares bit-equal to the fixed-order oracle, clip scale bit-equal."""
    opt, grads, ctl = c4["opt"], c4["grads"], c4["ctl"]
    shapes = {}
    for b in opt.muon.engine.batches:
        shapes[(b.M, b.Nn)] = shapes.get((b.M, b.Nn), 0) + b.E
    assert shapes == {(1024, 2048): 32, (1024, 3072): 24, (1024, 1024): 416}
    assert sum(g.size for g in grads.values()) == 734_565_376
    routers = [n for n in opt.adamw_names if "router" in n]
    assert len(routers) == 8 and all(opt.adamw.st[n]["wd"] == 0.0 for n in routers)
    order = opt.muon_names + opt.adamw_names
    fixed = gn.gradnorm_fixed([grads[n] for n in order])
    assert ctl["sumsq"] == fixed and not ctl["skip"]
    assert np.float32(ctl["clip_scale"]) == np.float32(gn.control(fixed)["clip_scale"]) and 0 < ctl["clip_scale"] < 0.01


def test_config4_adamw_group(c4):
    """Every router and every gain: fp32 master 0 ulp from the oracle (routers and gains undecayed);
    the embedding on sampled blocks."""
    opt, params, grads, clip = c4["opt"], c4["params"], c4["grads"], c4["ctl"]["clip_scale"]
    for n in opt.adamw_names:
        p0, g = params[n].ravel(), bits_to_f32(grads[n]).ravel()
        spans = [(0, 16384), (p0.size // 2, p0.size // 2 + 8192), (p0.size - 8192, p0.size)] if n == "embed" else [(0, p0.size)]
        P = opt.adamw.st[n]["p32"].to_numpy().ravel()
        wd = 0.0 if params[n].ndim == 1 or "router" in n else 0.1
        for lo, hi in spans:
            z = np.zeros(hi - lo, np.float32)
            pw, _, _ = adamw_step_div(p0[lo:hi], z, z, g[lo:hi], LR_ADAM, 0.9, 0.95, 1e-8, wd, 1, clip=clip)
            assert max_ulp(P[lo:hi], pw) == 0, (n, lo)


def test_config4_experts_and_dense_weights(c4):
    """Three working experts of each stacked tensor in the first, a middle and the last MoE layer,
    and two weights of each dense shape: momentum buffer bit-equal to the oracle, update direction
    within 2e-3 of the fp32 numpy chain. Idle experts: weights and momentum untouched."""
    opt, params, grads, clip = c4["opt"], c4["params"], c4["grads"], c4["ctl"]["clip_scale"]
    worst = {}

    def check(n, e=None):
        W0 = params[n] if e is None else params[n][e]
        g = bits_to_f32(grads[n]).reshape(params[n].shape)
        g = g if e is None else g[e]
        s = opt.muon.st[n]
        K = s["K"]
        sl = slice(0, None) if e is None else slice(e * K, (e + 1) * K)
        got = s["p32"].to_numpy().reshape(-1, s["N"])[sl]
        buf_got = s["buf"].to_numpy().reshape(-1, s["N"])[sl]
        if not g.any():
            assert bits_equal(got, W0) and not buf_got.any(), (n, e)
            return "idle"
        buf, u = muon_momentum(np.zeros_like(W0), g, clip=clip)
        assert bits_equal(buf_got, buf), (n, e)
        want = muon_update(W0, ns_any_shape(u, PE_SCHEDULE, 5), LR_MUON)
        err = rel_fro(W0.astype(np.float64) - got, W0.astype(np.float64) - want)
        key = n.split(".", 1)[1] + " " + str(W0.shape)
        worst[key] = max(worst.get(key, 0.0), err)
        return "worked"

    for layer in (1, 7, 15):
        for t in ("gate_proj", "up_proj", "down_proj"):
            n = f"layer{layer}.ffn.{t}"
            g = bits_to_f32(grads[n]).reshape(params[n].shape)
            idle = [e for e in range(16) if not g[e].any()]
            assert len(idle) == 4, (n, idle)
            working = [e for e in range(16) if e not in idle]
            for e in idle:
                assert check(n, e) == "idle"
            for e in (working[0], working[len(working) // 2], working[-1]):
                assert check(n, e) == "worked"
    for n in ("layer0.q_proj", "layer14.q_proj", "layer0.k_proj", "layer15.v_proj", "layer0.o_proj", "layer15.o_proj",
              "layer0.gate_proj", "layer14.up_proj", "layer0.down_proj", "layer14.down_proj"):
        assert check(n) == "worked"
    print("\nconfig 4, worst update-direction error per weight kind (bar 2e-3):")
    for k, err in worst.items():
        print(f"  {k:34s} {err:.3e}")
    assert all(err < 2e-3 for err in worst.values()), worst


def test_config4_every_muon_matrix_moved_by_an_orthogonal_update_or_not_at_all(c4):
    """Size-independent property over all 472 matrices: W0 - W1 = lr * scale * O with O
    near-orthogonal has Frobenius norm lr * scale * sqrt(min(K, N)) up to the spread the 5-step
    schedule leaves on the singular values; an idle expert has not moved."""
    opt, params, grads = c4["opt"], c4["params"], c4["grads"]
    seen = idle = 0
    for n, s in opt.muon.st.items():
        K, N = s["K"], s["N"]
        W0 = params[n].reshape(-1, K, N)
        W1 = s["p32"].to_numpy().reshape(-1, K, N)
        G = grads[n].reshape(-1, K, N)
        for e in range(W0.shape[0]):
            d = np.linalg.norm(W0[e].astype(np.float64) - W1[e])
            seen += 1
            if not G[e].any():
                assert d == 0.0, (n, e)
                idle += 1
                continue
            unit = LR_MUON * max(1.0, K / N) ** 0.5 * min(K, N) ** 0.5
            assert 0.6 * unit < d < 1.25 * unit, (n, e, d / unit)
    assert seen == 472 and idle == 8 * 3 * 4


def test_resident_moe_model_step_call_stack_equals_the_hybrid_optimizer(gpu):
    """The resident MoE model's step, piece by piece in the reference's order on one stream
    (ancora/model/resident_moe_model.py:357-374): `BatchedProjMuon.step` over every projection,
    then per layer the norm gains through `_adamw` and, on MoE layers, `GroupedMoEFFN.step` (expert
    Muon through one shared `ExpertMuonScratch`, router `_adamw` with wd = 0), then the tied
    embedding through `_adamw` with wd = 0, then the final norm. Two steps; every master weight and
    every bf16 weight bit-equal to `HybridOptimizer` on the same parameters and gradients (same
    formulas: the kernel form of AdamW, no decay, the process-wide Polar-Express toggle)."""
    from ancora_cutile_amd import (BatchedProjMuon, DevBuf, ExpertMuonScratch, GroupedMoEFFNOptim, HybridOptimizer,
                                   _adamw, _pick_otm, set_polar_express)
    from ancora_cutile_amd.hybrid import resident_is_muon
    from ancora_cutile_amd.bf16 import bf16_bits

    class Layer(StubMoELayer, GroupedMoEFFNOptim):
        pass

    H, E, V, L = 256, 4, 1024, 4
    rng = np.random.default_rng(31)
    proj_shapes = {"q_proj": (H, 2 * H), "k_proj": (H, H), "v_proj": (H, H), "o_proj": (2 * H, H)}
    dense_ffn = {"gate_proj": (H, 3 * H), "up_proj": (H, 3 * H), "down_proj": (3 * H, H)}
    gains = ("input_ln", "post_ln")
    prev = set_polar_express(True)
    try:
        # ---- the model's own buffers
        params, moe_layers = {"embed": (0.02 * rng.standard_normal((V, H))).astype(np.float32)}, {}
        for i in range(L):
            for g in gains:
                params[f"layer{i}.{g}"] = (1 + 0.05 * rng.standard_normal(H)).astype(np.float32)
            for n, s in proj_shapes.items():
                params[f"layer{i}.{n}"] = (0.02 * rng.standard_normal(s)).astype(np.float32)
            if i % 2 == 0:
                for n, s in dense_ffn.items():
                    params[f"layer{i}.{n}"] = (0.02 * rng.standard_normal(s)).astype(np.float32)
            else:
                lay = Layer(E, H, rng, "muon", True)
                moe_layers[i] = lay
                for k in ("gate_proj", "up_proj", "down_proj"):
                    params[f"layer{i}.ffn.{k}"] = lay.w[k]
                params[f"layer{i}.ffn.router"] = lay.w["router"]
        params["final_norm"] = (1 + 0.05 * rng.standard_normal(H)).astype(np.float32)
        steps = [{n: (1e-2 * rng.standard_normal(p.shape)).astype(np.float32) for n, p in params.items()} for _ in range(2)]

        hyb = HybridOptimizer(params, is_muon=resident_is_muon,
                              adamw_kw=dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, wd=0.0, form="ibc"))

        # ---- the call stack's state: projections for BatchedProjMuon, plain AdamW tensors, MoE layers
        scr = ExpertMuonScratch(E, H)
        proj, adam = [], {}
        for n, p in params.items():
            if ".ffn." in n:
                continue
            if p.ndim == 2 and n != "embed":
                K, N = p.shape
                proj.append(dict(name=n, buf=DevBuf.zeros((K, N), np.float32), p32=DevBuf(p), p16=DevBuf(bf16_bits(p)),
                                 G=DevBuf.zeros((K, N), np.float32), K=K, N=N, lid=int(n.split(".")[0][5:])))
            else:
                R = p.size // 64
                adam[n] = dict(R=R, g=DevBuf.zeros((R, 64), np.float32), m=DevBuf.zeros((R, 64), np.float32),
                               v=DevBuf.zeros((R, 64), np.float32), p32=DevBuf(p.reshape(R, 64)),
                               p16=DevBuf.zeros((R, 64), np.uint16))
        bpm = BatchedProjMuon(proj, momentum=0.95, ns_steps=5, chunk=8, scope=2)
        for lay in moe_layers.values():
            lay._muon_scr = scr
            lay.init_adamw(0, betas=(0.9, 0.999), eps=1e-8, wd=0.0)

        def adamw_one(n, t):
            s = adam[n]
            _adamw(0, s["g"], s["m"], s["v"], s["p32"], s["p16"], _pick_otm(s["R"]), 0.9, 0.999, 1e-8, 1e-3, 0.0,
                   1.0 / (1.0 - 0.9 ** t), 1.0 / (1.0 - 0.999 ** t))

        for t, g in enumerate(steps, start=1):
            hyb.step(g, 0)
            # gradients into the model's buffers (what the backward leaves)
            for w in proj:
                w["G"].upload(g[w["name"]])
            for n, s in adam.items():
                s["g"].upload(g[n].reshape(s["R"], 64))
            for i, lay in moe_layers.items():
                for attr, k in (("dWg", "gate_proj"), ("dWu", "up_proj"), ("dWd", "down_proj")):
                    getattr(lay, attr).upload(g[f"layer{i}.ffn.{k}"].reshape(E * H, H))
                lay.Gr_acc.upload(g[f"layer{i}.ffn.router"].reshape(-1))
            # the step, in the reference's order
            bpm.step(0, lr=0.02)
            for i in range(L):
                for gname in gains:
                    adamw_one(f"layer{i}.{gname}", t)
                if i in moe_layers:
                    moe_layers[i].step(0, lr=1e-3, muon_lr=0.02)
            adamw_one("embed", t)
            adamw_one("final_norm", t)
            gpu.stream_sync(0)

        hm, ha = hyb.muon.master(), hyb.adamw.master()
        h16m, h16a = hyb.muon.weights16(), hyb.adamw.weights()
        for w in proj:
            n = w["name"]
            assert bits_equal(w["p32"].to_numpy().reshape(hm[n].shape), hm[n]), n
            assert bits_equal(bits_to_f32(w["p16"].to_numpy()).reshape(hm[n].shape), h16m[n]), n
        for n, s in adam.items():
            assert bits_equal(s["p32"].to_numpy().reshape(ha[n].shape), ha[n]), n
            assert bits_equal(bits_to_f32(s["p16"].to_numpy()).reshape(ha[n].shape), h16a[n]), n
        for i, lay in moe_layers.items():
            for attr, k in (("Wg", "gate_proj"), ("Wu", "up_proj"), ("Wd", "down_proj")):
                n = f"layer{i}.ffn.{k}"
                assert bits_equal(lay._muon[attr]["p32"].to_numpy().reshape(hm[n].shape), hm[n]), n
                assert bits_equal(bits_to_f32(getattr(lay, attr).to_numpy()).reshape(hm[n].shape), h16m[n]), n
            n = f"layer{i}.ffn.router"
            assert bits_equal(lay.Wr_dev.to_numpy().reshape(ha[n].shape), ha[n]), n
        assert scr.nbytes() > 0
        hyb.free(); bpm.free(); scr.free()
        for lay in moe_layers.values():
            lay.free_optim()
    finally:
        set_polar_express(bool(prev))
