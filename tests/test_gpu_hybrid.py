"""End-to-end GPU parity of the hybrid step (Muon on 2-D matrices, AdamW on the rest)."""
import numpy as np
import pytest

from oracle.adamw_ref import AdamWRef
from oracle.muon_ref import MuonRef, PE_SCHEDULE
from oracle.bf16_ref import bf16_rne_bits, bits_to_f32
from oracle import gradnorm_ref as gn
from util import max_ulp, rel_fro, bits_equal, bf16_grad, StubMoELayer as _StubMoELayer

pytestmark = pytest.mark.gpu


def test_config1_minimal_hybrid_step(gpu):
    """BASELINE config 1: AdamW on a 1024x1024 weight (routed by name) + a 1024 gain, Muon on a
    1024x1024 weight; bf16 grads ~N(0,1e-3); 5 Polar-Express iterations; seed 0; step 1."""
    from ancora_cutile_amd import HybridOptimizer, PE_SCHEDULE as PE
    rng = np.random.default_rng(0)
    params = {"embed": (0.02 * rng.standard_normal((1024, 1024))).astype(np.float32),
              "final_norm": (1 + 0.05 * rng.standard_normal(1024)).astype(np.float32),
              "layer0.q_proj": (0.02 * rng.standard_normal((1024, 1024))).astype(np.float32)}
    gb, g = {}, {}
    for n, p in params.items():
        gb[n], g[n] = bf16_grad(rng, p.shape, 1e-3)
    opt = HybridOptimizer(params, muon_kw=dict(schedule=PE),
                          adamw_kw=dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1),
                          grad_dtype=np.uint16)
    assert opt.routing() == {"muon": ["layer0.q_proj"], "adamw": ["embed", "final_norm"]}
    opt.step(gb, 0)
    ar = AdamWRef({n: params[n] for n in ("embed", "final_norm")}, lr=3e-4, betas=(0.9, 0.95),
                  eps=1e-8, wd=0.1, no_decay=("final_norm",))
    ar.step(g)
    mr = MuonRef({"layer0.q_proj": params["layer0.q_proj"]}, lr=0.02, momentum=0.95, sched=PE_SCHEDULE)
    mr.step(g)
    am = opt.adamw.master()
    for n in ("embed", "final_norm"):
        assert max_ulp(am[n], ar.st[n]["p"]) == 0
    mm = opt.muon.master()["layer0.q_proj"]
    # the update direction (W0 - W1)/lr is the orthogonalised momentum: 2e-3 bar
    upd_got = (params["layer0.q_proj"].astype(np.float64) - mm) / 0.02
    upd_ref = (params["layer0.q_proj"].astype(np.float64) - mr.w["layer0.q_proj"]) / 0.02
    assert rel_fro(upd_got, upd_ref) < 2e-3
    assert bits_equal(opt.muon.momentum_buffers()["layer0.q_proj"], mr.buf["layer0.q_proj"])
    w = opt.weights()
    assert np.array_equal(w["embed"], bits_to_f32(bf16_rne_bits(am["embed"])).reshape(1024, 1024))
    opt.free()


def test_guarded_step_clips_and_skips(gpu):
    from ancora_cutile_amd import HybridOptimizer
    rng = np.random.default_rng(1)
    params = {"embed": rng.standard_normal((128, 64)).astype(np.float32),
              "norm": np.ones(64, np.float32),
              "l0.up_proj": (0.02 * rng.standard_normal((128, 256))).astype(np.float32),
              "l0.down_proj": (0.02 * rng.standard_normal((256, 128))).astype(np.float32)}
    grads = {n: rng.standard_normal(p.shape).astype(np.float32) for n, p in params.items()}
    opt = HybridOptimizer(params, max_grad_norm=1.0)
    opt.step(grads, 0)
    assert not opt.last_skipped and 0 < opt.last_ctl["clip_scale"] < 1
    want = np.sqrt(sum(float(np.sum(g.astype(np.float64) ** 2)) for g in grads.values()))
    assert abs(opt.last_ctl["norm"] - want) / want < 1e-6
    snap = (opt.muon.master(), opt.adamw.master(), opt.muon.momentum_buffers())
    bad = {n: g.copy() for n, g in grads.items()}
    bad["l0.up_proj"][5, 5] = np.nan
    opt.step(bad, 0)
    assert opt.last_skipped and opt.adamw.t == 1 and opt.muon.engine.t == 1
    now = (opt.muon.master(), opt.adamw.master(), opt.muon.momentum_buffers())
    for a, b in zip(snap, now):
        for n in a:
            assert bits_equal(a[n], b[n])
    opt.free()


def test_descent_on_quadratic(gpu):
    """The pattern of tests/kernels/_probe_device_muon.py:72-101: Muon steps on 0.5*||W-T||^2
    drive the loss below 20% of its start, on square, wide and tall weights."""
    from ancora_cutile_amd import Muon, PE_SCHEDULE as PE
    rng = np.random.default_rng(2)
    shapes = {"a": (128, 128), "b": (128, 256), "c": (256, 128)}
    W = {n: (0.05 * rng.standard_normal(s)).astype(np.float32) for n, s in shapes.items()}
    T = {n: (0.05 * rng.standard_normal(s)).astype(np.float32) for n, s in shapes.items()}
    opt = Muon(W, lr=0.05, schedule=PE)
    host = MuonRef(W, lr=0.05, sched=PE_SCHEDULE)
    loss0 = {n: 0.5 * float(np.sum((W[n] - T[n]) ** 2)) for n in W}
    for _ in range(40):
        cur = opt.master()
        opt.step({n: cur[n] - T[n] for n in W}, 0)
        host.step({n: host.w[n] - T[n] for n in W})
    cur = opt.master()
    for n in W:
        drop_d = 0.5 * float(np.sum((cur[n] - T[n]) ** 2)) / loss0[n]
        drop_h = 0.5 * float(np.sum((host.w[n] - T[n]) ** 2)) / loss0[n]
        assert drop_d < 0.2 and drop_d < 3 * drop_h + 0.05     # _probe_device_muon.py:97
    opt.free()


def test_chunk_and_scope_are_bitwise_neutral(gpu):
    """tests/training/test_batched_proj_muon.py:74: per-layer buckets == global batches, bitwise."""
    from ancora_cutile_amd import BatchedProjMuon, DevBuf, PE_SCHEDULE as PE
    rng = np.random.default_rng(3)
    shapes = [(128, 128), (128, 256), (256, 128), (128, 128), (256, 128), (128, 256), (128, 128)]
    W0 = [(0.02 * rng.standard_normal(s)).astype(np.float32) for s in shapes]
    G = [rng.standard_normal(s).astype(np.float32) for s in shapes]

    def run(**kw):
        ws = [dict(buf=DevBuf.zeros(s, np.float32), p32=DevBuf(w), p16=DevBuf.zeros(s, np.uint16),
                   G=DevBuf(g), K=s[0], N=s[1], lid=i // 2) for i, (s, w, g) in enumerate(zip(shapes, W0, G))]
        opt = BatchedProjMuon(ws, **kw)
        for _ in range(2):
            opt.step(0, lr=0.02, schedule=PE)
        out = [(w["p32"].to_numpy(), w["p16"].to_numpy(), w["buf"].to_numpy()) for w in ws]
        opt.free()
        for w in ws:
            for k in ("buf", "p32", "p16", "G"):
                w[k].free()
        return out

    base = run(chunk=8)
    for kw in (dict(chunk=1), dict(chunk=2, scope=1), dict(chunk=None, scope=2)):
        other = run(**kw)
        for a, b in zip(base, other):
            for x, y in zip(a, b):
                assert bits_equal(x, y)


def test_weights_do_not_depend_on_what_shares_the_grouped_step(gpu):
    """A 1024x1024 weight (residual terms in its chain; its B operand is fetched by rows) stepped
    together with smaller shapes in one grouped, fused-update Muon step gets the bits it gets
    when stepped alone, and so do the others."""
    from ancora_cutile_amd import Muon, PE_SCHEDULE as PE
    rng = np.random.default_rng(8)
    shapes = {"a": (1024, 1024), "b": (512, 768), "c": (256, 256), "d": (768, 512)}
    W = {n: (0.02 * rng.standard_normal(s)).astype(np.float32) for n, s in shapes.items()}
    G = [{n: rng.standard_normal(s).astype(np.float32) for n, s in shapes.items()} for _ in range(2)]

    def run(names):
        opt = Muon({n: W[n] for n in names}, lr=0.02, momentum=0.95, ns_steps=5, schedule=PE)
        for g in G:
            opt.step({n: g[n] for n in names}, 0)
        out = opt.master()
        opt.free()
        return out

    together = run(list(shapes))
    for n in shapes:
        assert bits_equal(run([n])[n], together[n]), n


@pytest.mark.parametrize("Ie", [128, 256])
def test_expert_optimizer(gpu, Ie):
    """Stacked [E,K,N] experts: Muon per slice, idle experts (zero grad) leave their weights
    unchanged at step 1, router on AdamW with wd=0, transposed copies refreshed (wide
    gate/up and tall down projections when Ie != H)."""
    from ancora_cutile_amd import ExpertOptimizer, DevBuf, PE_SCHEDULE as PE
    from oracle.muon_ref import muon_momentum, ns_any_shape, muon_update, shape_scale
    rng = np.random.default_rng(4)
    E, H = 4, 128
    shp = {"gate_proj": (H, Ie), "up_proj": (H, Ie), "down_proj": (Ie, H)}
    W = {n: (0.02 * rng.standard_normal((E,) + kn)).astype(np.float32) for n, kn in shp.items()}
    router = (0.02 * rng.standard_normal((H, 16))).astype(np.float32)
    G = {n: rng.standard_normal(W[n].shape).astype(np.float32) for n in W}
    for n in G:
        G[n][2] = 0
    Gd = {n: DevBuf(g.reshape(E * shp[n][0], shp[n][1])) for n, g in G.items()}
    rg = rng.standard_normal((H, 16)).astype(np.float32)
    rgd = DevBuf(rg.reshape(-1, 64))
    opt = ExpertOptimizer(W, router)
    opt.step(Gd, 0, lr=1e-3, muon_lr=0.02, router_grad=rgd, schedule=PE)
    m = opt.master()
    for n in W:
        K, N = shp[n]
        assert bits_equal(m[n][2], W[n][2])                       # idle expert untouched
        _, u = muon_momentum(np.zeros((K, N), np.float32), G[n][0])
        want = muon_update(W[n][0], ns_any_shape(u, PE_SCHEDULE, 5), 0.02)
        step = 0.02 * shape_scale(K, N)
        assert rel_fro((W[n][0] - m[n][0]) / step, (W[n][0] - want) / step) < 2e-3
        s = opt.st[n]
        p16 = s["p16"].to_numpy().reshape(E, K, N)
        assert np.array_equal(s["p16T"].to_numpy().reshape(E, N, K), p16.transpose(0, 2, 1))
        assert bits_equal(p16, bf16_rne_bits(m[n]).reshape(E, K, N))
    assert not np.array_equal(m["router"], router)
    for b in list(Gd.values()) + [rgd]:
        b.free()
    opt.free()


def test_checkpoint_resume_is_bitwise(gpu, tmp_path):
    """save() after two steps, load() into a fresh optimizer, two more steps on both: masters,
    moments, momentum and bf16 weights agree bit for bit (stochastic rounding included: the step
    counters travel with the state)."""
    from ancora_cutile_amd import HybridOptimizer, PE_SCHEDULE
    rng = np.random.default_rng(5)
    params = {"embed": (0.02 * rng.standard_normal((256, 128))).astype(np.float32),
              "final_norm": np.ones(128, np.float32),
              "layer0.q_proj": (0.02 * rng.standard_normal((128, 256))).astype(np.float32),
              "layer0.down_proj": (0.02 * rng.standard_normal((384, 128))).astype(np.float32)}
    grads = [{n: (1e-2 * rng.standard_normal(p.shape)).astype(np.float32) for n, p in params.items()}
             for _ in range(4)]
    kw = dict(muon_kw=dict(schedule=PE_SCHEDULE, sr=True, seed=3), max_grad_norm=1.0,
              adamw_kw=dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=True, seed=9))
    a = HybridOptimizer(params, **kw)
    for g in grads[:2]:
        a.step(g, 0)
    path = str(tmp_path / "opt")              # no extension: save and load agree on "opt.npz"
    a.save(path)
    for g in grads[2:]:
        a.step(g, 0)
    b = HybridOptimizer(params, **kw)
    b.load(path)
    for g in grads[2:]:
        b.step(g, 0)
    sa, sb = a.state_dict(), b.state_dict()
    assert sa.keys() == sb.keys()
    for k in sa:
        assert np.atleast_1d(sa[k]).tobytes() == np.atleast_1d(sb[k]).tobytes(), k
    a.free(); b.free()


def test_default_predicate_with_a_misaligned_router(gpu):
    """`HybridOptimizer(model.params())` on a MoE parameter set with the default predicate
    (tests/training/test_moe_pipeline.py:36): the (H, E) router is 2-D, so the predicate names it
    for Muon, but it is not 128-aligned. The reference keeps it on Muon with Newton-Schulz on the
    host (ancora/optim/muon.py:37-41, 307); here it stays on Muon too, zero-padded through the
    device chain: its master weights follow the numpy Muon (Keller, the default) over three steps,
    the padding never leaks into what the accessors return, and it saves and reloads."""
    from ancora_cutile_amd import HybridOptimizer
    rng = np.random.default_rng(8)
    params = {"embed": (0.02 * rng.standard_normal((256, 128))).astype(np.float32),
              "layer1.ffn.router": (0.02 * rng.standard_normal((128, 16))).astype(np.float32),
              "layer1.ffn.gate_proj": (0.02 * rng.standard_normal((4, 128, 128))).astype(np.float32),
              "layer1.q_proj": (0.02 * rng.standard_normal((128, 256))).astype(np.float32)}
    opt = HybridOptimizer(params)
    assert opt.routing() == {"muon": ["layer1.ffn.router", "layer1.q_proj"],
                             "adamw": ["embed", "layer1.ffn.gate_proj"]}
    assert opt.muon_padded == ["layer1.ffn.router"]
    mr = MuonRef({n: params[n] for n in opt.muon_names})
    for step in range(3):
        grads = {n: (1e-2 * rng.standard_normal(p.shape)).astype(np.float32) for n, p in params.items()}
        opt.step(grads, 0)
        mr.step(grads)
    got = opt.muon.master()
    for n in opt.muon_names:
        assert got[n].shape == params[n].shape
        d = np.linalg.norm(got[n].astype(np.float64) - mr.w[n]) / np.linalg.norm(params[n] - mr.w[n])
        assert d < 2e-3, (n, d)
    # the shape factor is that of the router's own dims: sqrt(128 / 16), not of the padded ones
    upd = np.linalg.norm(params["layer1.ffn.router"] - got["layer1.ffn.router"])
    assert upd > 0.02 * (128 / 16) ** 0.5 * 3 * 0.5
    # padding rows and columns of the stored state stay exactly zero
    full = opt.muon.st["layer1.ffn.router"]["p32"].to_numpy().reshape(128, 128)
    assert not full[:, 16:].any()
    assert opt.muon.weights()["layer1.ffn.router"].shape == (128, 16)
    assert opt.muon.momentum_buffers()["layer1.ffn.router"].shape == (128, 16)
    opt.free()


def test_router_left_to_adamw_is_not_decayed(gpu):
    """Under the resident routing the router is an AdamW tensor, and the resident models run it
    with wd = 0 (ancora/kernels/moe.py:603-604): the default `no_decay` exempts it like the gains."""
    from ancora_cutile_amd import HybridOptimizer, resident_is_muon
    rng = np.random.default_rng(9)
    params = {"layer1.ffn.router": (0.02 * rng.standard_normal((128, 16))).astype(np.float32),
              "layer1.post_ln": (1 + 0.05 * rng.standard_normal(128)).astype(np.float32),
              "layer1.q_proj": (0.02 * rng.standard_normal((128, 256))).astype(np.float32)}
    opt = HybridOptimizer(params, is_muon=resident_is_muon)
    assert opt.routing() == {"muon": ["layer1.q_proj"], "adamw": ["layer1.ffn.router", "layer1.post_ln"]}
    assert opt.adamw.st["layer1.ffn.router"]["wd"] == 0.0 and opt.adamw.st["layer1.post_ln"]["wd"] == 0.0
    grads = {n: (1e-2 * rng.standard_normal(p.shape)).astype(np.float32) for n, p in params.items()}
    opt.step(grads, 0)
    ar = AdamWRef({n: params[n] for n in opt.adamw_names}, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.01,
                  no_decay=tuple(opt.adamw_names))
    ar.step(grads)
    assert max_ulp(opt.adamw.master()["layer1.ffn.router"], ar.st["layer1.ffn.router"]["p"]) == 0
    opt.free()


def test_unsynchronised_guarded_steps_equal_the_synchronous_ones(gpu, monkeypatch):
    """`step(..., sync=False)`: six guarded steps with resident bf16 gradients, the second and the
    fifth with a non-finite gradient, issued without a single host synchronisation (every
    synchronising library call is counted), as the reference's resident step is
    (ancora/model/resident_train.py:338-339). The steps are counted on the device, so a skipped
    step needs no undo: every state tensor equals, bit for bit, the state after the same six
    synchronous steps, the step count is 4, and the AdamW master weights equal the numpy oracle's
    after its four steps (bias corrections of steps 1..4, rounding seeds of steps 1..4)."""
    from ancora_cutile_amd import HybridOptimizer, DevBuf, PE_SCHEDULE, resident_is_muon, _lib
    rng = np.random.default_rng(21)
    params = {"embed": (0.02 * rng.standard_normal((512, 256))).astype(np.float32),
              "final_norm": (1 + 0.05 * rng.standard_normal(256)).astype(np.float32),
              "layer0.q_proj": (0.02 * rng.standard_normal((256, 512))).astype(np.float32),
              "layer0.o_proj": (0.02 * rng.standard_normal((512, 256))).astype(np.float32)}
    steps = []
    for t in range(6):
        g = {n: bf16_rne_bits((1e-2 * rng.standard_normal(p.shape)).astype(np.float32)).reshape(p.shape)
             for n, p in params.items()}
        if t in (1, 4):
            g["embed"] = g["embed"].copy()
            g["embed"][3, 5] = 0x7FC0 if t == 1 else 0x7F80          # NaN, +Inf
        steps.append(g)
    kw = dict(is_muon=resident_is_muon, muon_kw=dict(schedule=PE_SCHEDULE, sr=True, seed=5),
              adamw_kw=dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=True, seed=7),
              max_grad_norm=1.0, grad_dtype=np.uint16)

    def run(sync):
        opt = HybridOptimizer(params, **kw)
        bufs = [{n: DevBuf(g[n]) for n in params} for g in steps]       # resident before the steps
        _lib.stream_sync(0)
        calls = {"n": 0}
        names = ("anc_stream_sync", "anc_device_sync", "anc_memcpy_d2h", "anc_memcpy_h2d", "anc_event_sync")
        if not sync:
            for name in names:
                real = getattr(_lib.api, name)
                monkeypatch.setattr(_lib.api, name, (lambda real: lambda *a: (calls.__setitem__("n", calls["n"] + 1), real(*a))[1])(real))
        # one set of gradient buffers for every step, as in a training loop (the descriptor tables
        # are built for them once, at the first step); each step's gradient arrives by an
        # asynchronous device copy on the step's stream
        cur = {n: DevBuf(steps[0][n]) for n in params}
        opt.step(cur, 0)                   # first step: descriptor and step tables are uploaded here
        calls["n"] = 0
        skipped = []
        for b in bufs[1:]:
            for n in params:
                _lib.api.anc_memcpy_d2d(cur[n].ptr, b[n].ptr, cur[n].nbytes, 0)
            opt.step(cur, 0, sync=sync)
            if sync:
                skipped.append(opt.last_skipped)
        n_sync = calls["n"]
        monkeypatch.undo()
        state = opt.state_dict()
        out = dict(state=state, t=opt.step_count(), skipped=skipped, n_sync=n_sync, last=dict(opt.last_ctl),
                   adamw=opt.adamw.master(), at=opt.adamw.t, mt=opt.muon.engine.t)
        opt.free()
        for b in bufs + [cur]:
            for d in b.values():
                d.free()
        return out

    a, b = run(True), run(False)
    assert a["skipped"] == [True, False, False, True, False]
    assert b["n_sync"] == 0, "an unsynchronised step called a synchronising entry point"
    assert a["t"] == b["t"] == 4 and a["at"] == b["at"] == 4 and a["mt"] == b["mt"] == 4
    assert a["state"].keys() == b["state"].keys()
    for k in a["state"]:
        assert np.atleast_1d(a["state"][k]).tobytes() == np.atleast_1d(b["state"][k]).tobytes(), k
    assert a["last"] == b["last"] and not b["last"]["skip"]
    # the oracle takes the four finite steps
    ar = AdamWRef({n: params[n] for n in ("embed", "final_norm")}, lr=3e-3, betas=(0.9, 0.95), eps=1e-8,
                  wd=0.1, no_decay=("final_norm",))
    order = ["layer0.q_proj", "layer0.o_proj", "embed", "final_norm"]
    for t, g in enumerate(steps):
        if t in (1, 4):
            continue
        gf = {n: bits_to_f32(g[n]).reshape(g[n].shape) for n in g}
        ar.step(gf, clip=gn.control(gn.gradnorm_fixed([g[n] for n in order]), 1.0, 1e-6)["clip_scale"])
    for n in ("embed", "final_norm"):
        assert max_ulp(b["adamw"][n], ar.st[n]["p"]) == 0, n


@pytest.mark.parametrize("sr", [False, True])
def test_fused_update_equals_separate_update_kernel(gpu, sr):
    """The chain whose last epilogue applies W -= lr*O gives the bits of the chain followed by the
    update kernel: square, wide and tall (transposed) weights, with and without a bf16 copy,
    RNE and stochastic rounding, two steps, and a skipped step leaves everything untouched."""
    from ancora_cutile_amd import BatchedProjMuon, DevBuf, StepGuard, PE_SCHEDULE as PE
    rng = np.random.default_rng(21)
    shapes = [(256, 256), (256, 512), (512, 256), (256, 256), (768, 256), (256, 512), (512, 256)]
    W0 = [(0.02 * rng.standard_normal(s)).astype(np.float32) for s in shapes]
    G = [rng.standard_normal(s).astype(np.float32) for s in shapes]

    def run(fused, skip_second=False, shared=False):
        ws = [dict(buf=DevBuf.zeros(s, np.float32), p32=DevBuf(w),
                   p16=None if i == 3 else DevBuf.zeros(s, np.uint16),
                   G=DevBuf(g), K=s[0], N=s[1], lid=i) for i, (s, w, g) in enumerate(zip(shapes, W0, G))]
        opt = BatchedProjMuon(ws, chunk=None, sr=sr, seed=5)
        if shared:       # one packed buffer and workspace for all batches: one batch per call
            from ancora_cutile_amd.muon import MuonEngine
            opt.engine.free()
            opt.engine = MuonEngine(ws, 0.95, 5, True, None, None, "bf16", sr, 5, concurrent=False)
        opt.engine.fused_update = fused
        guard = StepGuard(1e9)
        grads = [w["G"] for w in ws]
        for t in range(2):
            if skip_second and t == 1:
                bad = G[0].copy(); bad[3, 7] = np.inf
                ws[0]["G"].upload(bad)
            guard.compute(grads, 0)
            opt.step(0, lr=0.02, schedule=PE, guard=guard)
        out = [(w["p32"].to_numpy(), None if w["p16"] is None else w["p16"].to_numpy(), w["buf"].to_numpy())
               for w in ws]
        opt.free(); guard.free()
        for w in ws:
            for k in ("buf", "p32", "p16", "G"):
                if w[k] is not None:
                    w[k].free()
        return out

    for skip in (False, True):
        a, b = run(True, skip), run(False, skip)
        for x, y in zip(a, b):
            for u, v in zip(x, y):
                assert (u is None and v is None) or bits_equal(u, v)
    a, b = run(True, shared=True), run(False)
    for x, y in zip(a, b):
        for u, v in zip(x, y):
            assert (u is None and v is None) or bits_equal(u, v)
    one = run(True, True)
    # the skipped second step changed nothing: equal to a single step
    from ancora_cutile_amd import BatchedProjMuon as BPM
    ws = [dict(buf=DevBuf.zeros(s, np.float32), p32=DevBuf(w), p16=None if i == 3 else DevBuf.zeros(s, np.uint16),
               G=DevBuf(g), K=s[0], N=s[1], lid=i) for i, (s, w, g) in enumerate(zip(shapes, W0, G))]
    opt = BPM(ws, chunk=None, sr=sr, seed=5)
    opt.step(0, lr=0.02, schedule=PE)
    for w, o in zip(ws, one):
        assert bits_equal(w["p32"].to_numpy(), o[0])
    opt.free()
    for w in ws:
        for k in ("buf", "p32", "p16", "G"):
            if w[k] is not None:
                w[k].free()


@pytest.mark.parametrize("optimizer", ["muon", "adamw"])
@pytest.mark.parametrize("device_route", [True, False])
def test_grouped_moe_ffn_optimizer_methods(gpu, optimizer, device_route):
    """`init_adamw` / `step` under the reference's names (ancora/kernels/moe.py:525-609) on a layer
    object's own buffers: experts bit-equal to `ExpertOptimizer` on the same data, the bf16 forward
    weights updated in place, their transposes refreshed, the router against the oracle."""
    from ancora_cutile_amd import DevBuf, GroupedMoEFFNOptim, ExpertOptimizer
    from oracle.adamw_ref import adamw_step_ibc

    class Layer(_StubMoELayer, GroupedMoEFFNOptim):
        pass

    E, H = 4, 256
    rng = np.random.default_rng(21)
    layer = Layer(E, H, rng, optimizer, device_route)
    layer.init_adamw(0, betas=(0.9, 0.999), eps=1e-8, wd=0.01)
    ref = ExpertOptimizer({k: layer.w[k] for k in ExpertOptimizer.NAMES}, router=None, optimizer=optimizer,
                          betas=(0.9, 0.999), eps=1e-8, wd=0.01)
    router0 = layer.w["router"].copy()
    rm = np.zeros_like(router0); rv = np.zeros_like(router0); rw = router0.copy()
    names = (("Wg", "gate_proj"), ("Wu", "up_proj"), ("Wd", "down_proj"))
    for t in (1, 2):
        g = {key: (1e-2 * rng.standard_normal((E * H, H))).astype(np.float32) for _, key in names}
        gr = (1e-2 * rng.standard_normal((H, E))).astype(np.float32)
        gdev = {}
        for attr, key in names:
            getattr(layer, "d" + attr).upload(g[key])
            gdev[key] = DevBuf(g[key])
        layer.Gr_acc.upload(gr.reshape(-1))
        layer.G_router = gr
        layer.step(0, lr=1e-3)
        ref.step(gdev, 0, lr=1e-3, muon_lr=0.02)
        gpu.stream_sync(0)
        assert layer._wq_dirty_mx and layer._t == t
        rw, rm, rv = adamw_step_ibc(rw, rm, rv, gr, 1e-3, 0.9, 0.999, 1e-8, 0.0 if device_route else 0.01,
                                    1.0 / (1.0 - 0.9 ** t), 1.0 / (1.0 - 0.999 ** t))
        for b in gdev.values():
            b.free()
    state = layer._muon if optimizer == "muon" else layer._eopt
    for attr, key in names:
        want = ref.st[key]
        assert bits_equal(state[attr]["p32"].to_numpy().ravel(), want["p32"].to_numpy().ravel()), attr
        p16 = getattr(layer, attr).to_numpy()
        assert bits_equal(p16.ravel(), want["p16"].to_numpy().ravel()), attr          # forward weights, in place
        p16T = getattr(layer, attr + "T").to_numpy().reshape(E, H, H)
        assert all(bits_equal(p16T[e], np.ascontiguousarray(p16.reshape(E, H, H)[e].T)) for e in range(E)), attr
    if device_route:
        assert max_ulp(layer.Wr_dev.to_numpy().reshape(H, E), rw) <= 1
        assert bits_equal(layer.G_router_dev.to_numpy(), layer.Gr_acc.to_numpy())
    else:
        assert np.abs(layer.w["router"] - rw).max() < 1e-7
    layer.free_optim(); ref.free()


def test_wide_spectrum_gradients_through_the_grouped_step(gpu):
    """Gradients whose spectrum spans three decades (wide and tall weights), beside Gaussian ones of the
    same shapes, through the grouped Muon step with the update fused into the chain's last
    product: the wide gate's terms run for the matrices in its band only, the update direction
    meets the 2e-3 bar for every weight (the reference's chain sits at 5e-3 .. 7e-3 on such
    inputs), and a weight's new bits do not depend on which other weights share the step."""
    from ancora_cutile_amd import Muon, PE_SCHEDULE as PE

    def wide(rng, K, N):
        m, n = min(K, N), max(K, N)
        U, _ = np.linalg.qr(rng.standard_normal((m, m)))
        V, _ = np.linalg.qr(rng.standard_normal((n, m)))
        X = ((U * np.exp(rng.uniform(0, np.log(1e3), m))) @ V.T).astype(np.float32)
        X *= np.float32(1e-3 / X.std())
        return X if K <= N else np.ascontiguousarray(X.T)

    rng = np.random.default_rng(21)
    shapes = {"l0.q_proj": (1024, 2048), "l0.o_proj": (2048, 1024), "l0.k_proj": (1024, 1024),
              "l1.q_proj": (1024, 2048), "l1.k_proj": (1024, 1024)}
    params = {n: (0.02 * rng.standard_normal(s)).astype(np.float32) for n, s in shapes.items()}
    grads = {n: (wide(rng, *s) if n.startswith("l0.") else (1e-3 * rng.standard_normal(s)).astype(np.float32))
             for n, s in shapes.items()}
    opt = Muon(params, lr=0.02, schedule=PE)
    opt.step(grads, 0)
    got = opt.master()
    ref = MuonRef(params, lr=0.02, momentum=0.95, sched=PE_SCHEDULE)
    ref.step(grads)
    for n, (K, N) in shapes.items():
        scale = 0.02 * max(1.0, K / N) ** 0.5
        d_got = (params[n].astype(np.float64) - got[n]) / scale
        d_ref = (params[n].astype(np.float64) - ref.w[n]) / scale
        err = rel_fro(d_got, d_ref)
        print(n, f"{err:.3e}")
        assert err < (1e-3 if n.startswith("l0.") else 2e-3), n
    opt.free()
    alone = Muon({"l0.q_proj": params["l0.q_proj"]}, lr=0.02, schedule=PE)
    alone.step({"l0.q_proj": grads["l0.q_proj"]}, 0)
    assert bits_equal(alone.master()["l0.q_proj"], got["l0.q_proj"])
    alone.free()
