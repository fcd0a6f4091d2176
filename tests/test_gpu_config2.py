"""BASELINE config 2 at full size: one guarded hybrid step over the Qwen3-0.6B-shaped parameter set
(596,049,920 parameters; bf16 gradients ~N(0,1e-3) with 1 % of the rows of every matrix scaled
x100; global grad-norm clip at 1.0; stochastic bf16 weight downcast; 5 Polar-Express iterations),
built with the benchmark's own generator, checked against the numpy oracle.

The outlier rows make every Newton-Schulz input ill-conditioned: ten to thirty rows carry ~99 % of
the Frobenius norm. Weights that keep their orientation (q, k, v, gate, up) see them as rows of the
iterate, tall weights (o, down), which enter the chain transposed, as columns.
"""
import numpy as np
import pytest

from oracle import gradnorm_ref as gn
from oracle.adamw_ref import adamw_step_div
from oracle.bf16_ref import bf16_sr_bits, bits_to_f32
from oracle.muon_ref import PE_SCHEDULE, muon_momentum, muon_update, ns_any_shape
from util import bits_equal, max_ulp, rel_fro

pytestmark = pytest.mark.gpu

LR_MUON, LR_ADAM = 0.02, 3e-4
MUON_SEED, ADAM_SEED = 1, 2


@pytest.fixture(scope="module")
def c2(gpu):
    import bench
    from ancora_cutile_amd import HybridOptimizer, PE_SCHEDULE as PE
    from ancora_cutile_amd.hybrid import resident_is_muon
    from ancora_cutile_amd.shapes import qwen3_shapes
    params, grads = bench.synth(qwen3_shapes())
    opt = HybridOptimizer(params, is_muon=resident_is_muon,
                          muon_kw=dict(lr=LR_MUON, momentum=0.95, ns_steps=5, schedule=PE, sr=True, seed=MUON_SEED),
                          adamw_kw=dict(lr=LR_ADAM, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=True, seed=ADAM_SEED),
                          max_grad_norm=1.0, grad_dtype=np.uint16)
    opt.step(grads, 0)
    yield dict(params=params, grads=grads, opt=opt, ctl=dict(opt.last_ctl))
    opt.free()


def test_config2_norm_and_clip(c2):
    """One norm over all 310 gradients: sum of squares bit-equal to the fixed-order oracle, norm
    within 1 ulp of the fp64 closed form, clip scale bit-equal to min(1, 1/(norm + eps))."""
    opt, grads, ctl = c2["opt"], c2["grads"], c2["ctl"]
    order = opt.muon_names + opt.adamw_names
    assert len(order) == 310 and sum(grads[n].size for n in order) == 596_049_920
    assert not ctl["skip"] and not opt.last_skipped
    fixed = gn.gradnorm_fixed([grads[n] for n in order])
    assert ctl["sumsq"] == fixed
    closed = gn.control(gn.gradnorm_f64([grads[n] for n in order]))
    assert max_ulp(np.float32(ctl["norm"]), np.float32(closed["norm"])) <= 1
    want = gn.control(fixed)
    assert np.float32(ctl["clip_scale"]) == np.float32(want["clip_scale"]) and 0 < ctl["clip_scale"] < 0.01
    assert opt.adamw.t == 1 and opt.muon.engine.t == 1


def test_config2_adamw_group(c2):
    """Embedding (sampled blocks, first / outlier-row / last) and every gain: m, v and the fp32
    master 0 ulp from the oracle, bf16 weights bit-equal to the stochastic rounding of the master."""
    from ancora_cutile_amd.adamw import sr_seed_base
    opt, params, grads, clip = c2["opt"], c2["params"], c2["grads"], c2["ctl"]["clip_scale"]
    sb = sr_seed_base(ADAM_SEED, 1)
    names = list(opt.adamw.st)
    assert names == opt.adamw_names and names[0] == "embed" and len(names) == 114
    for ti, n in enumerate(names):
        s = opt.adamw.st[n]
        p0, g = params[n].ravel(), bits_to_f32(grads[n]).ravel()
        size = p0.size
        if n == "embed":
            hot = int(np.argmax(np.abs(g)))                    # inside one of the x100 rows
            spans = [(0, 16384), (hot // 64 * 64 - 4096, hot // 64 * 64 + 4096), (size // 2 + 4096 * 5, size // 2 + 4096 * 7),
                     (size - 8192, size)]
        else:
            spans = [(0, size)]
        P, M_, V, P16 = (s[k].to_numpy().ravel() for k in ("p32", "m", "v", "p16"))
        wd = 0.0 if params[n].ndim == 1 else 0.1
        for lo, hi in spans:
            z = np.zeros(hi - lo, np.float32)
            pw, mw, vw = adamw_step_div(p0[lo:hi], z, z, g[lo:hi], LR_ADAM, 0.9, 0.95, 1e-8, wd, 1, clip=clip)
            assert max_ulp(P[lo:hi], pw) == 0 and max_ulp(M_[lo:hi], mw) == 0 and max_ulp(V[lo:hi], vw) == 0, (n, lo)
            assert bits_equal(P16[lo:hi], bf16_sr_bits(pw, (sb + ti) & 0xFFFFFFFF, first_index=lo)), (n, lo)


SHAPE_SAMPLES = {
    "q_proj (1024,2048)": ["layer0.q_proj", "layer27.q_proj"],
    "k/v_proj (1024,1024)": ["layer0.k_proj", "layer13.v_proj", "layer27.k_proj"],
    "o_proj (2048,1024) tall": ["layer0.o_proj", "layer27.o_proj"],
    "gate/up_proj (1024,3072)": ["layer0.gate_proj", "layer14.up_proj", "layer27.gate_proj"],
    "down_proj (3072,1024) tall": ["layer0.down_proj", "layer13.down_proj", "layer27.down_proj"],
}


def test_config2_muon_group(c2):
    """Per Muon shape, two or three weights from the first, a middle and the last layer: momentum
    buffer bit-equal to the oracle, update direction (W0 - W1) within 2e-3 (relative Frobenius) of
    momentum -> fp32 Polar-Express chain -> update in numpy, bf16 weights bit-equal to the
    stochastic rounding of the master the GPU holds."""
    from ancora_cutile_amd.adamw import sr_seed_base
    opt, params, grads, clip = c2["opt"], c2["params"], c2["grads"], c2["ctl"]["clip_scale"]
    sb = sr_seed_base(MUON_SEED, 1)
    index = {n: i for i, n in enumerate(opt.muon.st)}
    assert len(index) == 196
    worst = {}
    for shape, names in SHAPE_SAMPLES.items():
        for n in names:
            s = opt.muon.st[n]
            W0, g = params[n], bits_to_f32(grads[n]).reshape(params[n].shape)
            buf, u = muon_momentum(np.zeros_like(W0), g, clip=clip)
            assert bits_equal(s["buf"].to_numpy().reshape(W0.shape), buf), n
            want = muon_update(W0, ns_any_shape(u, PE_SCHEDULE, 5), LR_MUON)
            got = s["p32"].to_numpy().reshape(W0.shape)
            err = rel_fro(W0.astype(np.float64) - got, W0.astype(np.float64) - want)
            worst[shape] = max(worst.get(shape, 0.0), err)
            assert bits_equal(s["p16"].to_numpy().ravel(), bf16_sr_bits(got.ravel(), (sb + index[n]) & 0xFFFFFFFF)), n
    print("\nconfig 2, worst update-direction error per Muon shape (bar 2e-3):")
    for shape, err in worst.items():
        print(f"  {shape:28s} {err:.3e}")
    for shape, err in worst.items():
        assert err < 2e-3, (shape, err)


def test_config2_every_muon_weight_moved_by_an_orthogonal_update(c2):
    """Size-independent property over all 196 matrices: the update W0 - W1 = lr * scale * O with O
    near-orthogonal has Frobenius norm lr * scale * sqrt(min(K, N)) up to the spread the 5-step
    schedule leaves on the singular values (0.7 .. 1.2)."""
    opt, params = c2["opt"], c2["params"]
    for n, s in opt.muon.st.items():
        W0 = params[n]
        K, N = W0.shape
        d = np.linalg.norm(W0.astype(np.float64) - s["p32"].to_numpy().reshape(W0.shape))
        unit = LR_MUON * max(1.0, K / N) ** 0.5 * min(K, N) ** 0.5
        assert 0.6 * unit < d < 1.25 * unit, (n, d / unit)
