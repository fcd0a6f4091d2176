"""GPU parity of the weight-gradient GEMM dW (+)= x^T dy against the fp64 product of the bf16
inputs (the reference's own checker, tests/kernels/test_gemm_bwd.py), plus what the build adds:
accumulation in place, the bf16 copy, independence of the result's bits from grouping."""
import numpy as np
import pytest

from oracle.gemm_ref import gemm_dw
from oracle.bf16_ref import bf16_rne_bits
from util import rel_fro, bits_equal

pytestmark = pytest.mark.gpu


def _inputs(T, K, N, seed):
    rng = np.random.default_rng(seed)
    x = bf16_rne_bits((0.1 * rng.standard_normal((T, K))).astype(np.float32)).reshape(T, K)
    dy = bf16_rne_bits((0.1 * rng.standard_normal((T, N))).astype(np.float32)).reshape(T, N)
    return x, dy


def _problem(x, dy, T, K, N, emit=False, dW0=None):
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd.grads import transpose_acts, DwWorkspace
    xd, xT = DevBuf(x), DevBuf.zeros((K, T), np.uint16)
    transpose_acts(xd, xT, T, K)
    p = dict(xT=xT, dy=DevBuf(dy), dW=DevBuf.zeros((K, N), np.float32) if dW0 is None else DevBuf(dW0),
             T=T, K=K, N=N, workspace=DwWorkspace(), g16=DevBuf.zeros((K, N), np.uint16) if emit else None,
             accumulate=dW0 is not None)
    p["_x"] = xd
    return p


def _free(p):
    for k in ("xT", "dy", "dW", "g16", "_x"):
        if p.get(k) is not None:
            p[k].free()
    p["workspace"].free()


@pytest.mark.parametrize("T,K,N", [(512, 1024, 1024), (256, 1024, 3072), (64, 128, 256), (2048, 128, 256),
                                   (4096, 256, 512), (96, 384, 768)])
def test_matches_fp64_product(gpu, T, K, N):
    """The first two shapes are the reference's (test_gemm_bwd.py:49-50); the others reach a single
    tile and a token count that is not a multiple of 64. Default: the token axis is not cut; then the
    opt-in shape rule (one to many token segments) on the same inputs."""
    from ancora_cutile_amd.grads import gemm_dW, dw_info
    x, dy = _inputs(T, K, N, T + K + N)
    p = _problem(x, dy, T, K, N, emit=True) if T % 64 == 0 else None
    if p is None:                                  # the device transpose works on 64x64 tiles
        from ancora_cutile_amd import DevBuf
        from ancora_cutile_amd.grads import DwWorkspace
        p = dict(xT=DevBuf(np.ascontiguousarray(x.T)), dy=DevBuf(dy), dW=DevBuf.zeros((K, N), np.float32),
                 T=T, K=K, N=N, workspace=DwWorkspace(), g16=DevBuf.zeros((K, N), np.uint16), accumulate=False)
    gemm_dW([p])
    got = p["dW"].to_numpy()
    want = gemm_dw(x, dy)
    assert rel_fro(got, want) < 2e-5
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-4        # reference bar: 2e-2
    assert bits_equal(p["g16"].to_numpy(), bf16_rne_bits(got).reshape(K, N))
    fl, seg = dw_info(T, K, N)
    assert fl == 2.0 * T * K * N and seg >= 1 and T % (32 * seg) == 0
    gemm_dW([p], segments="shape")
    split = p["dW"].to_numpy()
    assert rel_fro(split, want) < 2e-5
    if seg == 1:
        assert bits_equal(split, got)
    _free(p)


def test_accumulates_in_place_and_is_deterministic(gpu):
    from ancora_cutile_amd.grads import gemm_dW
    T, K, N = 1024, 256, 512
    x1, dy1 = _inputs(T, K, N, 1)
    x2, dy2 = _inputs(T, K, N, 2)
    p1 = _problem(x1, dy1, T, K, N)
    gemm_dW([p1])
    first = p1["dW"].to_numpy()
    p2 = _problem(x2, dy2, T, K, N, emit=True, dW0=first)
    gemm_dW([p2])
    total = p2["dW"].to_numpy()
    assert rel_fro(total, gemm_dw(x2, dy2, gemm_dw(x1, dy1))) < 2e-5
    assert bits_equal(p2["g16"].to_numpy(), bf16_rne_bits(total).reshape(K, N))
    # the same call again on the same inputs gives the same bits
    p3 = _problem(x2, dy2, T, K, N, dW0=first)
    gemm_dW([p3])
    assert bits_equal(p3["dW"].to_numpy(), total)
    for p in (p1, p2, p3):
        _free(p)


def test_grouping_does_not_change_bits(gpu):
    """q, k, v style: three weights that share the activations, alone and in one call."""
    from ancora_cutile_amd.grads import gemm_dW
    T, K = 1024, 256
    Ns = (512, 256, 768)
    x, _ = _inputs(T, K, 256, 5)
    dys = [_inputs(T, K, N, 10 + i)[1] for i, N in enumerate(Ns)]
    alone = []
    for dy, N in zip(dys, Ns):
        p = _problem(x, dy, T, K, N)
        gemm_dW([p])
        alone.append(p["dW"].to_numpy())
        _free(p)
    ps = [_problem(x, dy, T, K, N) for dy, N in zip(dys, Ns)]
    gemm_dW(ps)
    for p, a in zip(ps, alone):
        assert bits_equal(p["dW"].to_numpy(), a)
        _free(p)


def test_whole_layer_in_one_call_with_explicit_segments(gpu):
    """Seven weights of four shapes in one call, one token segment each (the launch a caller makes
    who collects a layer's gradient GEMMs), against the fp64 product; a weight's bits are the
    same alone and in the group, equal to the shape rule's when that also gives one segment, and
    2 and 4 segments stay within the same error."""
    from ancora_cutile_amd.grads import gemm_dW, dw_info
    T = 512
    shapes = [(256, 512), (256, 256), (256, 256), (512, 256), (256, 768), (256, 768), (768, 256)]
    xs, ps = {}, []
    for i, (K, N) in enumerate(shapes):
        x, dy = _inputs(T, K, N, 40 + i)
        ps.append(_problem(x, dy, T, K, N, emit=True))
        xs[i] = (x, dy)
    gemm_dW(ps, segments=1)
    outs = [p["dW"].to_numpy() for p in ps]
    for i, (K, N) in enumerate(shapes):
        assert rel_fro(outs[i], gemm_dw(*xs[i])) < 2e-5
        assert bits_equal(ps[i]["g16"].to_numpy(), bf16_rne_bits(outs[i]).reshape(K, N))
    for i in (0, 6):
        K, N = shapes[i]
        q = _problem(xs[i][0], xs[i][1], T, K, N)
        gemm_dW([q], segments=1)
        assert bits_equal(q["dW"].to_numpy(), outs[i])
        for S in (2, 4):
            gemm_dW([q], segments=S)
            assert rel_fro(q["dW"].to_numpy(), gemm_dw(*xs[i])) < 2e-5
        q["segments"] = 2                       # per problem, and again: same bits
        gemm_dW([q])
        a = q["dW"].to_numpy()
        gemm_dW([q], segments=2)
        assert bits_equal(q["dW"].to_numpy(), a)
        _free(q)
    # the per-launch rule: 3 weights of 4 + 2 + 2 tiles at 512 tokens -> 2 segments of 256 tokens
    for p3 in ps[:3]:
        p3["dW"].upload(np.zeros(p3["dW"].shape, np.float32))
    gemm_dW(ps[:3], segments="fill")
    for i in range(3):
        got = ps[i]["dW"].to_numpy()
        assert rel_fro(got, gemm_dw(*xs[i])) < 2e-5
        K, N = shapes[i]
        q = _problem(xs[i][0], xs[i][1], T, K, N)
        gemm_dW([q], segments=2)
        assert bits_equal(q["dW"].to_numpy(), got)
        _free(q)
    # shape rule with one segment == explicit one segment
    K, N = 2048, 4096
    assert dw_info(64, K, N)[1] == 1
    x, dy = _inputs(64, K, N, 50)
    q = _problem(x, dy, 64, K, N)
    gemm_dW([q])
    a = q["dW"].to_numpy()
    gemm_dW([q], segments=1)
    assert bits_equal(q["dW"].to_numpy(), a)
    _free(q)
    for p in ps:
        _free(p)


def test_one_segment_route_through_the_epilogue_has_the_two_kernel_bits(gpu):
    """With one token segment and no grad-norm sums asked for, the GEMM's epilogue adds onto dW and
    writes the bf16 copy itself; asking for the sums sends the same problem through the partial
    tile and the finishing kernel. Same bits either way, with and without accumulation."""
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd.grads import gemm_dW
    T, K, N = 512, 256, 768
    x, dy = _inputs(T, K, N, 60)
    dW0 = (0.5 * np.random.default_rng(61).standard_normal((K, N))).astype(np.float32)
    sums = DevBuf.zeros((K * N // 8192,), np.float64)
    for prev in (None, dW0):
        a = _problem(x, dy, T, K, N, emit=True, dW0=prev)
        b = _problem(x, dy, T, K, N, emit=True, dW0=prev)
        b["gn_partials"] = sums.ptr
        gemm_dW([a], segments=1)
        gemm_dW([b], segments=1)
        assert a["workspace"].buf is None and b["workspace"].buf is not None
        assert bits_equal(a["dW"].to_numpy(), b["dW"].to_numpy())
        assert bits_equal(a["g16"].to_numpy(), b["g16"].to_numpy())
        assert rel_fro(a["dW"].to_numpy(), gemm_dw(x, dy, prev)) < 2e-5
        _free(a); _free(b)
    # all-zero activations: the product is +0 on both routes
    z = np.zeros_like(x)
    a, b = _problem(z, dy, T, K, N), _problem(z, dy, T, K, N)
    b["gn_partials"] = sums.ptr
    gemm_dW([a], segments=1)
    gemm_dW([b], segments=1)
    assert bits_equal(a["dW"].to_numpy(), b["dW"].to_numpy()) and not a["dW"].to_numpy().any()
    _free(a); _free(b)
    sums.free()


@pytest.mark.parametrize("T,K,N,S", [(512, 1024, 1024, None), (256, 1024, 3072, 1), (2048, 128, 256, None),
                                     (96, 384, 768, 1), (1024, 256, 512, 4)])
def test_activations_as_they_lie_give_the_bits_of_the_transposed_route(gpu, T, K, N, S):
    """`x` (T, K), the reference's argument, against `xT` (K, T): the same products summed in the
    same order, so the same bits; and within the bar of the fp64 product."""
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd.grads import gemm_dW, DwWorkspace
    x, dy = _inputs(T, K, N, 70 + T)
    dW0 = (0.5 * np.random.default_rng(71).standard_normal((K, N))).astype(np.float32)
    outs = []
    for lay in ("x", "xT"):
        p = dict(dy=DevBuf(dy), dW=DevBuf(dW0), T=T, K=K, N=N, workspace=DwWorkspace(),
                 g16=DevBuf.zeros((K, N), np.uint16), accumulate=True)
        p[lay] = DevBuf(x if lay == "x" else np.ascontiguousarray(x.T))
        gemm_dW([p], segments=S)
        outs.append((p["dW"].to_numpy(), p["g16"].to_numpy()))
        p.pop(lay).free()
        _free(p)
    assert rel_fro(outs[0][0], gemm_dw(x, dy, dW0)) < 2e-5
    assert bits_equal(outs[0][0], outs[1][0]) and bits_equal(outs[0][1], outs[1][1])


def test_qwen3_layer_at_full_shape(gpu):
    """The launch the benchmark times: the 7 weight gradients of one Qwen3-0.6B layer in one call
    (activations as they lie, one token segment, accumulation, bf16 copy), 4096 tokens, against the
    fp64 product."""
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd.grads import gemm_dW, DwWorkspace
    rng = np.random.default_rng(5)
    T = 4096
    layer = [(1024, 2048), (1024, 1024), (1024, 1024), (2048, 1024), (1024, 3072), (1024, 3072), (3072, 1024)]
    xs, probs, refs = {}, [], []
    for (K, N) in layer:
        if K not in xs:
            x = bf16_rne_bits((0.1 * rng.standard_normal((T, K))).astype(np.float32)).reshape(T, K)
            xs[K] = (x, DevBuf(x))
        x, xd = xs[K]
        dy = bf16_rne_bits((0.1 * rng.standard_normal((T, N))).astype(np.float32)).reshape(T, N)
        dW0 = (0.3 * rng.standard_normal((K, N))).astype(np.float32)
        probs.append(dict(x=xd, dy=DevBuf(dy), dW=DevBuf(dW0), g16=DevBuf.zeros((K, N), np.uint16), T=T, K=K,
                          N=N, workspace=DwWorkspace(), accumulate=True))
        refs.append((x, dy, dW0))
    gemm_dW(probs, 0, segments=1)
    for p, (x, dy, dW0) in zip(probs, refs):
        got = p["dW"].to_numpy()
        assert rel_fro(got, gemm_dw(x, dy, dW0)) < 2e-5
        assert bits_equal(p["g16"].to_numpy(), bf16_rne_bits(got).reshape(p["K"], p["N"]))
        for k in ("dy", "dW", "g16"):
            p[k].free()
    for _, xd in xs.values():
        xd.free()


def test_shape_checks(gpu):
    from ancora_cutile_amd import _lib
    from ancora_cutile_amd.grads import dw_workspace_bytes
    with pytest.raises(_lib.AncoraError):
        dw_workspace_bytes(100, 128, 256)
    with pytest.raises(_lib.AncoraError):
        dw_workspace_bytes(128, 64, 256)
    assert dw_workspace_bytes(64, 128, 256) == 128 * 256 * 4
    from ancora_cutile_amd.grads import gemm_dW
    x, dy = _inputs(64, 128, 256, 1)
    q = _problem(x, dy, 64, 128, 256)
    with pytest.raises(_lib.AncoraError):
        gemm_dW([q], segments=4)                # 64 tokens do not split into 4 x 32k
    _free(q)


def test_producer_writes_the_grad_norm_partials(gpu):
    """With `gn_partials` the reduce kernel leaves the chunk sums of squares of the gradient it
    emits (bf16 copy, or the fp32 gradient when there is none) where StepGuard keeps them; the
    control block then has the bits of a norm pass over the stored gradients."""
    from ancora_cutile_amd import DevBuf, StepGuard
    from ancora_cutile_amd.grads import gemm_dW
    T, K = 512, 256
    Ns = (512, 256)
    x, _ = _inputs(T, K, 256, 3)
    ps = [_problem(x, _inputs(T, K, N, 20 + i)[1], T, K, N, emit=(i == 0)) for i, N in enumerate(Ns)]
    other = DevBuf(bf16_rne_bits((1e-2 * np.random.default_rng(4).standard_normal(50000)).astype(np.float32)))
    grads = [ps[0]["g16"], other, ps[1]["dW"]]          # bf16 copy, an unrelated tensor, an fp32 gradient
    guard = StepGuard(1.0)
    guard.plan(grads)
    ps[0]["gn_partials"], ps[1]["gn_partials"] = guard.partials_ptr(0), guard.partials_ptr(2)
    gemm_dW(ps)
    guard.compute(grads, 0, produced=(0, 2))
    got = guard.ctl.to_numpy()
    guard2 = StepGuard(1.0)
    guard2.compute(grads, 0)
    want = guard2.ctl.to_numpy()
    assert np.array_equal(got, want)
    c = guard.read()
    assert c["norm"] > 0 and not c["skip"]
    guard.free(); guard2.free(); other.free()
    for p in ps:
        _free(p)


def test_backward_to_step_hand_off(gpu):
    """The weight-gradient GEMM feeds the optimizer step directly: bf16 gradients and grad-norm
    partial sums from the producer, `step(..., produced=...)`; same weights, bit for bit, as the
    step computing the norm itself from the same gradients."""
    from ancora_cutile_amd import HybridOptimizer, DevBuf, PE_SCHEDULE as PE
    from ancora_cutile_amd.grads import gemm_dW
    rng = np.random.default_rng(12)
    T, K = 512, 256
    shapes = {"layer0.q_proj": (K, 512), "layer0.k_proj": (K, 256)}
    params = {n: (0.02 * rng.standard_normal(s)).astype(np.float32) for n, s in shapes.items()}
    params["layer0.input_ln"] = (1.0 + 0.05 * rng.standard_normal(256)).astype(np.float32)
    x, _ = _inputs(T, K, 256, 30)
    dys = {n: _inputs(T, K, s[1], 31 + i)[1] for i, (n, s) in enumerate(shapes.items())}
    g_ln = DevBuf(bf16_rne_bits((1e-2 * rng.standard_normal(256)).astype(np.float32)))

    def run(use_produced):
        opt = HybridOptimizer(params, max_grad_norm=1.0, grad_dtype=np.uint16,
                              muon_kw=dict(lr=0.02, momentum=0.95, ns_steps=5, schedule=PE))
        ps = {n: _problem(x, dys[n], T, K, s[1], emit=True) for n, s in shapes.items()}
        grads = {n: ps[n]["g16"] for n in shapes}
        grads["layer0.input_ln"] = g_ln
        if use_produced:
            for n in shapes:
                ps[n]["gn_partials"] = opt.gn_partials_ptr(grads, n)
        gemm_dW(list(ps.values()))
        opt.step(grads, 0, produced=list(shapes) if use_produced else ())
        out = {**opt.muon.master(), **opt.adamw.master()}, opt.last_ctl
        opt.free()
        for p in ps.values():
            _free(p)
        return out

    (ma, ca), (mb, cb) = run(True), run(False)
    assert ca == cb and ca["clip_scale"] < 1.0
    for n in params:
        assert bits_equal(ma[n], mb[n])
    g_ln.free()


def test_accumulated_micro_batches_against_one_batch(gpu):
    """The reference's accumulation check (tests/training/test_grad_accum.py:60-93) on this path:
    the gradient of 2T tokens in one call against two calls of T tokens, the second accumulating
    onto the first. (B) the two gradients agree to the reference's bar (rel < 2e-3; here only the
    fp32 regrouping of the sum separates them); (C) the accumulated route repeats bit for bit;
    (D) after one AdamW step on each, at least 98 % of the updated weights are bit-identical."""
    from ancora_cutile_amd import AdamW, DevBuf
    from ancora_cutile_amd.grads import gemm_dW
    T, K, N = 1024, 512, 1024
    x, dy = _inputs(2 * T, K, N, 77)
    rng = np.random.default_rng(5)
    w0 = (0.02 * rng.standard_normal((K, N))).astype(np.float32)

    def one_batch():
        p = _problem(x, dy, 2 * T, K, N, emit=True)
        gemm_dW([p])
        out = p["dW"].to_numpy(), p["g16"].to_numpy()
        _free(p)
        return out

    def accumulated():
        p0 = _problem(x[:T], dy[:T], T, K, N, emit=True)
        gemm_dW([p0])
        first = p0["dW"].to_numpy()
        p1 = _problem(x[T:], dy[T:], T, K, N, emit=True, dW0=first)
        gemm_dW([p1])
        out = p1["dW"].to_numpy(), p1["g16"].to_numpy()
        _free(p0); _free(p1)
        return out

    (gA, hA), (gB, hB), (gB2, hB2) = one_batch(), accumulated(), accumulated()
    assert rel_fro(gB, gA) < 2e-3 and rel_fro(gB, gA) < 1e-6          # (B): reference bar, then what it is here
    assert bits_equal(gB, gB2) and bits_equal(hB, hB2)                 # (C)
    assert rel_fro(gA, gemm_dw(x, dy)) < 2e-5 and rel_fro(gB, gemm_dw(x, dy)) < 2e-5
    new = []
    for h in (hA, hB):
        opt = AdamW({"w": w0}, lr=1e-3, grad_dtype=np.uint16)
        g = DevBuf(h)
        opt.step({"w": g}, 0)
        new.append(opt.weights()["w"])
        opt.free(); g.free()
    same = float((new[0].view(np.uint32) == new[1].view(np.uint32)).mean())
    assert same >= 0.98, same                                          # (D): the reference's bar
