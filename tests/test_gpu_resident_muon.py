"""The per-weight resident Muon classes (`DeviceMuon`, `ResidentMuon` over one shared
`MuonScratch`), the device `newton_schulz5`, `ns_fp32_batched` and `anc_cast_bf16`, on the shapes
and step counts of the reference's harness for them (tests/kernels/_probe_device_muon.py:43-138:
(1024,1024), (1024,2048), (2048,1024); T = 5; W0 ~ 0.05 N(0,1), g ~ N(0,1); accumulated update
cos > 0.99 and rel < 0.06 against the host class; descent on 0.5 ||W - T||^2 below 20 %)."""
import numpy as np
import pytest

from oracle.bf16_ref import bf16_rne_bits, bf16_sr_bits, bits_to_f32
from oracle.muon_ref import MuonRef, PE_SCHEDULE, host_ns, newton_schulz5 as ns5_ref
from util import bits_equal, rel_fro

pytestmark = pytest.mark.gpu

SHAPES = [(1024, 1024), (1024, 2048), (2048, 1024)]          # square, wide, tall (transposed chain)


def _cos(a, b):
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))


@pytest.mark.parametrize("K,N", SHAPES)
@pytest.mark.parametrize("sched", ["keller", "pe"])
def test_device_muon_reproduces_the_host_class(gpu, K, N, sched):
    """Same W0, same five gradients: the accumulated update W0 - W5 against the numpy class.
    The momentum buffer never depends on the weights, so it is bit-equal after every step and the
    five update directions are each one chain call: the reference's bars and the 2e-3 bar hold
    with its default (Keller) schedule and with Polar-Express."""
    from ancora_cutile_amd import DeviceMuon, DevBuf
    from ancora_cutile_amd.muon import _f32bf_trunc
    schedule = None if sched == "keller" else PE_SCHEDULE
    rng = np.random.default_rng(0)
    W0 = (0.05 * rng.standard_normal((K, N))).astype(np.float32)
    grads = [rng.standard_normal((K, N)).astype(np.float32) for _ in range(5)]
    host = MuonRef({"w": W0}, lr=0.02, momentum=0.95, nesterov=True, ns_steps=5, sched=schedule)
    dm = DeviceMuon(W0.copy(), lr=0.02, momentum=0.95, ns_steps=5)
    assert bits_equal(dm.p16.to_numpy(), _f32bf_trunc(W0))          # initial bf16 weights: truncation
    g_dev = DevBuf.zeros((K, N), np.float32)
    for g in grads:
        host.step({"w": g})
        g_dev.upload(g)
        dm.step(g_dev, 0, schedule=schedule)
        gpu.stream_sync(0)
        assert bits_equal(dm.buf.to_numpy(), host.buf["w"])
    Wd, Wh = dm.master(), host.w["w"]
    du_d, du_h = W0 - Wd, W0 - Wh
    c, r = _cos(du_d, du_h), rel_fro(du_d, du_h)
    print(f"({K},{N}) {sched}: accumulated update cos {c:.6f} rel {r:.3e}")
    assert c > 0.99 and r < 0.06                                    # _probe_device_muon.py:65
    assert r < 2e-3
    assert bits_equal(dm.p16.to_numpy(), bf16_rne_bits(Wd))         # refreshed by RNE after a step
    g_dev.free()
    dm.free()


def test_device_muon_descends_on_a_quadratic(gpu):
    """_probe_device_muon.py:72-101 on the square and the tall shape: g = W - T, 30 steps."""
    from ancora_cutile_amd import DeviceMuon, DevBuf
    for K, N in ((1024, 1024), (2048, 1024)):
        rng = np.random.default_rng(1)
        T = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
        dm = DeviceMuon(np.zeros((K, N), np.float32), lr=0.02, momentum=0.95, ns_steps=5)
        g_dev = DevBuf.zeros((K, N), np.float32)
        loss = []
        for _ in range(30):
            g = dm.master() - T
            loss.append(0.5 * float(np.sum(g.astype(np.float64) ** 2)))
            g_dev.upload(g)
            dm.step(g_dev, 0)
            gpu.stream_sync(0)
        assert loss[-1] / loss[0] < 0.2, (K, N, loss[-1] / loss[0])
        g_dev.free()
        dm.free()


@pytest.mark.parametrize("gdtype", [np.float32, np.uint16])
def test_resident_muon_shares_one_scratch_across_shapes(gpu, gdtype):
    """`ResidentMuon` over existing p32 / p16 buffers with ONE `MuonScratch` for the square, the
    wide and the tall weight, all stepping in the same five steps, nothing synchronised in between
    (_probe_device_muon.py:104-138): no cross-contamination through the shared scratch, the tall
    path right, fp32 and bf16 device gradients."""
    from ancora_cutile_amd import ResidentMuon, MuonScratch, DevBuf
    from ancora_cutile_amd.muon import _f32bf_trunc
    rng = np.random.default_rng(0)
    sc = MuonScratch(SHAPES)
    assert sc.nbytes() > 2048 * 1024 * 4
    rms = []
    for K, N in SHAPES:
        W0 = (0.05 * rng.standard_normal((K, N))).astype(np.float32)
        host = MuonRef({"w": W0}, lr=0.02, momentum=0.95, ns_steps=5, sched=PE_SCHEDULE)
        p32, p16 = DevBuf(W0.copy()), DevBuf(_f32bf_trunc(W0))
        rm = ResidentMuon(p32, p16, K, N, sc, momentum=0.95, ns_steps=5)
        rms.append((K, N, W0, host, p32, p16, rm, [DevBuf.zeros((K, N), gdtype) for _ in range(5)]))
    for t in range(5):
        for K, N, W0, host, p32, p16, rm, gbufs in rms:
            g = rng.standard_normal((K, N)).astype(np.float32)
            if gdtype == np.uint16:
                bits = bf16_rne_bits(g).reshape(K, N)
                g = bits_to_f32(bits).reshape(K, N)
                gbufs[t].upload(bits)
            else:
                gbufs[t].upload(g)
            host.step({"w": g})
            rm.step(gbufs[t], 0, 0.02, schedule=PE_SCHEDULE)
    gpu.stream_sync(0)
    for K, N, W0, host, p32, p16, rm, gbufs in rms:
        Wd, Wh = p32.to_numpy(), host.w["w"]
        c, r = _cos(W0 - Wd, W0 - Wh), rel_fro(W0 - Wd, W0 - Wh)
        print(f"({K},{N}) shared scratch, {np.dtype(gdtype).name} gradients: cos {c:.6f} rel {r:.3e}")
        assert c > 0.99 and r < 0.06 and r < 2e-3
        assert bits_equal(rm.buf.to_numpy(), host.buf["w"])
        assert bits_equal(p16.to_numpy(), bf16_rne_bits(Wd))
        for b in [p32, p16] + gbufs:
            b.free()
        rm.free()
    sc.free()


def test_device_newton_schulz5_matches_the_host_function(gpu):
    """`newton_schulz5(G)`: host matrix in, host matrix out, Keller by default, tall inputs
    transposed in and out (ancora/optim/muon.py:67-80)."""
    from ancora_cutile_amd import newton_schulz5
    rng = np.random.default_rng(3)
    for K, N in ((256, 256), (128, 512), (1024, 2048), (2048, 1024), (384, 128)):
        G = rng.standard_normal((K, N)).astype(np.float32)
        want = ns5_ref(G, 5)
        got = newton_schulz5(G)
        assert got.shape == (K, N) and got.dtype == np.float32
        assert rel_fro(got, want) < 2e-3, (K, N)                     # Keller, default bf16 mode
        assert rel_fro(newton_schulz5(G, mode="fp32"), want) < 1e-5, (K, N)
        X = G.T if K > N else G
        pe = host_ns(X, PE_SCHEDULE, 5)
        got_pe = newton_schulz5(G, schedule=PE_SCHEDULE)
        assert rel_fro(got_pe, pe.T if K > N else pe) < 2e-3, (K, N)
    with pytest.raises(ValueError):
        newton_schulz5(np.zeros((100, 128), np.float32))


def test_ns_fp32_batched_is_the_native_driver(gpu):
    from ancora_cutile_amd import DevBuf, ns_fp32_batched
    rng = np.random.default_rng(4)
    X = rng.standard_normal((3, 256, 384)).astype(np.float32)
    d = DevBuf(X.reshape(3 * 256, 384))
    ns_fp32_batched(d, 3, 256, 384, 0, schedule=PE_SCHEDULE, mode="fp32")
    got = d.to_numpy().reshape(3, 256, 384)
    for e in range(3):
        assert rel_fro(got[e], host_ns(X[e], PE_SCHEDULE, 5)) < 1e-5
    d.free()


@pytest.mark.parametrize("n", [4, 64, 4096, 4096 * 3 + 8, 1 << 20])
def test_cast_bf16_rne_and_stochastic(gpu, n):
    """`anc_cast_bf16` (`_cast_bf16`, ancora/kernels/fused.py:285-290): round-to-nearest-even bits,
    and the counter-based stochastic rounding keyed on the flat index, Inf/NaN passed through."""
    from ancora_cutile_amd import DevBuf
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32) * np.float32(10.0) ** rng.integers(-6, 6, n).astype(np.float32)
    x[::97] = bits_to_f32(bf16_rne_bits(x[::97]))            # values already on the bf16 grid
    if n >= 64:
        x[3], x[17], x[40] = np.inf, -np.inf, np.nan
        x[5] = np.float32(1.0 + 2.0 ** -8)                   # exact tie: to even
    p32, p16 = DevBuf(x), DevBuf.zeros((max(n, 2),), np.uint16)
    gpu.api.anc_cast_bf16(p32.ptr, p16.ptr, n, 0, 0, 0)
    got = p16.to_numpy()[:n]
    want = bf16_rne_bits(x)
    finite = np.isfinite(x)
    assert bits_equal(got[finite], want[finite])
    assert np.array_equal(np.isnan(bits_to_f32(got)), np.isnan(x))
    assert np.array_equal(bits_to_f32(got)[np.isinf(x)], x[np.isinf(x)])
    for seed in (0, 12345, 0xFFFFFFFF):
        gpu.api.anc_cast_bf16(p32.ptr, p16.ptr, n, 1, seed, 0)
        assert bits_equal(p16.to_numpy()[:n], bf16_sr_bits(x, seed)), seed
    with pytest.raises(gpu.AncoraError):
        gpu.api.anc_cast_bf16(p32.ptr, p16.ptr, 6, 0, 0, 0)
    p32.free(); p16.free()
