"""GPU parity of Muon's elementwise stages (momentum + Nesterov, update + bf16 refresh,
transposes) against the numpy oracle: bit-exact."""
import numpy as np
import pytest

from oracle.bf16_ref import bf16_rne_bits, bf16_sr_bits, bits_to_f32
from oracle.muon_ref import muon_momentum, muon_update, shape_scale
from util import bits_equal, bf16_grad

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("K,N", [(128, 128), (256, 128), (128, 384)])
@pytest.mark.parametrize("gdt", ["f32", "bf16"])
@pytest.mark.parametrize("udt", ["f32", "bf16"])
def test_momentum_both_orientations(gpu, K, N, gdt, udt):
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd._lib import api
    rng = np.random.default_rng(K * 7 + N)
    buf0 = rng.standard_normal((K, N)).astype(np.float32)
    if gdt == "bf16":
        gbits, g = bf16_grad(rng, (K, N), 1.0)
        gdev, gcode = DevBuf(gbits), _lib.BF16
    else:
        g = rng.standard_normal((K, N)).astype(np.float32)
        gdev, gcode = DevBuf(g), _lib.F32
    want_buf, want_u = muon_momentum(buf0, g, 0.95, True)
    for tr in (0, 1):
        buf = DevBuf(buf0)
        shape = (N, K) if tr else (K, N)
        u = DevBuf.zeros(shape, np.uint16 if udt == "bf16" else np.float32)
        api.anc_muon_momentum(buf.ptr, gdev.ptr, u.ptr, K, N, 0.95, 1, tr, gcode,
                              _lib.BF16 if udt == "bf16" else _lib.F32, 0, 0)
        assert bits_equal(buf.to_numpy(), want_buf)
        wu = want_u.T if tr else want_u
        got = u.to_numpy()
        if udt == "bf16":
            assert bits_equal(got, bf16_rne_bits(np.ascontiguousarray(wu)).reshape(shape))
        else:
            assert bits_equal(got, np.ascontiguousarray(wu))
        buf.free(); u.free()
    gdev.free()


def test_momentum_without_nesterov(gpu):
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd._lib import api
    rng = np.random.default_rng(0)
    buf0 = rng.standard_normal((128, 128)).astype(np.float32)
    g = rng.standard_normal((128, 128)).astype(np.float32)
    buf, gd, u = DevBuf(buf0), DevBuf(g), DevBuf.zeros((128, 128), np.float32)
    api.anc_muon_momentum(buf.ptr, gd.ptr, u.ptr, 128, 128, 0.9, 0, 0, _lib.F32, _lib.F32, 0, 0)
    wb, wu = muon_momentum(buf0, g, 0.9, False)
    assert bits_equal(buf.to_numpy(), wb) and bits_equal(u.to_numpy(), wu)
    for b in (buf, gd, u):
        b.free()


@pytest.mark.parametrize("K,N", [(128, 128), (256, 128), (384, 128), (128, 256)])
@pytest.mark.parametrize("odt", ["f32", "bf16"])
@pytest.mark.parametrize("sr", [0, 1])
def test_update_and_cast(gpu, K, N, odt, sr):
    """p32 -= lr*sqrt(max(1,K/N))*O with O given in the NS orientation (transposed for tall
    weights); p16 = RNE or SR of the new p32."""
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd._lib import api
    rng = np.random.default_rng(K + 3 * N + sr)
    W = (0.05 * rng.standard_normal((K, N))).astype(np.float32)
    O = rng.standard_normal((K, N)).astype(np.float32)
    if odt == "bf16":
        O = bits_to_f32(bf16_rne_bits(O)).reshape(K, N)
    tr = int(K > N)
    O_dev_host = np.ascontiguousarray(O.T) if tr else O
    Od = DevBuf(bf16_rne_bits(O_dev_host).reshape(O_dev_host.shape)) if odt == "bf16" else DevBuf(O_dev_host)
    p32, p16 = DevBuf(W), DevBuf.zeros((K, N), np.uint16)
    lr = 0.02
    seed = 77
    api.anc_muon_update(p32.ptr, p16.ptr, Od.ptr, K, N, lr * shape_scale(K, N), tr,
                        _lib.BF16 if odt == "bf16" else _lib.F32, sr, seed, 0, 0)
    want = muon_update(W, O, lr)
    assert bits_equal(p32.to_numpy(), want)
    w16 = bf16_sr_bits(want, seed) if sr else bf16_rne_bits(want)
    assert bits_equal(p16.to_numpy(), w16.reshape(K, N))
    for b in (Od, p32, p16):
        b.free()


def test_bf16_transpose_batched(gpu):
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd._lib import api
    rng = np.random.default_rng(4)
    X = rng.integers(0, 65536, (3, 128, 320), dtype=np.uint16)
    xd, xt = DevBuf(X.reshape(3 * 128, 320)), DevBuf.zeros((3 * 320, 128), np.uint16)
    api.anc_transpose_bf16(xd.ptr, xt.ptr, 3, 128, 320, 0)
    assert np.array_equal(xt.to_numpy().reshape(3, 320, 128), X.transpose(0, 2, 1))
    xd.free(); xt.free()


def test_shape_checks(gpu):
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd._lib import api
    b = DevBuf.zeros((128, 128), np.float32)
    with pytest.raises(_lib.AncoraError):
        api.anc_muon_momentum(b.ptr, b.ptr, b.ptr, 100, 128, 0.95, 1, 0, _lib.F32, _lib.F32, 0, 0)
    with pytest.raises(_lib.AncoraError):
        api.anc_muon_update(0, 0, b.ptr, 128, 128, 0.1, 0, _lib.F32, 0, 0, 0, 0)
    b.free()


@pytest.mark.parametrize("K,N", [(128, 256), (256, 128)])
def test_momentum_pair_output_and_frobenius_partials(gpu, K, N):
    """The pair momentum kernel: momentum buffer bit-exact, u leaves as hi = bf16(u) and
    lo = bf16(u - hi) in the chain's orientation, and the per-block sums of u*u add up to the
    fp64 sum of squares (each block sums 4096 fp32 values in fp64: exact to ~1e-15 relative)."""
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd._lib import api, MuonDesc
    from ancora_cutile_amd.devbuf import upload_table
    rng = np.random.default_rng(K + N)
    E = 3
    M, Nn = min(K, N), max(K, N)
    tr = int(K > N)
    bufs0 = [rng.standard_normal((K, N)).astype(np.float32) for _ in range(E)]
    gs = [rng.standard_normal((K, N)).astype(np.float32) for _ in range(E)]
    U = DevBuf.zeros((E * M * Nn,), np.float32)
    fro = DevBuf.zeros((E * K * N // 4096,), np.float64)
    bd = [DevBuf(b) for b in bufs0]
    gd = [DevBuf(g) for g in gs]
    descs, blk0 = [], 0
    for i in range(E):
        descs.append(MuonDesc(bd[i].ptr, gd[i].ptr, 0, 0, U.ptr + i * M * Nn * 4, K, N, tr, _lib.F32, 0, i, blk0))
        blk0 += K * N // 4096
    table = upload_table(descs)
    api.anc_muon_momentum_multi_pair(table.ptr, E, blk0, 0.95, 1, U.ptr, E * M * Nn * 2, fro.ptr, 0, 0)
    pair = U.view((2, E, M, Nn), np.uint16).to_numpy()
    parts = fro.to_numpy().reshape(E, -1)
    for i in range(E):
        wb, wu = muon_momentum(bufs0[i], gs[i], 0.95, True)
        assert bits_equal(bd[i].to_numpy(), wb)
        wu = np.ascontiguousarray(wu.T) if tr else wu
        hi = bf16_rne_bits(wu).reshape(M, Nn)
        lo = bf16_rne_bits(wu - bits_to_f32(hi).reshape(M, Nn)).reshape(M, Nn)
        assert bits_equal(pair[0, i], hi) and bits_equal(pair[1, i], lo)
        want = float(np.sum(wu.astype(np.float64) ** 2))
        assert abs(parts[i].sum() - want) <= 1e-12 * want
    for b in bd + gd + [U, fro, table]:
        b.free()


@pytest.mark.parametrize("K,N", [(128, 256), (256, 128), (192, 192)])
@pytest.mark.parametrize("sr", [0, 1])
def test_update_multi_refreshes_the_transposed_copy(gpu, K, N, sr):
    """With `p16t` set in the descriptor, the update leaves p16t == p16^T bit for bit (what a
    separate transpose launch after the step would leave), p32 and p16 exactly as without it;
    a weight with p16t = 0 in the same table is untouched by the new path."""
    import ctypes as C
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd._lib import api, MuonDesc
    from ancora_cutile_amd.devbuf import upload_table
    rng = np.random.default_rng(7 * K + N + sr)
    E = 3
    M, Nn = min(K, N), max(K, N)
    tr = int(K > N)
    Ws = [(0.05 * rng.standard_normal((K, N))).astype(np.float32) for _ in range(E)]
    Os = [rng.standard_normal((K, N)).astype(np.float32) for _ in range(E)]
    U = DevBuf(np.stack([np.ascontiguousarray(o.T) if tr else o for o in Os]).reshape(E * M, Nn))
    p32 = [DevBuf(w) for w in Ws]
    p16 = [DevBuf.zeros((K, N), np.uint16) for _ in range(E)]
    p16t = [DevBuf.zeros((N, K), np.uint16) for _ in range(E - 1)]
    descs, blk0 = [], 0
    for i in range(E):
        descs.append(MuonDesc(0, 0, p32[i].ptr, p16[i].ptr, U.ptr + i * M * Nn * 4, K, N, tr, _lib.F32, 0,
                              11 * i, blk0, p16t[i].ptr if i < E - 1 else 0))
        blk0 += K * N // 4096
    table = upload_table(descs)
    lr, seed_base = 0.02, 1234
    scales = (C.c_float * _lib.MUON_MAX_SCALES)(*([lr * shape_scale(K, N)] * _lib.MUON_MAX_SCALES))
    api.anc_muon_update_multi(table.ptr, E, blk0, scales, _lib.F32, sr, seed_base, 0, 0)
    for i in range(E):
        want = muon_update(Ws[i], Os[i], lr)
        assert bits_equal(p32[i].to_numpy(), want)
        w16 = (bf16_sr_bits(want, seed_base + 11 * i) if sr else bf16_rne_bits(want)).reshape(K, N)
        assert bits_equal(p16[i].to_numpy(), w16)
        if i < E - 1:
            assert np.array_equal(p16t[i].to_numpy(), w16.T)
    for b in p32 + p16 + p16t + [U, table]:
        b.free()
