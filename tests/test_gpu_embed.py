"""Sorted-scatter embedding gradient (bit-exact against the sequential fp32 sum, the shapes of
tests/kernels/test_embed_dw_scatter.py:96-98) and the row-sparse AdamW (bit-identical to the dense
optimizer on gradients that are zero outside the touched rows)."""
import numpy as np
import pytest

from oracle.adamw_ref import adamw_step_div
from oracle.bf16_ref import bf16_rne_bits, bf16_sr_bits, bits_to_f32
from oracle.embed_ref import embed_dw_rows, embed_dw_scatter as scatter_ref
from util import bits_equal, max_ulp

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,V,H,seed", [(512, 2048, 1024, 0), (512, 64, 1024, 1), (2048, 151936, 1024, 2),
                                        (384, 1000, 192, 3)])
def test_embed_dw_scatter_is_the_sequential_sum(gpu, M, V, H, seed):
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd.embed import IdGroups, embed_dw_scatter
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, V, M).astype(np.int32)
    dyb = bf16_rne_bits(rng.standard_normal((M, H)).astype(np.float32)).reshape(M, H)
    base = (0.1 * rng.standard_normal((V, H))).astype(np.float32)
    grp = IdGroups(ids)
    gdy, out = DevBuf(dyb), DevBuf(base)
    embed_dw_scatter(grp, gdy, 0, out=out)
    got = out.to_numpy()
    assert bits_equal(got, scatter_ref(ids, dyb, base))                 # same association order: same bits
    ref = base.astype(np.float64)
    np.add.at(ref, ids, bits_to_f32(dyb).reshape(M, H).astype(np.float64))
    assert np.abs(got - ref).max() / np.abs(ref).max() < 5e-5           # the reference's own gate
    out.upload(base)
    embed_dw_scatter(grp, gdy, 0, out=out)
    assert bits_equal(out.to_numpy(), got)                              # run to run
    compact = DevBuf.zeros((M, H), np.float32)
    embed_dw_scatter(grp, gdy, 0, compact=compact)
    gid, rows = embed_dw_rows(ids, dyb)
    assert grp.n_groups == gid.size and np.array_equal(grp.host[3][:gid.size, 0], gid)
    assert bits_equal(compact.to_numpy()[:gid.size], rows)
    for b in (gdy, out, compact):
        b.free()
    grp.free()


@pytest.mark.parametrize("sr", [False, True])
def test_row_sparse_adamw_equals_the_dense_optimizer(gpu, sr):
    """Eight steps on a (4096, 256) table; each step's tokens come from a skewed distribution, so
    rows are revisited after gaps of every length and many never; the learning rate changes every
    step. Before each forward the rows about to be gathered are brought up to date and must equal
    the dense oracle's rows; after a final flush all of m, v, the master and the bf16 weights equal
    the dense oracle, and the dense GPU optimizer, bit for bit."""
    from ancora_cutile_amd import AdamW, DevBuf
    from ancora_cutile_amd.adamw import sr_seed_base
    from ancora_cutile_amd.embed import IdGroups, RowSparseAdamW, embed_dw_scatter
    V, H, M, T = 4096, 256, 384, 8
    rng = np.random.default_rng(9)
    W0 = (0.02 * rng.standard_normal((V, H))).astype(np.float32)
    opt = RowSparseAdamW(W0, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=sr, seed=5, tensor_seed=3)
    dense = AdamW({"e": W0}, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=sr, seed=5)
    dense_seed_off = 0                                     # the dense class numbers its tensors from 0
    opt.tensor_seed = dense_seed_off
    p, m, v = W0.copy(), np.zeros_like(W0), np.zeros_like(W0)
    p16 = np.zeros((V, H), np.uint16)
    compact = DevBuf.zeros((M, H), np.float32)
    for t in range(1, T + 1):
        ids = np.minimum((V * rng.random(M) ** 3).astype(np.int32), V - 1)      # skewed: low ids are hot
        lr = 3e-4 * (1.0 + 0.1 * t)
        # forward: the rows it gathers are current
        opt.catch_up(ids, 0)
        u = np.unique(ids)
        got_rows = opt.p32.to_numpy()[u]
        assert max_ulp(got_rows, p[u]) == 0, t
        if t > 1:
            assert bits_equal(opt.p16.to_numpy()[u], p16[u]), t
        # backward: gradient rows by sorted scatter, then the step
        dyb = bf16_rne_bits((1e-2 * rng.standard_normal((M, H))).astype(np.float32)).reshape(M, H)
        grp, gdy = IdGroups(ids), DevBuf(dyb)
        embed_dw_scatter(grp, gdy, 0, compact=compact)
        opt.lr = lr
        opt.step(grp.gid, grp.n_groups, compact, 0)
        # dense oracle on the dense gradient
        gid, rows = embed_dw_rows(ids, dyb)
        G = np.zeros((V, H), np.float32)
        G[gid] = rows
        p, m, v = adamw_step_div(p, m, v, G, lr, 0.9, 0.95, 1e-8, 0.1, t)
        p16 = (bf16_sr_bits(p, (sr_seed_base(5, t) + dense_seed_off) & 0xFFFFFFFF) if sr else bf16_rne_bits(p)).reshape(V, H)
        dense.lr = lr
        dense.step({"e": G}, 0)
        gpu.stream_sync(0)
        gdy.free(); grp.free()
    stale = int(np.count_nonzero(opt.last.to_numpy() < T))
    assert stale > V // 4                                  # most rows really were left behind
    opt.flush(0)
    gpu.stream_sync(0)
    assert max_ulp(opt.p32.to_numpy(), p) == 0 and max_ulp(opt.m.to_numpy(), m) == 0 and max_ulp(opt.v.to_numpy(), v) == 0
    assert bits_equal(opt.p16.to_numpy(), p16)
    ds = dense.st["e"]
    assert bits_equal(opt.p32.to_numpy().ravel(), ds["p32"].to_numpy().ravel())
    assert bits_equal(opt.p16.to_numpy().ravel(), ds["p16"].to_numpy().ravel())
    assert bits_equal(opt.m.to_numpy().ravel(), ds["m"].to_numpy().ravel())
    compact.free(); opt.free(); dense.free()


def test_row_sparse_adamw_skip_and_clip(gpu):
    """A non-finite gradient norm skips the step (no row touched, counter not advanced); a finite one
    clips the gradient rows exactly as the dense kernel does."""
    from ancora_cutile_amd import DevBuf, StepGuard
    from ancora_cutile_amd.embed import RowSparseAdamW
    V, H = 512, 128
    rng = np.random.default_rng(10)
    W0 = (0.02 * rng.standard_normal((V, H))).astype(np.float32)
    opt = RowSparseAdamW(W0, lr=1e-3, wd=0.0)
    rows = np.array([3, 77, 500], np.int32)
    g = rng.standard_normal((3, H)).astype(np.float32)
    gid, grads = DevBuf(rows), DevBuf(g)
    guard = StepGuard(1.0)
    bad = g.copy(); bad[1, 5] = np.inf
    grads.upload(bad)
    guard.compute([grads], 0)
    opt.step(gid, 3, grads, 0, guard=guard)
    assert opt.last_skipped and opt.t == 0 and bits_equal(opt.master(), W0) and not opt.last.to_numpy().any()
    grads.upload(g)
    guard.compute([grads], 0)
    opt.step(gid, 3, grads, 0, guard=guard)
    clip = guard.read(0)["clip_scale"]
    assert not opt.last_skipped and opt.t == 1 and 0 < clip < 1
    want, _, _ = adamw_step_div(W0[rows], 0 * g, 0 * g, g, 1e-3, 0.9, 0.95, 1e-8, 0.0, 1, clip=clip)
    got = opt.master()
    assert max_ulp(got[rows], want) == 0
    keep = np.setdiff1d(np.arange(V), rows)
    assert bits_equal(got[keep], W0[keep])
    for b in (gid, grads):
        b.free()
    guard.free(); opt.free()


def test_row_sparse_adamw_step_table_capacity_and_constant_rate_uploads(gpu, monkeypatch):
    """The step table is written ahead in blocks (one upload per block of steps at a constant
    learning rate, a rewrite when the rate changes), and a step beyond its capacity raises before
    the counter moves, so `t` never runs ahead of the table."""
    from ancora_cutile_amd import DevBuf, _lib
    from ancora_cutile_amd.embed import RowSparseAdamW
    V, H = 256, 64
    rng = np.random.default_rng(1)
    opt = RowSparseAdamW((0.02 * rng.standard_normal((V, H))).astype(np.float32), max_steps=3)
    gid = DevBuf(np.arange(4, dtype=np.int32))
    g = DevBuf((1e-2 * rng.standard_normal((4, H))).astype(np.float32))
    uploads = {"n": 0}
    real = _lib.api.anc_memcpy_h2d
    monkeypatch.setattr(_lib.api, "anc_memcpy_h2d", lambda *a: (uploads.__setitem__("n", uploads["n"] + 1), real(*a))[1])
    opt.step(gid, 4, g, 0)
    opt.step(gid, 4, g, 0)
    assert uploads["n"] == 1                     # both steps' scalars went up with the first
    opt.lr = 1e-4
    opt.step(gid, 4, g, 0)
    assert uploads["n"] == 2 and opt.t == 3
    with pytest.raises(RuntimeError):
        opt.step(gid, 4, g, 0)
    assert opt.t == 3
    monkeypatch.undo()
    tab = opt.table.to_numpy().reshape(-1, 4)
    lrs = tab[1:4, 2].copy().view(np.float32)
    assert lrs[0] == lrs[1] == np.float32(3e-4) and lrs[2] == np.float32(1e-4)
    for b in (gid, g):
        b.free()
    opt.free()


def test_embed_dw_scatter_leaves_out_a_group_with_an_index_outside_the_batch(gpu):
    """A sorted index outside [0, M) cannot name a row of dy: its group writes nothing (it used to
    be served row 0), every other group is the sequential sum as before."""
    from ancora_cutile_amd import DevBuf
    from ancora_cutile_amd.embed import IdGroups, embed_dw_scatter
    M, V, H = 64, 32, 64
    rng = np.random.default_rng(2)
    ids = rng.integers(0, V, M).astype(np.int32)
    dyb = bf16_rne_bits(rng.standard_normal((M, H)).astype(np.float32)).reshape(M, H)
    base = (0.1 * rng.standard_normal((V, H))).astype(np.float32)
    grp = IdGroups(ids)
    want = scatter_ref(ids, dyb, base)
    srt = grp.srt.to_numpy().copy()
    start, gids = grp.host[1].reshape(-1), grp.host[3].reshape(-1)
    victim = 1                                       # break the first sorted index of group 1
    srt[start[victim]] = M + 7
    grp.srt.upload(srt)
    gdy, out = DevBuf(dyb), DevBuf(base)
    embed_dw_scatter(grp, gdy, 0, out=out)
    got = out.to_numpy()
    row = int(gids[victim])
    assert bits_equal(got[row], base[row])
    keep = np.ones(V, bool)
    keep[row] = False
    assert bits_equal(got[keep], want[keep])
    for b in (gdy, out):
        b.free()
    grp.free()
