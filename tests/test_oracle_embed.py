"""Pins of oracle/embed_ref.py and of the host-side group builder (CPU only)."""
import numpy as np

from oracle.bf16_ref import bf16_rne_bits, bits_to_f32
from oracle.embed_ref import id_groups, embed_dw_rows, embed_dw_scatter


def test_group_arrays_have_their_defining_properties():
    rng = np.random.default_rng(0)
    for M, V in ((512, 2048), (512, 64), (1, 5), (300, 1)):
        ids = rng.integers(0, V, M).astype(np.int32)
        srt, start, cnt, gid = id_groups(ids)
        assert sorted(srt.tolist()) == list(range(M))                  # a permutation
        assert np.all(np.diff(ids[srt]) >= 0)                          # ids non-decreasing
        assert cnt.sum() == M and np.all(cnt > 0) and np.all(np.diff(gid) > 0)
        assert np.array_equal(gid, np.unique(ids))
        for g in range(gid.size):
            seg = srt[start[g]:start[g] + cnt[g]]
            assert np.all(ids[seg] == gid[g]) and np.all(np.diff(seg) > 0)   # original order kept
        assert np.array_equal(cnt, np.bincount(ids, minlength=V)[gid])


def test_host_builder_matches_the_oracle_and_pads():
    from ancora_cutile_amd.embed import build_id_groups
    rng = np.random.default_rng(1)
    ids = rng.integers(0, 97, 400).astype(np.int32)
    srt, start, cnt, gid = build_id_groups(ids)
    o_srt, o_start, o_cnt, o_gid = id_groups(ids)
    U = o_gid.size
    for a in (srt, start, cnt, gid):
        assert a.shape == (400, 1) and a.dtype == np.int32
    assert np.array_equal(srt[:, 0], o_srt)
    assert np.array_equal(start[:U, 0], o_start) and np.array_equal(cnt[:U, 0], o_cnt)
    assert np.array_equal(gid[:U, 0], o_gid) and not cnt[U:].any() and not start[U:].any()


def test_scatter_sum_exact_case_and_reference_gate():
    rng = np.random.default_rng(2)
    M, V, H = 512, 64, 128
    ids = rng.integers(0, V, M).astype(np.int32)
    ints = rng.integers(-8, 9, (M, H)).astype(np.float32)            # exact in bf16, sums exact in fp32
    gid, rows = embed_dw_rows(ids, bf16_rne_bits(ints).reshape(M, H))
    want = np.zeros((V, H), np.int64)
    np.add.at(want, ids, ints.astype(np.int64))
    assert np.array_equal(rows.astype(np.int64), want[gid])
    dyb = bf16_rne_bits(rng.standard_normal((M, H)).astype(np.float32)).reshape(M, H)
    base = (0.1 * rng.standard_normal((V, H))).astype(np.float32)
    got = embed_dw_scatter(ids, dyb, base)
    ref = base.astype(np.float64)
    np.add.at(ref, ids, bits_to_f32(dyb).reshape(M, H).astype(np.float64))
    assert np.abs(got - ref).max() / np.abs(ref).max() < 5e-5      # tests/kernels/test_embed_dw_scatter.py:91
    untouched = np.setdiff1d(np.arange(V), gid)
    assert np.array_equal(got[untouched], base[untouched])
