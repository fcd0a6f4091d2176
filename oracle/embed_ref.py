"""Sorted-scatter embedding gradient and its group arrays, restated in numpy.
Test infrastructure only.

Pinned by tests/test_oracle_embed.py: the group arrays through their defining properties
(permutation, non-decreasing ids, original order inside a group, counts), the sum through an
exact case (small integers, where any association order gives the same fp32 value as an integer
sum) and the reference's own gate against an fp64 scatter-add
(tests/kernels/test_embed_dw_scatter.py:55-61, rel < 5e-5)."""
import numpy as np

from .bf16_ref import bits_to_f32


def id_groups(ids_flat):
    """(srt, start, cnt, gid) as ancora/kernels/fused.py:411-424 builds them, unpadded: srt is the
    stable argsort of the ids; group g covers srt[start[g] : start[g] + cnt[g]], all with id gid[g]."""
    ids = np.asarray(ids_flat).reshape(-1)
    srt = np.argsort(ids, kind="stable").astype(np.int32)
    sids = ids[srt]
    starts = np.concatenate(([0], np.nonzero(np.diff(sids))[0] + 1)).astype(np.int32)
    counts = np.diff(np.concatenate((starts, [ids.size]))).astype(np.int32)
    return srt, starts, counts, sids[starts].astype(np.int32)


def embed_dw_rows(ids_flat, dy_bits):
    """Per group, the fp32 sum of its dy rows (bf16 bits -> fp32) added one after the other in
    sorted order starting from zero (the loop of ancora/kernels/fused.py:402-407). Returns
    (gid, rows) with rows (n_groups, H) fp32."""
    dy = bits_to_f32(np.asarray(dy_bits)).reshape(np.shape(dy_bits))
    srt, starts, counts, gid = id_groups(ids_flat)
    rows = np.zeros((gid.size, dy.shape[1]), np.float32)
    for g in range(gid.size):
        acc = np.zeros(dy.shape[1], np.float32)
        for r in range(counts[g]):
            acc = acc + dy[srt[starts[g] + r]]
        rows[g] = acc
    return gid, rows


def embed_dw_scatter(ids_flat, dy_bits, out):
    """out[gid[g]] += rows[g] (fused.py:408): returns the new (V, H) fp32 array."""
    gid, rows = embed_dw_rows(ids_flat, dy_bits)
    out = np.array(out, dtype=np.float32, copy=True)
    out[gid] = out[gid] + rows
    return out
