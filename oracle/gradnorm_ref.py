"""Global gradient norm, clip scale and skip flag. Test infrastructure only.

The reference has no gradient norm (a grep for grad-norm / clip / isnan over ancora/ finds
only quantizer np.clip calls), so the semantics are build-defined:
    sumsq = sum over every gradient element of g*g        (fp64)
    norm  = float32(sqrt(sumsq))
    clip  = min(1, max_norm / (norm + eps))   in fp32     (1 when max_norm <= 0)
    skip  = sumsq is not finite
`gradnorm_f64` is the closed form the parity bar (<= 1 ulp of fp32 on norm) is measured
against. `gradnorm_fixed` restates the library's fixed reduction order operation by
operation and therefore matches the device bit for bit.
"""
import numpy as np

CHUNK = 8192
_XOR = np.arange(64)


def _as_f32(g):
    g = np.asarray(g)
    if g.dtype == np.uint16:   # bf16 bit patterns
        return (g.astype(np.uint32) << np.uint32(16)).view(np.float32).reshape(-1)
    return np.ascontiguousarray(g, dtype=np.float32).reshape(-1)


def gradnorm_f64(grads):
    """sumsq as an fp64 sum over all elements of all gradients."""
    s = 0.0
    for g in grads:
        x = _as_f32(g).astype(np.float64)
        s += float(np.sum(x * x))
    return s


def _butterfly(v):
    """xor butterfly over 64 lanes, offsets 32..1: lane l gets v[l] + v[l ^ off]."""
    for off in (32, 16, 8, 4, 2, 1):
        v = v + v[..., _XOR ^ off]
    return v[..., 0]


def chunk_partials(g):
    """fp64 partial of every 8192-element chunk of one tensor, in the library's order:
    lane t of 256 takes, for j = 0..3, the 8 consecutive elements of vector j*256 + t, sums
    their squares left to right in fp32, widens to fp64 and accumulates over j; wavefronts
    are reduced by the butterfly; the 4 wavefront sums are added in order."""
    x = _as_f32(g)
    n_chunks = (x.size + CHUNK - 1) // CHUNK
    pad = np.zeros(n_chunks * CHUNK, np.float32)
    pad[:x.size] = x
    v = pad.reshape(n_chunks, 4, 256, 8)                    # chunk, j, lane, k
    sq = v * v
    s = sq[..., 0]
    for k in range(1, 8):
        s = s + sq[..., k]                                  # fp32, left to right
    acc = np.zeros((n_chunks, 256), np.float64)
    for j in range(4):
        acc = acc + s[:, j, :].astype(np.float64)
    w = _butterfly(acc.reshape(n_chunks, 4, 64))            # chunk, wavefront
    t = w[:, 0]
    for k in range(1, 4):
        t = t + w[:, k]
    return t


def finalize_fixed(partials):
    """Stage 2: lane t of 1024 adds partials t, t+1024, ... in order; butterfly per
    wavefront; the 16 wavefront sums are added in order."""
    p = np.asarray(partials, dtype=np.float64)
    rounds = (p.size + 1023) // 1024
    pad = np.zeros(rounds * 1024, np.float64)
    pad[:p.size] = p
    acc = np.zeros(1024, np.float64)
    for r in range(rounds):
        acc = acc + pad[r * 1024:(r + 1) * 1024]
    w = _butterfly(acc.reshape(16, 64))
    t = w[0]
    for k in range(1, 16):
        t = t + w[k]
    return float(t)


def gradnorm_fixed(grads):
    """sumsq in the library's fixed order: per-tensor chunk partials, concatenated in tensor
    order, then the fixed stage-2 reduction."""
    return finalize_fixed(np.concatenate([chunk_partials(g) for g in grads]))


def control(sumsq, max_norm=1.0, eps=1e-6):
    """{norm, clip_scale, skip} from sumsq, in the library's fp32 arithmetic."""
    finite = bool(np.isfinite(sumsq))
    with np.errstate(invalid="ignore"):
        norm = np.float32(np.sqrt(np.float64(sumsq)))
    clip = np.float32(1.0)
    if finite and max_norm is not None and max_norm > 0:
        s = np.float32(max_norm) / (norm + np.float32(eps))
        clip = s if s < np.float32(1.0) else np.float32(1.0)
    return {"sumsq": float(sumsq), "norm": float(norm), "clip_scale": float(clip),
            "skip": not finite}
