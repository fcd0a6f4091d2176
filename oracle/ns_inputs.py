"""Input families for examining the bf16 Newton-Schulz chain's gates, each with one knob that
moves a matrix across a threshold of the plan. Test infrastructure only (numpy).

proxy = N * ||offdiag(X X^T)||_F^2 at ||X||_F = 1 is the statistic the chain gates on
(csrc/ns.hip: k_ns_cond); colc and bulk are its column statistics (k_ns_colstat)."""
import numpy as np

f32 = np.float32


def proxy_of(X):
    """The conditioning proxy in fp64 (the chain computes it from bf16 values: same to 3 digits)."""
    X = np.asarray(X, dtype=np.float64)
    X = X / np.linalg.norm(X)
    A = X @ X.T
    return X.shape[1] * float(np.sum(A * A) - np.sum(np.diag(A) ** 2))


def scaled_columns(M, N, sigma, seed=0):
    """Independent entries, columns scaled by exp(sigma z): proxy about exp(4 sigma^2), colc = proxy."""
    rng = np.random.default_rng(seed)
    g = rng.standard_normal((M, N)).astype(f32)
    return g * np.exp(sigma * rng.standard_normal(N)).astype(f32)[None, :]


def duplicated_rows(M, N, frac, seed=0):
    """A fraction of the rows are near-copies (1 % noise) of other rows: a gap in the spectrum with
    flat column norms; proxy about 1 + 2 frac N / M."""
    rng = np.random.default_rng(seed)
    g = rng.standard_normal((M, N)).astype(f32)
    k = int(round(frac * M / 2))
    g[M - k:] = g[:k] + f32(0.01) * g[M - k:]
    return g


def gap_scaled_columns(M, N, frac, sigma, seed=0):
    """`duplicated_rows` with its columns scaled by exp(sigma z): the gap raises the proxy and leaves
    the column concentration alone, the scaling raises both by the same amount."""
    scale = np.exp(sigma * np.random.default_rng(seed + 1).standard_normal(N)).astype(f32)
    return duplicated_rows(M, N, frac, seed) * scale[None, :]


def unexplained_proxy(X):
    """proxy - colc in fp64 over all rows: the part of the proxy the column norms do not explain
    (the chain samples every fourth row for colc: flat columns then read 0.006 more)."""
    X = np.asarray(X, dtype=np.float64)
    c2 = np.sum(X * X, axis=0)
    return proxy_of(X) - X.shape[1] * float(np.sum(c2 * c2)) / float(np.sum(c2)) ** 2


def log_spectrum(M, N, decades, seed=0):
    """Singular values log-uniform over `decades` decades, random singular vectors."""
    rng = np.random.default_rng(seed)
    U, _ = np.linalg.qr(rng.standard_normal((M, M)))
    V, _ = np.linalg.qr(rng.standard_normal((N, M)))
    s = np.logspace(0.0, -decades, M)
    return ((U * s) @ V.T).astype(f32)


def outlier_columns(M, N, n_cols, factor, seed=0):
    """Independent entries with n_cols columns scaled by `factor`."""
    rng = np.random.default_rng(seed)
    g = rng.standard_normal((M, N)).astype(f32)
    g[:, rng.choice(N, n_cols, replace=False)] *= f32(factor)
    return g


def low_rank_plus_columns(M, N, rank, noise, n_cols, factor, seed=0):
    """A rank-`rank` signal over `noise` x independent entries, plus n_cols outlier columns: the knob
    `factor` moves the column concentration between that of the signal (about 1) and the proxy."""
    rng = np.random.default_rng(seed)
    g = rng.standard_normal((M, N)).astype(f32)
    x = (rng.standard_normal((M, rank)) @ rng.standard_normal((rank, N))).astype(f32) + f32(noise) * g
    x[:, rng.choice(N, n_cols, replace=False)] *= f32(factor)
    return x


def solve_knob(make, target, lo, hi, stat=proxy_of, iters=18):
    """The knob value in [lo, hi] at which stat(make(knob)) = target (stat increasing in the knob)."""
    for _ in range(iters):
        mid = 0.5 * (lo + hi)
        if stat(make(mid)) < target:
            lo = mid
        else:
            hi = mid
    return 0.5 * (lo + hi)
