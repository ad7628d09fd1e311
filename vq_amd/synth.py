"""Seeded synthetic inputs of the benchmark configurations, and index streams.

The reference's generators use the `rand` crate (not reproducible here), so the inputs are
numpy Generator(PCG64) draws with the seeds the configurations name; oracle and GPU always
receive the same byte-identical buffers and the same index streams.
"""
import numpy as np

F = np.float32


def uniform(n, dim, seed):
    """i.i.d. U[0,1) rows (the reference's eval data, src/bin/utils.rs:31-41)."""
    return np.random.default_rng(seed).random((n, dim), dtype=F)


def gaussian_mixture(n, dim, n_centers, sigma, seed, centers="uniform"):
    rng = np.random.default_rng(seed)
    if centers == "uniform":
        c = rng.random((n_centers, dim), dtype=F)
    else:
        c = rng.standard_normal((n_centers, dim), dtype=F)
    lab = rng.integers(0, n_centers, n)
    x = c[lab]
    x += rng.standard_normal((n, dim), dtype=F) * F(sigma)
    return np.ascontiguousarray(x, F)


def unit_rows(n, dim, seed):
    x = np.random.default_rng(seed).standard_normal((n, dim), dtype=F)
    x /= np.sqrt((x.astype(np.float64) ** 2).sum(1, keepdims=True)).astype(F)
    return np.ascontiguousarray(x, F)


def index_streams(n, m, k, max_iters, seed):
    """k distinct initial rows and k*max_iters re-seed draws for each of m problems."""
    rng = np.random.default_rng([seed, 0x1b6])
    init = np.stack([rng.choice(n, k, replace=False) for _ in range(m)]).astype(np.uint32)
    reseed = rng.integers(0, n, (m, max(1, k * max_iters))).astype(np.uint32)
    return init, reseed
