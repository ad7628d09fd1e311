#!/usr/bin/env python3
"""Evaluation harness in the reference's protocol, on the GPU path.

Mirrors `src/bin/eval_{pq,opq,rvq,tsvq}.rs` and `src/bin/utils.rs` of the reference: synthetic
uniform [0,1) rows, one timed `fit` / `new`, one timed quantize-all, mean squared reconstruction
error, recall@10, and a CSV with the reference's columns
(`n_samples,n_dims,training_time_ms,quantization_time_ms,reconstruction_error,recall`,
`src/bin/eval_pq.rs:103-119`).  The data generator is numpy's (the reference's `rand` stream is not
reproducible outside Rust), so figures agree with the published ones statistically, not bit by bit.

    python -m vq_amd.eval --eval pq --samples 1000 10000 --out eval_pq_results.csv
"""
import argparse
import sys
import time

import numpy as np

# src/bin/utils.rs:11-16
SEED = 66
NUM_SAMPLES = [1_000, 5_000, 10_000, 50_000, 100_000]
DIM = 128
M = 16
K = 256
MAX_ITERS = 10
# src/bin/eval_opq.rs:42, src/bin/eval_rvq.rs:22-23, src/bin/eval_tsvq.rs:22
OPQ_ITERS = 5
RVQ_STAGES = 4
RVQ_EPSILON = 0.01
TSVQ_MAX_DEPTH = 10
FIT_SEED = 42  # src/bin/eval_pq.rs:41


def generate_synthetic_data(n_samples, n_dims, seed):
    """Uniform [0,1) rows (src/bin/utils.rs:31-41)."""
    return np.random.default_rng(seed).random((n_samples, n_dims), dtype=np.float32)


def calculate_reconstruction_error(original, reconstructed):
    """sum((x - y)^2) / (N * D) (src/bin/utils.rs:50-67); the differences are f32 as in the
    reference, the sum is carried in f64 so that its order does not matter."""
    d = original.astype(np.float32) - reconstructed.astype(np.float32)
    return float((d.astype(np.float64) ** 2).sum() / d.size)


def calculate_recall(original, approx, k):
    """recall@k of the reference (src/bin/utils.rs:70-127): at most 1000 strided queries, each
    searched in a window of 5000 rows around it when there are more than 10,000 rows; neighbours
    by Euclidean distance among the original rows and among the reconstructed rows; ties keep
    the index order (stable sort)."""
    n = len(original)
    eval_samples = min(n, 1000)
    step = max(n // eval_samples, 1)
    window = 5000 if n > 10_000 else n
    total = 0.0
    for i in range(0, n, step):
        start = i - window // 2 if i > window // 2 else 0
        end = min(i + window // 2, n)
        idx = np.arange(start, end)
        idx = idx[idx != i]

        def nearest(rows):
            d = np.sqrt(((rows[idx] - rows[i]) ** 2).sum(axis=1, dtype=np.float32))
            return set(idx[np.argsort(d, kind="stable")[:k]].tolist())

        total += len(nearest(original) & nearest(approx)) / k
    return total / (n // step)


def run_benchmark(alg, n_samples, n_dims=DIM, m=M, k=K, max_iters=MAX_ITERS):
    from . import api
    data = generate_synthetic_data(n_samples, n_dims, SEED)
    dist = api.Distance.Euclidean
    t0 = time.perf_counter()
    if alg == "pq":
        q = api.ProductQuantizer.fit(data, m, k, max_iters, dist, FIT_SEED)
    elif alg == "opq":
        q = api.OptimizedProductQuantizer.fit(data, m, k, max_iters, OPQ_ITERS, dist, FIT_SEED)
    elif alg == "rvq":
        q = api.ResidualQuantizer.fit(data, RVQ_STAGES, k, max_iters, RVQ_EPSILON, dist, FIT_SEED)
    elif alg == "tsvq":
        q = api.TSVQ.new(data, TSVQ_MAX_DEPTH, dist)
    else:
        raise ValueError(f"unknown algorithm {alg!r}")
    training_time_ms = (time.perf_counter() - t0) * 1e3
    t0 = time.perf_counter()
    reconstructed = q.quantize_batch(data).astype(np.float32)  # Vector<f16> -> f32, eval_pq.rs:51-59
    quantization_time_ms = (time.perf_counter() - t0) * 1e3
    return {
        "n_samples": n_samples,
        "n_dims": n_dims,
        "training_time_ms": training_time_ms,
        "quantization_time_ms": quantization_time_ms,
        "reconstruction_error": calculate_reconstruction_error(data, reconstructed),
        "recall": calculate_recall(data, reconstructed, 10),
    }


COLUMNS = ["n_samples", "n_dims", "training_time_ms", "quantization_time_ms", "reconstruction_error", "recall"]


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--eval", required=True, choices=["pq", "opq", "rvq", "tsvq"])
    ap.add_argument("--samples", type=int, nargs="*", default=NUM_SAMPLES)
    ap.add_argument("--out", default=None, help="CSV file (default: stdout)")
    args = ap.parse_args(argv)
    rows = []
    for n in args.samples:
        r = run_benchmark(args.eval, n)
        print(f"[{args.eval}] {n} samples: train {r['training_time_ms']:.2f} ms, quantize "
              f"{r['quantization_time_ms']:.2f} ms, error {r['reconstruction_error']:.6f}, "
              f"recall@10 {r['recall']:.4f}", file=sys.stderr, flush=True)
        rows.append(r)
    out = open(args.out, "w") if args.out else sys.stdout
    print(",".join(COLUMNS), file=out)
    for r in rows:
        print(",".join(str(r[c]) for c in COLUMNS), file=out)
    if args.out:
        out.close()


if __name__ == "__main__":
    main()
