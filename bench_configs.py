#!/usr/bin/env python3
"""bench_configs.py — device-resident timings of the other full-size configurations.

`bench.py` measures the headline PQ workload; this script times, with the rows already in HBM,
the configurations that are otherwise parity-test cases:

  c3  OPQ   1,000,000 x 128, m = 16, k = 256, 5 outer x 10 LBG iterations, Euclidean
  c4  RVQ   1,000,000 x 256, 8 stages, k = 256, 10 LBG iterations, epsilon = 0
  c5  TSVQ  1,000,000 x 128 unit rows, depth 8; cosine, then Manhattan descent

    python bench_configs.py [c3] [c4] [c5]

Prints one JSON object (milliseconds).  One GPU; inputs are the seeded generators of vq_amd/synth.py.
"""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

F = np.float32


def main():
    import vq_amd
    from vq_amd import synth as data

    which = sys.argv[1:] or ["c4", "c5", "c3"]
    ctx = vq_amd.Context(0)
    out = {}

    def timed(fn, reps=1):
        ctx.sync()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        ctx.sync()
        return (time.perf_counter() - t0) / reps * 1e3

    if "c4" in which:
        n, dim, stages, k, iters = 1_000_000, 256, 8, 256, 10
        x = data.gaussian_mixture(n, dim, 4096, 0.1, seed=7, centers="normal")
        init, reseed = data.index_streams(n, stages, k, iters, seed=7)
        dx = ctx.to_device(x)
        dres = ctx.empty((n, dim), F)
        dcb = ctx.empty((stages, k, dim), F)
        dcodes = ctx.empty(n, np.uint8)

        def rvq_fit():  # ResidualQuantizer::fit, src/rvq.rs:87-154
            ctx.copy_f32(dres, dx, n * dim)
            for st in range(stages):
                cbp = dcb.ptr + st * k * dim * 4
                ctx.lbg_fit(dres, n, dim, 1, dim, k, iters, init[st], reseed[st], cbp)
                ctx.assign(vq_amd.EUCLIDEAN, dres, n, dim, 1, dim, k, cbp, dcodes)
                ctx.residual_sub(dres, n, dim, dim, k, cbp, dcodes)
                # (epsilon = 0: the mean residual norm, src/rvq.rs:131-141, cannot stop the fit and is skipped,
                # as the host class does)

        rvq_fit()  # first call: workspace allocations
        each = [round(timed(rvq_fit), 3) for _ in range(3)]  # (the clock is still ramping during the first)
        out["c4_rvq_fit_ms"] = min(each[1:])
        out["c4_rvq_fit_ms_each"] = each
        dall = ctx.empty((n, stages), np.uint8)
        drec = ctx.empty((n, dim), np.uint16)
        enc = lambda: ctx.rvq_encode(vq_amd.EUCLIDEAN, dx, n, dim, dim, stages, k, dcb, 0.0, dall, None, drec)
        enc()
        out["c4_rvq_encode_ms"] = timed(enc)
        out["c4_recheck_fraction_last_stage"] = ctx.last_recheck_count() / n
        allc, two = ctx.last_recheck_split()
        out["c4_recheck_all_centroids_fraction"] = allc / n
        out["c4_recheck_two_candidates_fraction"] = two / n
        one = lambda: ctx.assign(vq_amd.EUCLIDEAN, dx, n, dim, 1, dim, k, dcb.ptr, dcodes)
        ctx.set_assign_path(1)
        one()
        out["c4_assign_pass_vector_alu_ms"] = timed(one)
        ctx.set_assign_path(0)
        one()
        out["c4_assign_pass_matrix_cores_ms"] = timed(one, 3)
        norm = lambda: ctx.mean_l2norm(dres, n, dim, dim)
        norm()
        out["c4_mean_residual_norm_ms"] = timed(norm, 3)
        del dx, dres, dall, drec
    if "c5" in which:
        n, dim, depth = 1_000_000, 128, 8
        x = data.unit_rows(n, dim, seed=3)
        dx = ctx.to_device(x)
        ctx.tsvq_build(dx, n, dim, dim, depth).free()  # first call: workspace allocations
        builds = []
        for _ in range(4):  # (the clock is still ramping during the first of them)
            ctx.sync()
            t0 = time.perf_counter()
            tree = ctx.tsvq_build(dx, n, dim, dim, depth)
            builds.append((time.perf_counter() - t0) * 1e3)
            if len(builds) < 4:
                tree.free()
        out["c5_tsvq_build_ms"] = sum(builds[1:]) / 3
        out["c5_tsvq_build_ms_each"] = [round(b, 3) for b in builds]
        out["c5_nodes"] = tree.n_nodes
        dleaf = ctx.empty(n, np.int32)
        for name, metric in (("cosine", vq_amd.COSINE), ("manhattan", vq_amd.MANHATTAN)):
            f = lambda: ctx.tsvq_descend(metric, dx, n, dim, tree, dleaf)
            f()
            out[f"c5_descend_{name}_ms"] = timed(f, 3)
        del dx
    if "c3" in which:
        n, dim, m, k, iters, outer = 1_000_000, 128, 16, 256, 10, 5
        from vq_amd import api

        x = data.gaussian_mixture(n, dim, 1024, 0.05, seed=1)
        streams = data.index_streams(n, m, k, iters, seed=1)
        # the first call of a process also pays for the library's first allocations and the clock's ramp
        each = []
        for _ in range(3):
            t0 = time.perf_counter()
            q = api.OptimizedProductQuantizer.fit(x, m, k, iters, outer, api.Distance.Euclidean, 0, streams=streams)
            each.append(round((time.perf_counter() - t0) * 1e3, 3))
        out["c3_opq_fit_host_classes_ms_incl_pack_and_upload"] = min(each[1:])
        out["c3_opq_fit_ms_each"] = each
        R = q.rotation().astype(np.float64)
        out["c3_rotation_orthogonality_err"] = float(np.abs(R.T @ R - np.eye(dim)).max())
        dx = ctx.to_device(x)
        dy = ctx.empty((n, dim), F)
        dR = ctx.to_device(q.rotation())
        f = lambda: ctx.rotate(dx, n, dim, dim, dR, dy)
        f()
        out["c3_rotate_ms"] = timed(f, 5)
        f = lambda: ctx.cross_cov(dy, dx, n, dim)
        f()
        out["c3_cross_cov_ms"] = timed(f, 2)
    print(json.dumps(out, indent=1))


if __name__ == "__main__":
    main()
