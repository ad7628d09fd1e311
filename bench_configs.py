#!/usr/bin/env python3
"""bench_configs.py — the other full-size configurations, rows resident in HBM, one GPU.

`bench.py` measures the headline PQ workload and then calls `other_configs()` of this module, so
that its one JSON line also carries, for each of these, the times, the dominant kernel with its
fraction of the peak of the unit that bounds it, and the parity triple (code mismatch
rate, centroid relative L2, reconstruction-MSE relative difference) against the CPU oracle on a
sample the oracle finishes in seconds:

  c3  OPQ   1,000,000 x 128, m = 16, k = 256, 5 outer x 10 LBG iterations, Euclidean
            (protocol of the reference's src/bin/eval_opq.rs; parity after 1, 3 and 5 outer iterations)
  c4  RVQ   1,000,000 x 256, 8 stages, k = 256, 10 LBG iterations, epsilon = 0   (src/bin/eval_rvq.rs)
  c5  TSVQ  1,000,000 x 128 unit rows, depth 8; cosine, then Manhattan descent  (src/bin/eval_tsvq.rs)

    python bench_configs.py [c3] [c4] [c5] [--no-parity]

prints the same object alone; --no-parity leaves out the comparisons with the oracle, so that a
profile of the command holds dispatches of the full-size workloads only.  Inputs are the seeded generators of vq_amd/synth.py.
"""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

F = np.float32
PEAK_HBM_GBS = 8000.0
PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_VALU_TLANESLOTS = 78.6


def _timed(ctx, fn, reps=1):
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    ctx.sync()
    return (time.perf_counter() - t0) / reps * 1e3


def _rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    den = np.sqrt((b ** 2).sum())
    return float(np.sqrt(((a - b) ** 2).sum()) / den) if den else 0.0


def _rel(a, b):
    return float(abs(a - b) / abs(b)) if b else 0.0


def _bfs_order(tree):
    """An oracle tree (pre-order node ids) renumbered breadth-first, left before right: the library's
    numbering.  Returns the tree and the map old id -> new id."""
    order, frontier = [], [0]
    while frontier:
        nxt = []
        for v in frontier:
            order.append(v)
            for c in (tree["left"][v], tree["right"][v]):
                if c >= 0:
                    nxt.append(c)
        frontier = nxt
    new_id = np.full(len(order), -1, np.int32)
    new_id[order] = np.arange(len(order), dtype=np.int32)
    remap = lambda a: np.where(a[order] >= 0, new_id[np.maximum(a[order], 0)], -1).astype(np.int32)
    return dict(n_nodes=len(order), centroids=tree["centroids"][order], left=remap(tree["left"]),
                right=remap(tree["right"]), split_dim=tree["split_dim"][order],
                split_val=tree["split_val"][order], count=tree["count"][order]), new_id


def _kernel_avg(ctx, fn):
    """Average duration (ms) and count of the main assignment kernel's launches inside fn, from the
    start and stop events of the launches themselves."""
    import vq_amd
    ctx.sync()
    ctx.prof_enable(True)
    fn()
    ms, cnt = ctx.prof_read(vq_amd._ffi.PROF_ASSIGN_KERNEL)
    ctx.prof_enable(False)
    return (ms / cnt if cnt else 0.0), cnt


# ---- c3: OPQ ---------------------------------------------------------------------------------
def opq_fit_device(ctx, dx, n, dim, m, k, iters, outer, streams, metric, bufs=None, snapshots=(), trace=None):
    """OptimizedProductQuantizer::fit (src/opq.rs:90-205) on rows already in HBM, the calls of the
    host class (vq_amd/host/vq.hpp) one by one.  Returns (rotation f32, buffers,
    {outer iteration: (rotation, codebooks)} for the iterations named in snapshots).  trace (a list):
    receives (rows the iteration trained on, its codebooks, A, R) of every outer iteration."""
    import vq_amd
    sd = dim // m
    init, reseed = streams
    if bufs is None:
        bufs = dict(rot=ctx.empty((n, dim), F), rec=ctx.empty((n, dim), F), codes=ctx.empty((n, m), np.uint8),
                    cb=ctx.empty((m, k, sd), F), R=ctx.empty((dim, dim), F))
    drot, drec, dcodes, dcb, dR = bufs["rot"], bufs["rec"], bufs["codes"], bufs["cb"], bufs["R"]
    ctx.copy_f32(drot, dx, n * dim)                                         # opq.rs:121
    R = np.eye(dim, dtype=F)
    snaps = {}
    for it in range(outer):
        rows = drot.download() if trace is not None else None
        ctx.lbg_fit(drot, n, dim, m, sd, k, iters, init, reseed, dcb)       # 127-142
        ctx.assign(metric, drot, n, dim, m, sd, k, dcb, dcodes)             # 146-163
        ctx.decode_f32(dcodes, n, m, sd, k, dcb, drec)                      # 164-167
        A = ctx.cross_cov(drec, drot, n, dim).astype(F).astype(np.float64)  # 172-179 (a DMatrix<f32>)
        R = ctx.procrustes_rotation(A).astype(F)                            # 180-183
        dR.upload(R)
        ctx.rotate(dx, n, dim, dim, dR, drot)                               # 186-194
        if it + 1 in snapshots:
            snaps[it + 1] = (R.copy(), dcb.download())
        if trace is not None:
            trace.append((rows, dcb.download(), dcodes.download(), A, R.copy()))
    return R, bufs, snaps


def run_c3(ctx, log, x=None, dx=None, parity=True):
    import vq_amd
    from oracle import oracle as O
    from vq_amd import api
    from vq_amd import synth as data

    n, dim, m, k, iters, outer = 1_000_000, 128, 16, 256, 10, 5
    sd = dim // m
    out = {"workload": "OPQ fit, 1,000,000 x 128 mixture rows (seed 1), m=16, k=256, 5 outer x 10 LBG "
                       "iterations, Euclidean"}
    if x is None:
        x = data.gaussian_mixture(n, dim, 1024, 0.05, seed=1)
    if dx is None:
        dx = ctx.to_device(x)
    streams = data.index_streams(n, m, k, iters, seed=1)
    _, bufs, _ = opq_fit_device(ctx, dx, n, dim, m, k, iters, outer, streams, vq_amd.EUCLIDEAN)  # allocations
    each = []
    for _ in range(2):
        each.append(round(_timed(ctx, lambda: opq_fit_device(ctx, dx, n, dim, m, k, iters, outer, streams,
                                                              vq_amd.EUCLIDEAN, bufs)), 3))
    out["opq_fit_ms"] = min(each)
    out["opq_fit_ms_each"] = each
    avg, cnt = _kernel_avg(ctx, lambda: opq_fit_device(ctx, dx, n, dim, m, k, iters, outer, streams,
                                                       vq_amd.EUCLIDEAN, bufs))
    slots = 2.0 * m * k * n
    out["dominant_kernel"] = {
        "name": "k_assign_mfma_bf (the same kernel as the headline: 5 x (10 LBG passes + 1 reconstruction pass))",
        "bound": "valu", "avg_launch_ms": round(avg, 4), "launches": cnt,
        "achieved": round(slots / (avg * 1e-3) / 1e12, 3) if avg else None, "peak": PEAK_VALU_TLANESLOTS,
        "unit": "T lane-slots/s", "frac": round(slots / (avg * 1e-3) / 1e12 / PEAK_VALU_TLANESLOTS, 4) if avg else None,
        "algorithmic_work": "2*m*k = 8192 selection lane-slots per row and pass"}
    f = lambda: ctx.rotate(dx, n, dim, dim, bufs["R"], bufs["rot"])
    f()
    out["rotate_ms"] = round(_timed(ctx, f, 5), 4)
    out["rotate_hbm_frac"] = round(8.0 * dim * n / (out["rotate_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
    f = lambda: ctx.cross_cov(bufs["rec"], bufs["rot"], n, dim)
    f()
    out["cross_cov_ms_incl_readback"] = round(_timed(ctx, f, 3), 4)
    A = ctx.cross_cov(bufs["rec"], bufs["rot"], n, dim).astype(F).astype(np.float64)
    f = lambda: ctx.procrustes_rotation(A)
    f()
    out["procrustes_rotation_ms"] = round(_timed(ctx, f, 5), 4)
    # through the host classes from a pageable host array: pack, upload, fit (what a caller of the crate's API pays)
    hs = []
    for _ in range(2):
        t0 = time.perf_counter()
        q = api.OptimizedProductQuantizer.fit(x, m, k, iters, outer, api.Distance.Euclidean, 0, streams=streams)
        hs.append(round((time.perf_counter() - t0) * 1e3, 3))
    out["opq_fit_with_upload_ms"] = min(hs)
    out["opq_fit_with_upload_ms_each"] = hs
    R = q.rotation().astype(np.float64)
    out["rotation_orthogonality_err"] = float(np.abs(R.T @ R - np.eye(dim)).max())
    del q
    for b in bufs.values():
        b.free()
    if not parity:
        return out

    # parity against the oracle after 1, 3 and 5 outer iterations, on the first rows of the same data
    ns = 20_000
    xs = np.ascontiguousarray(x[:ns])
    st_s = data.index_streams(ns, m, k, iters, seed=3)
    dxs = ctx.to_device(xs)
    trace = []
    _, sb, snaps = opq_fit_device(ctx, dxs, ns, dim, m, k, iters, outer, st_s, vq_amd.EUCLIDEAN, snapshots=(1, 3, 5),
                                  trace=trace)
    par = {}
    t0 = time.perf_counter()
    for it in (1, 3, 5):
        ref = O.opq_fit(O.EUCLIDEAN, xs, m, k, iters, it, st_s[0], st_s[1])
        Rg, cbg = snaps[it]
        # codes and reconstruction of the sample under each side's own rotation and codebooks
        # (OptimizedProductQuantizer::quantize, src/opq.rs:222-264)
        dRg, dcbg = ctx.to_device(Rg), ctx.to_device(cbg)
        ctx.rotate(dxs, ns, dim, dim, dRg, sb["rot"])
        ctx.assign(vq_amd.EUCLIDEAN, sb["rot"], ns, dim, m, sd, k, dcbg, sb["codes"])
        drec = ctx.empty((ns, dim), np.uint16)
        ctx.decode_f16(sb["codes"], ns, m, sd, k, dcbg, drec)
        codes_g = sb["codes"].download()
        codes_r = O.opq_encode(O.EUCLIDEAN, xs, ref["rotation"], ref["codebooks"]).astype(np.uint8)
        mse_g = O.mse_f16(xs, drec.download())
        mse_r = O.mse_f16(xs, O.pq_decode_f16(codes_r, ref["codebooks"]))
        par[f"outer_{it}"] = {
            "centroid_rel_l2": _rel_l2(cbg, ref["codebooks"]),
            "rotation_max_abs_diff": float(np.abs(Rg.astype(np.float64) - ref["rotation"]).max()),
            "code_mismatch_rate": float(np.mean(codes_g != codes_r)),
            "mse_gpu": mse_g, "mse_ref": mse_r, "mse_rel_diff": _rel(mse_g, mse_r)}
        for b in (dRg, dcbg, drec):
            b.free()
    # Where the difference from the second outer iteration on comes from.  (1) Step by step along the
    # GPU's own trajectory: the oracle, given the rows each outer iteration of the GPU trained on,
    # must reproduce that iteration's codebooks and codes bit for bit and its rotation update to
    # rounding, so nothing but the rotated rows' last bits separates the two runs (the rotation is a
    # tolerance quantity: a matrix product and an SVD whose rounding the reference leaves to
    # nalgebra; the library's product runs on the matrix cores, the oracle's is a sequential sum).
    step = []
    for it, (rows, cbg, codes_g, A_g, R_g) in enumerate(trace):
        ref_cb = O.pq_fit(rows, m, k, iters, st_s[0], st_s[1])["codebooks"]
        ref_codes = O.pq_encode(O.EUCLIDEAN, rows, ref_cb).astype(np.uint8)
        rec = ref_cb[np.arange(m)[None, :], ref_codes.astype(np.int64)].reshape(ns, dim).astype(np.float64)
        A_ref = (rec.T @ rows.astype(np.float64)).astype(F).astype(np.float64)
        step.append({"outer": it + 1,
                     "centroids_bit_identical": bool(np.array_equal(cbg.view(np.uint32), ref_cb.view(np.uint32))),
                     "code_mismatch_rate": float(np.mean(codes_g != ref_codes)),
                     "cross_cov_rel_diff": _rel_l2(A_g, A_ref),
                     "rotation_max_abs_diff_f32": float(np.abs(R_g - O.procrustes(A_ref).astype(F)).max())})
    par["stepwise_from_the_rows_the_gpu_trained_on"] = step
    # (2) The algorithm's own sensitivity: the oracle against itself when every input value moves by
    # at most one unit in the last place (a random half of them up, the other half down) — Lloyd
    # iterations amplify such differences, a row that changes its cluster moves two centroids.
    rng = np.random.default_rng(11)
    up = rng.random(xs.shape) < 0.5
    xp = np.where(up, np.nextafter(xs, F(np.inf)), np.nextafter(xs, F(-np.inf))).astype(F)
    for it in (1, 3, 5):
        a = O.opq_fit(O.EUCLIDEAN, xs, m, k, iters, it, st_s[0], st_s[1])
        b = O.opq_fit(O.EUCLIDEAN, xp, m, k, iters, it, st_s[0], st_s[1])
        ca = O.opq_encode(O.EUCLIDEAN, xs, a["rotation"], a["codebooks"])
        cb_ = O.opq_encode(O.EUCLIDEAN, xs, b["rotation"], b["codebooks"])
        par[f"outer_{it}"]["oracle_vs_oracle_inputs_moved_one_ulp"] = {
            "centroid_rel_l2": _rel_l2(b["codebooks"], a["codebooks"]),
            "code_mismatch_rate": float(np.mean(ca != cb_))}
    par["sample"] = (f"first {ns} rows, own index streams (seed 3); oracle = vqo_opq_fit (host Jacobi SVD), "
                     f"{time.perf_counter() - t0:.1f} s")
    out["parity"] = par
    for b in sb.values():
        b.free()
    dxs.free()
    log(f"[configs] c3 done: fit {out['opq_fit_ms']} ms resident, {out['opq_fit_with_upload_ms']} ms with upload")
    return out


# ---- c4: RVQ ---------------------------------------------------------------------------------
def rvq_fit_device(ctx, dx, dres, dcb, dcodes, n, dim, stages, k, iters, init, reseed, metric, final_residual=False):
    """ResidualQuantizer::fit (src/rvq.rs:87-154) with epsilon = 0, as the host class runs it: the
    mean residual norm (131-141) cannot stop the fit and is skipped, and so is the residual update of
    the last stage, which nothing can observe (the residuals are a local of fit) unless
    final_residual asks for it."""
    ctx.copy_f32(dres, dx, n * dim)
    prev = None  # the codebook of a residual update that rides on the next stage's fit (vq_lbg_fit_residual)
    for st in range(stages):
        cbp = dcb.ptr + st * k * dim * 4
        if prev is None:
            ctx.lbg_fit(dres, n, dim, 1, dim, k, iters, init[st], reseed[st], cbp)
        else:
            ctx.lbg_fit_residual(dres, n, dim, dim, k, iters, init[st], reseed[st], cbp, prev, k, dcodes)
        prev = None
        if st + 1 == stages and not final_residual:
            break
        ctx.assign(metric, dres, n, dim, 1, dim, k, cbp, dcodes)
        if st + 1 < stages:
            prev = cbp
        else:
            ctx.residual_sub(dres, n, dim, dim, k, cbp, dcodes)


def run_c4(ctx, log, parity=True):
    import vq_amd
    from oracle import oracle as O
    from vq_amd import synth as data

    n, dim, stages, k, iters = 1_000_000, 256, 8, 256, 10
    out = {"workload": "RVQ fit + encode, 1,000,000 x 256 rows from 4,096 Gaussians (seed 7), 8 stages, k=256, "
                       "10 LBG iterations, epsilon 0, Euclidean"}
    x = data.gaussian_mixture(n, dim, 4096, 0.1, seed=7, centers="normal")
    init, reseed = data.index_streams(n, stages, k, iters, seed=7)
    dx = ctx.to_device(x)
    dres = ctx.empty((n, dim), F)
    dcb = ctx.empty((stages, k, dim), F)
    dcodes = ctx.empty(n, np.uint8)
    fit = lambda: rvq_fit_device(ctx, dx, dres, dcb, dcodes, n, dim, stages, k, iters, init, reseed, vq_amd.EUCLIDEAN)
    fit()  # first call: workspace allocations
    each = [round(_timed(ctx, fit), 3) for _ in range(2)]
    out["rvq_fit_ms"] = min(each)
    out["rvq_fit_ms_each"] = each
    avg, cnt = _kernel_avg(ctx, fit)
    flop = 2.0 * k * dim * n
    tf = flop / (avg * 1e-3) / 1e12 if avg else 0.0
    out["dominant_kernel"] = {
        "name": "k_assign_mfma_wide_bf (bf16-split scores of 32 rows x 256 centroids per wave, three matrix "
                "instructions per 16 dimensions; 8 x 10 LBG passes + 7 residual passes)",
        "bound": "mfma", "avg_launch_ms": round(avg, 4), "launches": cnt,
        "algorithmic_work": "2*k*D = 131,072 flop per row and pass",
        # the distance sums priced as fp32 matrix work (what the accounting of the path asks for) ...
        "achieved": round(tf, 1), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4),
        # ... and as what is issued on the bf16 units they run on (three bf16 products per fp32 one)
        "issued_bf16_TFLOPs": round(3.0 * tf, 1), "issued_frac_of_bf16_peak": round(3.0 * tf / PEAK_BF16_MFMA_TFLOPS, 4),
        "note": "frac above 1: the fp32-grade scores come from the bf16 matrix units, which the second pair of fields prices"}
    dall = ctx.empty((n, stages), np.uint8)
    drec = ctx.empty((n, dim), np.uint16)
    enc = lambda: ctx.rvq_encode(vq_amd.EUCLIDEAN, dx, n, dim, dim, stages, k, dcb, 0.0, dall, None, drec)
    enc()
    out["rvq_encode_ms"] = round(_timed(ctx, enc, 2), 3)
    allc, two = ctx.last_recheck_split()
    out["recheck_fraction_last_stage"] = {"all_centroids": allc / n, "two_candidates": two / n}
    for b in (dx, dres, dall, drec):
        b.free()
    if not parity:
        dcb.free()
        dcodes.free()
        return out

    # parity on a sample: whole fit and encode against the oracle
    ns, st_s = 20_000, 4
    xs = np.ascontiguousarray(x[:ns])
    del x
    init_s, reseed_s = data.index_streams(ns, st_s, k, iters, seed=8)
    t0 = time.perf_counter()
    ref = O.rvq_fit(O.EUCLIDEAN, xs, st_s, k, iters, 0.0, init_s, reseed_s)
    codes_r, rec_r = O.rvq_quantize(O.EUCLIDEAN, xs, ref["codebooks"], 0.0)
    cpu_s = time.perf_counter() - t0
    dxs = ctx.to_device(xs)
    dres = ctx.empty((ns, dim), F)
    dcbs = ctx.empty((st_s, k, dim), F)
    dc1 = ctx.empty(ns, np.uint8)
    rvq_fit_device(ctx, dxs, dres, dcbs, dc1, ns, dim, st_s, k, iters, init_s, reseed_s, vq_amd.EUCLIDEAN,
                   final_residual=True)
    dall = ctx.empty((ns, st_s), np.uint8)
    drec = ctx.empty((ns, dim), np.uint16)
    ctx.rvq_encode(vq_amd.EUCLIDEAN, dxs, ns, dim, dim, st_s, k, dcbs, 0.0, dall, None, drec)
    cbg = dcbs.download()
    mse_g, mse_r = O.mse_f16(xs, drec.download()), O.mse_f16(xs, rec_r)
    out["parity"] = {
        "sample": f"first {ns} rows, {st_s} stages, own index streams (seed 8); oracle fit + quantize {cpu_s:.1f} s",
        "centroid_rel_l2": _rel_l2(cbg, ref["codebooks"]),
        "centroids_bit_identical": bool(np.array_equal(cbg.view(np.uint32), ref["codebooks"].view(np.uint32))),
        "residual_rel_l2": _rel_l2(dres.download(), ref["residuals"]),
        "code_mismatch_rate": float(np.mean(dall.download() != codes_r.astype(np.uint8))),
        "mse_gpu": mse_g, "mse_ref": mse_r, "mse_rel_diff": _rel(mse_g, mse_r)}
    for b in (dxs, dres, dcbs, dc1, dall, drec, dcb, dcodes):
        b.free()
    log(f"[configs] c4 done: fit {out['rvq_fit_ms']} ms, encode {out['rvq_encode_ms']} ms")
    return out


# ---- c5: TSVQ --------------------------------------------------------------------------------
def run_c5(ctx, log, parity=True):
    import vq_amd
    from oracle import oracle as O
    from vq_amd import synth as data

    n, dim, depth = 1_000_000, 128, 8
    out = {"workload": "TSVQ build (median split on the maximum-variance coordinate, src/tsvq.rs:71-148) + "
                       "descent, 1,000,000 x 128 unit rows (seed 3), depth 8; cosine, then Manhattan"}
    x = data.unit_rows(n, dim, seed=3)
    dx = ctx.to_device(x)
    ctx.tsvq_build(dx, n, dim, dim, depth).free()  # first call: workspace allocations
    builds = []
    tree = None
    for i in range(4):  # (the clock is still ramping during the first of them)
        ctx.sync()
        t0 = time.perf_counter()
        tree = ctx.tsvq_build(dx, n, dim, dim, depth)
        builds.append((time.perf_counter() - t0) * 1e3)
        if i < 3:
            tree.free()
    out["tsvq_build_ms"] = round(sum(builds[1:]) / 3, 3)
    out["tsvq_build_ms_each"] = [round(b, 3) for b in builds]
    out["nodes"] = tree.n_nodes
    # three passes over the rows per level (node sums, squared deviations, maps) + the partition's gather
    out["tsvq_build_hbm_frac"] = round(depth * 3.0 * 4.0 * dim * n / (out["tsvq_build_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
    dleaf = ctx.empty(n, np.int32)
    bytes_row = 4.0 * dim + 1.0
    for name, metric in (("cosine", vq_amd.COSINE), ("manhattan", vq_amd.MANHATTAN)):
        f = lambda: ctx.tsvq_descend(metric, dx, n, dim, tree, dleaf)
        f()
        ms = _timed(ctx, f, 5)
        out[f"descend_{name}_ms"] = round(ms, 4)
        gbs = bytes_row * n / (ms * 1e-3) / 1e9
        out[f"descend_{name}_roofline"] = {
            "kernel": "k_tsvq_descend_w (one inner product per node, the two distances where it cannot decide)"
                      if metric == vq_amd.COSINE else "k_tsvq_descend_reg (two distances per node)", "bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
            "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
            "algorithmic_bytes": "4*D + 1 = 513 per row"}
    tree.free()
    # The configuration's wording ("2-means with 10 LBG iterations per node") as the explicit,
    # non-default mode: the split is lbg_quantize with k = 2 instead of the reference's median split.
    lbg_iters = 10
    draws = np.random.default_rng(5).integers(0, 2 ** 32, (2 ** depth - 1, 2 + lbg_iters), dtype=np.uint64).astype(np.uint32)
    ctx.tsvq_build_kmeans(dx, n, dim, dim, depth, lbg_iters, draws).free()
    kb = []
    for i in range(3):
        ctx.sync()
        t0 = time.perf_counter()
        tk = ctx.tsvq_build_kmeans(dx, n, dim, dim, depth, lbg_iters, draws)
        kb.append(round((time.perf_counter() - t0) * 1e3, 3))
        if i < 2:
            tk.free()
    out["kmeans_mode"] = {"note": "explicit non-default mode (vq_tsvq_build_kmeans): 2-means split with 10 LBG iterations "
                                  "per node; not the reference's behaviour (src/tsvq.rs:87-123 splits at the median)",
                          "tsvq_build_ms": min(kb), "tsvq_build_ms_each": kb, "nodes": tk.n_nodes}
    f = lambda: ctx.tsvq_descend(vq_amd.COSINE, dx, n, dim, tk, dleaf)
    f()
    out["kmeans_mode"]["descend_cosine_ms"] = round(_timed(ctx, f, 5), 4)
    tk.free()
    dx.free()
    dleaf.free()
    if not parity:
        return out

    # parity on a sample: whole build and both descents against the oracle
    ns = 200_000
    xs = np.ascontiguousarray(x[:ns])
    del x
    t0 = time.perf_counter()
    ref_pre = O.tsvq_fit(xs, depth)
    cpu_s = time.perf_counter() - t0
    ref, new_id = _bfs_order(ref_pre)
    dxs = ctx.to_device(xs)
    tg = ctx.tsvq_build(dxs, ns, dim, dim, depth)
    g = tg.download()
    par = {"sample": f"first {ns} rows; oracle build {cpu_s:.1f} s",
           "nodes_equal": bool(g["n_nodes"] == ref["n_nodes"]),
           "tree_structure_equal": bool(g["n_nodes"] == ref["n_nodes"] and np.array_equal(g["left"], ref["left"])
                                        and np.array_equal(g["right"], ref["right"])
                                        and np.array_equal(g["split_dim"], ref["split_dim"])),
           "centroid_rel_l2": _rel_l2(g["centroids"], ref["centroids"]) if g["n_nodes"] == ref["n_nodes"] else None,
           "centroids_bit_identical": bool(g["n_nodes"] == ref["n_nodes"] and np.array_equal(
               g["centroids"].view(np.uint32), ref["centroids"].view(np.uint32)))}
    dl = ctx.empty(ns, np.int32)
    dre = ctx.empty((ns, dim), np.uint16)
    for name, metric, om in (("cosine", vq_amd.COSINE, O.COSINE), ("manhattan", vq_amd.MANHATTAN, O.MANHATTAN)):
        ctx.tsvq_descend(metric, dxs, ns, dim, tg, dl)
        ctx.tsvq_decode_f16(tg, dl, ns, dre)
        leaf_r = new_id[O.tsvq_descend(om, xs, ref_pre)]
        rec_r = O.f32_to_f16_bits(ref["centroids"][leaf_r])
        mse_g, mse_r = O.mse_f16(xs, dre.download()), O.mse_f16(xs, rec_r)
        par[name] = {"leaf_mismatch_rate": float(np.mean(dl.download() != leaf_r)),
                     "mse_gpu": mse_g, "mse_ref": mse_r, "mse_rel_diff": _rel(mse_g, mse_r)}
    tg.free()
    # the 2-means mode on a smaller sample (the oracle runs ten LBG iterations per node)
    nk = 50_000
    xk = np.ascontiguousarray(xs[:nk])
    t0 = time.perf_counter()
    rk, _ = _bfs_order(O.tsvq_fit_kmeans(xk, depth, lbg_iters, draws))
    cpu_k = time.perf_counter() - t0
    dxk = ctx.to_device(xk)
    gk_tree = ctx.tsvq_build_kmeans(dxk, nk, dim, dim, depth, lbg_iters, draws)
    gk = gk_tree.download()
    same = gk["n_nodes"] == rk["n_nodes"]
    par["kmeans_mode"] = {
        "sample": f"first {nk} rows; oracle build {cpu_k:.1f} s",
        "tree_structure_equal": bool(same and np.array_equal(gk["left"], rk["left"]) and np.array_equal(gk["right"], rk["right"])),
        "centroid_rel_l2": _rel_l2(gk["centroids"], rk["centroids"]) if same else None,
        "centroids_bit_identical": bool(same and np.array_equal(gk["centroids"].view(np.uint32),
                                                                rk["centroids"].view(np.uint32)))}
    gk_tree.free()
    dxk.free()
    out["parity"] = par
    for b in (dxs, dl, dre):
        b.free()
    log(f"[configs] c5 done: build {out['tsvq_build_ms']} ms, descent {out['descend_cosine_ms']} / "
        f"{out['descend_manhattan_ms']} ms")
    return out


def other_configs(ctx, log, which=("c3", "c4", "c5"), x_c2=None, dx_c2=None, parity=True):
    out = {}
    if "c3" in which:
        out["c3_opq"] = run_c3(ctx, log, x_c2, dx_c2, parity)
    if "c4" in which:
        out["c4_rvq"] = run_c4(ctx, log, parity)
    if "c5" in which:
        out["c5_tsvq"] = run_c5(ctx, log, parity)
    return out


def main():
    import vq_amd
    args = sys.argv[1:]
    parity = "--no-parity" not in args  # full-size dispatches only: what the profiles are taken with
    which = [a for a in args if not a.startswith("--")] or ["c3", "c4", "c5"]
    ctx = vq_amd.Context(0)
    print(json.dumps(other_configs(ctx, lambda *a: print(*a, file=sys.stderr, flush=True), which, parity=parity), indent=1))


if __name__ == "__main__":
    main()
