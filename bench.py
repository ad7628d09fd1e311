#!/usr/bin/env python3
"""bench.py — PQ fit + encode throughput on one MI355X, with roofline and CPU baseline.

One step = ProductQuantizer::fit (10 LBG iterations) followed by the encode of every row
(the headline configuration: 1,000,000 x 128 f32 rows from a mixture of 1,024 isotropic Gaussians,
m = 16, k = 256, Euclidean encode), with the rows already resident in HBM.

Prints ONE JSON line:
  value        rows / second over fit + encode (whole job, one GPU)
  roofline     the dominant kernel (the assignment pass) against the bound that binds it, the
               vector ALU: algorithmic selection lane-slots per second over the issue peak; its
               time is measured with HIP events on the library's stream (the start and stop
               events of each launch's own dispatch) during the timed steps; the matrix-core and
               HBM views of the same time and the floor set by the selection's instructions at
               their measured issue rate are secondary fields
  end_to_end   one pass pageable host rows -> upload -> fit -> encode -> codes on the host
  calibration  measured peaks of the box: plain-copy HBM rate, vector instruction issue rates
  cpu_baseline the C restatement of the reference (oracle/) timed on the host cores on the same
               workload with the same index streams; `parity` compares its codebooks and codes with
               the buffers the timed steps wrote
  other_configs  after the headline measurement: the OPQ, RVQ and TSVQ configurations at full size
               (bench_configs.py), each with its times, its dominant kernel against its bound and
               the parity triple against the oracle on a sample
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N_ROWS, DIM, M, K, ITERS = 1_000_000, 128, 16, 256, 10
PEAK_FP32_MFMA_TFLOPS = 157.3  # MI355X published dense fp32 matrix peak
PEAK_VALU_TLANESLOTS = 78.6    # 256 CUs x 128 lanes x 2.4 GHz (= the 157.3 TFLOP/s fp32 vector figure / 2)
PEAK_HBM_GBS = 8000.0
PEAK_BF16_MFMA_TFLOPS = 2500.0  # MI355X published dense bf16 matrix peak
# rocprofv3 FETCH_SIZE / WRITE_SIZE of one LBG launch of k_assign_mfma_bf (KiB per dispatch), scaled by
# the plain copy kernel (FETCH x 2.000, WRITE x 1.000): profiles/pq_fit_encode_1Mx128.md
MEASURED_ASSIGN_TRAFFIC_BYTES = int((273044.0 * 2.000 + 12678.0 * 1.000) * 1024)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--rows", type=int, default=N_ROWS, help="rows of the workload (default 1M)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the plain copy kernel on the workload's rows (3 launches): the "
                         "known-size kernel the FETCH_SIZE / WRITE_SIZE counters are scaled by")
    ap.add_argument("--no-end-to-end", dest="end_to_end", action="store_false",
                    help="skip the one-off host-to-codes measurement")
    ap.add_argument("--cpu-sample", type=int, default=1_000_000,
                    help="rows of the CPU-baseline sample (0 = skip)")
    ap.add_argument("--configs", default="c3,c4,c5",
                    help="other configurations to run after the headline measurement (\"\" = none)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
            "(the path would shard by rows, one exchange of per-part sums per LBG iteration, "
            "but no multi-GPU code is built).")
        sys.exit(2)

    import vq_amd
    from vq_amd import synth as data

    n = args.rows
    sd = DIM // M
    t0 = time.time()
    x = data.gaussian_mixture(n, DIM, 1024, 0.05, seed=1)
    init, reseed = data.index_streams(n, M, K, ITERS, seed=1)
    log(f"[bench] generated {n} x {DIM} mixture rows in {time.time() - t0:.1f}s")

    ctx = vq_amd.Context(0)
    dx = ctx.to_device(x)
    dcb = ctx.empty((M, K, sd), np.float32)
    dcodes = ctx.empty((n, M), np.uint8)

    if args.copy_calibration:
        dy = ctx.empty((n, DIM), np.float32)
        for _ in range(3):
            ctx.copy_f32(dy, dx, n * DIM)
        ctx.sync()
        print(json.dumps({"copy_calibration_bytes_read": n * DIM * 4,
                          "copy_calibration_bytes_written": n * DIM * 4, "launches": 3}))
        return

    iters_seen = []

    def step():
        it, _ = ctx.lbg_fit(dx, n, DIM, M, sd, K, ITERS, init, reseed, dcb)
        ctx.assign(vq_amd.EUCLIDEAN, dx, n, DIM, M, sd, K, dcb, dcodes)
        iters_seen.append(it)

    for _ in range(args.warmup):
        step()
    ctx.sync()
    ctx.prof_enable(True)
    ctx.sync()
    del iters_seen[:]
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(args.steps):
        step()
    gpu_ms = ctx.timer_stop()
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    assign_ms, assign_n = ctx.prof_read(vq_amd._ffi.PROF_LBG_ASSIGN)
    update_ms, update_n = ctx.prof_read(vq_amd._ffi.PROF_LBG_UPDATE)
    enc_ms, enc_n = ctx.prof_read(vq_amd._ffi.PROF_ENCODE)
    kern_ms, kern_n = ctx.prof_read(vq_amd._ffi.PROF_ASSIGN_KERNEL)
    ctx.prof_enable(False)
    recheck_pairs = ctx.last_recheck_count()
    # what the timed steps left in their output buffers, and how many LBG iterations each column
    # block ran in them (a block that converges leaves its later passes at once: the line says so)
    timed_cb, timed_codes = dcb.download(), dcodes.download()
    timed_iters = np.concatenate(iters_seen) if iters_seen else np.zeros(1, np.int32)
    ms_per_step = wall_ms / args.steps
    value = n / (ms_per_step * 1e-3)

    # Dominant kernel: the assignment pass (k_assign_mfma_bf), timed alone by HIP events on the
    # library's stream (start and stop events of each launch's own dispatch).  What binds it is
    # instruction issue: the n x (m*k) scores come out of the matrix cores, every one of them has
    # to pass through the selection of the row's two smallest keys on the vector ALU, and on this
    # chip the two kinds of instruction take turns on a SIMD (one more matrix instruction per tile
    # lengthens the pass by that instruction's 32 clocks).
    #   algorithmic vector work per row = 2 lane-slots per score (one to tag or compare, one to
    #   select) = 2*m*k = 8,192; the 2*k*D lane-slots of the distance sums are on the matrix cores
    #   and priced there (mfma_* fields), so they are NOT counted against the vector peak.
    #   peak = 78.6 T lane-slots/s (256 CUs x 128 lanes x 2.4 GHz: one instruction per lane per
    #   clock; the published 157.3 TFLOP/s fp32 vector figure counts a fused multiply-add as two).
    # The kernel spends 17 instructions on 16 scores (v_min_i32 / v_min3_i32 over runs of four
    # centroids, one v_and_or_b32 tag per run, v_min3_i32 / v_med3_i32 for the two smallest keys),
    # each 4.2 clocks per wave64 on this chip, not 1; selection_floor_ms prices exactly those, and
    # issue_floor_ms adds the two matrix instructions per 32 x 32 tile at the nominal clock.
    flop_per_launch = 2.0 * K * DIM * n
    bytes_per_launch = (4.0 * DIM + 2.0 * M) * n
    slots_per_launch = 2.0 * M * K * n
    avg_kern_ms = kern_ms / max(kern_n, 1)
    sec = avg_kern_ms * 1e-3
    achieved_tflops = flop_per_launch / sec / 1e12
    achieved_slots = slots_per_launch / sec / 1e12
    roofline = {
        "bound": "valu",
        "kernel": "k_assign_mfma_bf (bf16-split matrix-core scores, top-2 selection over runs of four "
                  "centroids on the vector ALU, exact pick inside the best run, in-wave exact re-check; "
                  "the 10 LBG passes and the encode pass)",
        "achieved": round(achieved_slots, 3),
        "peak": PEAK_VALU_TLANESLOTS,
        "unit": "T lane-slots/s",
        "frac": round(achieved_slots / PEAK_VALU_TLANESLOTS, 4),
        "algorithmic_work": "2*m*k = 8192 vector lane-slots per row (selection only; the 2*k*D of the "
                            "distance sums run on the matrix cores)",
        # HBM bytes per launch: rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by the plain copy kernel,
        # taken from the committed profile of this workload, not measured in this run
        "traffic": MEASURED_ASSIGN_TRAFFIC_BYTES if n == N_ROWS else None,
        "traffic_source": "profiles/pq_fit_encode_1Mx128.md (static; rocprofv3 --pmc, not this run)",
        "algorithmic_bytes": int(bytes_per_launch),
        "avg_launch_ms": round(avg_kern_ms, 4),
        "launches": kern_n,
        # secondary views of the same launch time; none of them is the bound
        "mfma_fp32_equiv_TFLOPs": round(achieved_tflops, 1),
        "mfma_fp32_equiv_frac_of_157.3": round(achieved_tflops / PEAK_FP32_MFMA_TFLOPS, 4),
        "mfma_issued_bf16_TFLOPs": round(4.0 * achieved_tflops, 1),
        "mfma_issued_frac_of_bf16_peak": round(4.0 * achieved_tflops / PEAK_BF16_MFMA_TFLOPS, 4),
        "hbm_GBs_algorithmic": round(bytes_per_launch / sec / 1e9, 1),
        "hbm_frac": round(bytes_per_launch / sec / 1e9 / PEAK_HBM_GBS, 4),
        "assign_ms_incl_tables": round(assign_ms / max(assign_n, 1), 4),
    }
    # Measured issue rates of this box (vq_calibrate).  Per 16 scores the kernel issues 8 minima
    # (v_min_i32 / v_min3_i32, one class) for the four runs, 4 v_and_or_b32 (the runs' tags), and
    # 3 v_min3_i32 + 2 v_med3_i32 (top-2 update); one wave64 instruction handles 64 lanes.  The
    # selection floor is the time those instructions alone take with every SIMD full; the issue
    # floor adds the matrix instructions (2 per 32 x 32 tile, 32 clocks each, 1024 SIMDs at 2.4 GHz).
    rate = {name: ctx.calibrate(kind) for kind, name in
            ((1, "v_fma_f32"), (2, "v_min3_i32"), (3, "v_med3_i32"), (4, "v_and_or_b32"), (5, "v_add_u32"))}
    scores = float(n) * M * K
    floor_ms = scores / 64.0 * ((11.0 / 16.0) / rate["v_min3_i32"] + 0.25 / rate["v_and_or_b32"]
                                + 0.125 / rate["v_med3_i32"]) * 1e3
    mfma_ms = scores / 1024.0 * 2.0 * 32.0 / (1024.0 * 2.4e9) * 1e3
    roofline["selection_floor_ms"] = round(floor_ms, 4)
    roofline["frac_of_selection_floor"] = round(floor_ms / avg_kern_ms, 4)
    roofline["issue_floor_ms"] = round(floor_ms + mfma_ms, 4)
    roofline["frac_of_issue_floor"] = round((floor_ms + mfma_ms) / avg_kern_ms, 4)
    # The peak above is the packed / dual-rate one.  The selection's instruction class (v_min3_i32,
    # v_med3_i32, v_and_or_b32) issues one wave64 per 4 clocks and SIMD: 256 CUs x 64 lanes x 2.4 GHz.
    roofline["peak_of_selection_class"] = PEAK_VALU_TLANESLOTS / 2.0
    roofline["frac_of_selection_class_peak"] = round(achieved_slots / (PEAK_VALU_TLANESLOTS / 2.0), 4)
    # Do matrix and vector instructions of a SIMD run side by side?  (ms: matrix alone, vector alone,
    # together.)  From different waves they take turns (together = sum), which is why issue_floor_ms
    # adds them; behind a matrix instruction of the SAME wave independent vector instructions issue
    # in its shadow, all but about a quarter of its 32 clocks — the kernel places half a block's
    # selection behind each matrix instruction for that reason.
    ov = {}
    for mode, name in ((0, "different_waves_8_min3_per_mfma"), (1, "same_wave_7_min3_per_mfma"),
                       (2, "same_wave_3_min3_per_mfma")):
        (t_m, t_v, t_b), waves = ctx.calibrate_overlap(mode)
        ov[name] = {"mfma_alone_ms": round(t_m, 4), "valu_alone_ms": round(t_v, 4), "together_ms": round(t_b, 4),
                    "together_over_sum": round(t_b / (t_m + t_v), 3), "together_over_max": round(t_b / max(t_m, t_v), 3)}
        if mode == 0:
            ov[name]["waves_per_simd_number_mfma_then_valu"] = list(waves)
    calibration = {
        "hbm_copy_GBs_read_plus_write": round(ctx.calibrate(0), 1),
        "valu_wave64_Ginstr_per_s": {k_: round(v / 1e9, 1) for k_, v in rate.items()},
        "valu_fma_TFLOPs": round(rate["v_fma_f32"] * 128.0 / 1e12, 1),
        "mfma_valu_overlap": ov,
    }
    breakdown = {
        "lbg_assign_ms_per_step": round(assign_ms / args.steps, 3),
        "lbg_update_ms_per_step": round(update_ms / args.steps, 3),
        "encode_ms_per_step": round(enc_ms / args.steps, 3),
        "gpu_event_ms_per_step": round(gpu_ms / args.steps, 3),
        "encode_recheck_fraction": round(recheck_pairs / float(n * M), 6),
        # LBG iterations run per column block over the timed steps: 10 = no block stopped early, every
        # timed pass did its full work
        "lbg_iters_run_min": int(timed_iters.min()),
        "lbg_iters_run_max": int(timed_iters.max()),
    }

    # End to end, once: what a host that starts from rows in its own (pageable) memory pays.  vq_h2d
    # stages a large pageable upload through page-locked buffers with several host threads while
    # the copy engine uploads the chunk before; then fit, encode, and the codes come back into
    # page-locked memory.  For comparison the same rows from a page-locked buffer (no staging).
    # Not part of `value`.
    end_to_end = None
    if args.end_to_end:
        hx = ctx.host_empty((n, DIM), np.float32)
        hcodes = ctx.host_empty((n, M), np.uint8)
        np.copyto(hx, x)
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            dx.upload(x)           # pageable numpy array
            t1 = time.perf_counter()
            step()
            ctx.sync()
            t2 = time.perf_counter()
            vq_amd._ffi.lib().vq_d2h(ctx._h, hcodes.ctypes.data, dcodes.ptr, hcodes.nbytes)
            t3 = time.perf_counter()
            dx.upload(hx)          # page-locked
            t4 = time.perf_counter()
            cur = {"upload_ms": (t1 - t0) * 1e3, "fit_encode_ms": (t2 - t1) * 1e3,
                   "d2h_codes_ms": (t3 - t2) * 1e3, "total_ms": (t3 - t0) * 1e3,
                   "upload_from_page_locked_ms": (t4 - t3) * 1e3}
            if best is None or cur["total_ms"] < best["total_ms"]:
                best = cur
        end_to_end = {k_: round(v, 3) for k_, v in best.items()}
        end_to_end["vectors_per_s"] = round(n / (best["total_ms"] * 1e-3), 1)
        end_to_end["upload_GBs"] = round(x.nbytes / (best["upload_ms"] * 1e-3) / 1e9, 1)
        end_to_end["upload_from_page_locked_GBs"] = round(
            x.nbytes / (best["upload_from_page_locked_ms"] * 1e-3) / 1e9, 1)
        end_to_end["note"] = ("best of 3; upload = vq_h2d of the 512 MB pageable array (staged through "
                              "page-locked chunks by host threads, overlapped with the copy engine); "
                              "codes back to page-locked memory")
        ctx.host_free(hx)
        ctx.host_free(hcodes)

    # CPU baseline on the same rows with the same index streams, and parity of what the TIMED steps
    # wrote (codebooks and codes of the last timed step) against it
    cpu = None
    parity = None
    if args.cpu_sample > 0:
        from oracle import oracle as O
        ns = min(args.cpu_sample, n)
        full = ns == n
        xs = x if full else np.ascontiguousarray(x[:ns])
        init_s, reseed_s = (init, reseed) if full else data.index_streams(ns, M, K, ITERS, seed=2)
        threads = min(os.cpu_count() or 1, 16)
        t0 = time.perf_counter()
        ref = O.pq_fit_encode(O.EUCLIDEAN, xs, M, K, ITERS, init_s, reseed_s, threads=threads)
        cpu_s = time.perf_counter() - t0
        cpu = {
            "value": round(ns / cpu_s, 1), "unit": "vectors/s", "cores": ref["threads"],
            "kind": "port",
            "sample": f"first {ns} rows of the same workload, full fit (10 LBG iterations) + "
                      f"encode, C restatement of the reference with OpenMP over rows, {cpu_s:.1f} s",
            "reference_published": "3,751 vectors/s (266.6 s for 1M x 128 uniform rows, "
                                   "i7-1355U laptop, reference README.md:79-80)",
        }
        if full:
            g_cb, g_codes = timed_cb, timed_codes
            dcodes_s, dcb_s = dcodes, dcb
        else:
            dxs = ctx.to_device(xs)
            dcb_s = ctx.empty((M, K, sd), np.float32)
            dcodes_s = ctx.empty((ns, M), np.uint8)
            ctx.lbg_fit(dxs, ns, DIM, M, sd, K, ITERS, init_s, reseed_s, dcb_s)
            ctx.assign(vq_amd.EUCLIDEAN, dxs, ns, DIM, M, sd, K, dcb_s, dcodes_s)
            g_cb, g_codes = dcb_s.download(), dcodes_s.download()
        num = np.sqrt(((g_cb.astype(np.float64) - ref["codebooks"]) ** 2).sum())
        den = np.sqrt((ref["codebooks"].astype(np.float64) ** 2).sum())
        # reconstruction MSE of the f16 reconstructions (src/bin/utils.rs:50-67), both sides
        dre = ctx.empty((ns, DIM), np.uint16)
        if full:
            dcodes_s.upload(g_codes)
            dcb_s.upload(g_cb)
        ctx.decode_f16(dcodes_s, ns, M, sd, K, dcb_s, dre)
        mse_gpu = O.mse_f16(xs, dre.download())
        mse_ref = O.mse_f16(xs, O.pq_decode_f16(ref["codes"], ref["codebooks"]))
        dre.free()
        parity = {
            "sample_rows": ns,
            "compared": "the codebooks and codes the timed steps wrote (same rows, same index streams)" if full
                        else "a separate fit + encode of the sample",
            "mse_gpu": float(mse_gpu), "mse_ref": float(mse_ref),
            "mse_rel_diff": float(abs(mse_gpu - mse_ref) / mse_ref) if mse_ref else 0.0,
            "code_mismatch_rate": float(np.mean(g_codes != ref["codes"].astype(np.uint8))),
            "centroid_rel_l2": float(num / den),
            "centroids_bit_identical": bool(np.array_equal(g_cb.view(np.uint32),
                                                           ref["codebooks"].view(np.uint32))),
        }

    # the other configurations, after the headline measurement (bench_configs.py)
    others = None
    which = [c for c in args.configs.split(",") if c]
    if which and n == N_ROWS:
        import bench_configs
        others = bench_configs.other_configs(ctx, log, which, x_c2=x, dx_c2=dx)

    out = {
        "metric": "PQ fit+encode vectors/sec at 1M x 128, m=16, k=256 (10 LBG iterations)",
        "value": round(value, 1),
        "unit": "vectors/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"PQ fit (10 LBG iterations) + encode of {n} x {DIM} f32 rows, "
                               "mixture of 1,024 isotropic Gaussians (sigma 0.05, seed 1), "
                               "m=16, k=256, Euclidean encode to 16 u8 codes per row",
                   "rows": n, "dim": DIM, "m": M, "k": K, "lbg_iters": ITERS},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "calibration": calibration,
        "breakdown": breakdown,
        "end_to_end": end_to_end,
        "parity": parity,
        "other_configs": others,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
