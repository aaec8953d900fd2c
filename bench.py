#!/usr/bin/env python3
"""Benchmark of the fp32 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras] [--all-extras]

A step is one cake_sgemm of BASELINE config 2 (M = K = N = 8192, row-major fp32,
A and B uniform[-1,1) from seeds 1 and 2), operands resident in HBM, launched
through the C-ABI on torch's current stream.  W untimed steps, then exactly K
timed steps between two synchronisations.  Prints ONE JSON line:

  value          whole-job TFLOP/s over the K steps (wall clock)
  roofline       the GEMM macro-tile kernel: algorithmic FLOPs per launch
                 (2*M*N*K) over its average launch duration, taken from HIP
                 events recorded around every launch inside the timed region,
                 against the 157.3 TFLOP/s fp32 matrix peak
  cpu_baseline   the CPU restatement of the reference cake_sgemm (oracle/, kind
                 "port") on this host's physical cores, same inputs, full 8192^3
                 product once after a small warm-up
  extras         the other four BASELINE configs (not bench lines: reported for
                 information), each with a roofline object of its own and the CPU
                 restatement of the reference's call timed beside it; with
                 --all-extras a dozen more workloads (the short-K, streaming and
                 1 x 1 kernels, the linear layer) and, in every roofline object,
                 the row of profiles/ its traffic figure was read from

Bandwidth-bound workloads (the matrix-vector products, the streaming kernels)
are timed twice: `same_buffer`, every launch on the same operand, and
`rotating`, consecutive launches on four different 1 GiB operands, so that no
launch finds part of its operand in the 256 MB memory-side cache from the launch
before.  Their roofline is computed from the rotating run.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

METRIC = "fp32 GEMM TFLOP/s @8192^3 (% MFMA peak); GEMV GB/s (% HBM peak)"
MFMA_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
HBM_PEAK_GBPS = 8000.0     # MI355X HBM3E peak

# HBM-side bytes per launch of the kernels behind each workload, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this script (KiB per dispatch, each scaled by what the same counter reads for a
# plain 256 MiB copy: FETCH_SIZE x 1.9998, WRITE_SIZE x 1.0000; `--copy-calibration`).  Every entry
# names the row of profiles/all_kernels_hbm_traffic_pmc.md it was read from.
# The figure is the column "with its helper kernels" of that file's workload table, in bytes.
MEASURED_TRAFFIC = {
    "sgemm_8192": (4563256106, "row `sgemm_tile_kernel<Tile<256, 128, 32, 64, 64, 2, 1, 1>, 0, 0>` grid 1048576"),
    "sgemm_1024": (29500957, "row `sgemm_tile_kernel<Tile<64, 64, 64, 32, 32, 2, 2, 2>, 0, 0>` grid 131072"),
    "sgemm_tall_skinny": (306412911, "row `sgemm_tile_kernel<Tile<256, 128, 32, 64, 64, 2, 1, 1>, 0, 0>` grid 131072"),
    "sgemv_16384_rowmajor": (1074454809, "row `sgemv_rowmajor_wg_kernel<2, 8>` grid 4194304"),
    "sgemv_16384_colmajor": (1075873287, "row `sgemv_colmajor_kernel<true>` grid 196608"),
    "conv_c5_gather": (278924379, "row `sgemm_conv_patch_kernel<Tile<256, 128, 32, 64, 64, 2, 1, 1>, 3, 3>` grid 524288"),
    "conv_c5_two_step": (2212324492, "row `sgemm_tile_kernel<Tile<256, 128, 32, 64, 64, 2, 1, 1>, 0, 6>` grid 516096"),
    "shortk_256x64x100352": (129060273, "row `sgemm_shortk_kernel<Tile<64, 64, 64, 32, 32, 1, 1, 1>, 0, true>` grid 262144"),
    "conv_1x1_14x14": (43096930, "row `sgemm_shortk_staged_flat_kernel` grid 262144"),
    "resident_8192x256x8192": (400702558, "row `sgemm_resident_kernel` grid 131072"),
    "staged_3000x100x3000": (44956993, "row `sgemm_shortk_staged_kernel` grid 262144"),
    "fewrows_nn": (1087400124, "row `sgemm_fewrows_nn_kernel<1, 2>` grid 65536"),
    "fewrows_nn_64rows": (1128387615, "row `sgemm_fewrows_nn_kernel<4, 2>` grid 65536"),
    "narrow_tile_32cols": (289075043, "row `sgemm_tile_kernel<Tile<128, 32, 32, 32, 32, 2, 1, 1>, 0, 0>` grid 131072"),
    "fewrows_nt": (1083225759, "row `sgemm_fewrows_nt_kernel<false, 1, 64, 32, 1>` grid 65536"),
    "linear_fwd_16x16384x16384": (1083225759, "row `sgemm_fewrows_nt_kernel<false, 1, 64, 32, 1>` grid 65536"),
    "pack_a_8192": (542362035, "row `pack_tile_kernel<false, 24, 128, true>` grid 5603328"),
    "pack_b_8192": (538087108, "row `pack_tile_kernel<false, 16, 128, true>` grid 8388608"),
    "pack_c_8192": (538227331, "row `pack_tile_kernel<false, 16, 128, true>` grid 8404992"),
    "unpack_c_8192": (538110727, "row `pack_tile_kernel<true, 16, 128, true>` grid 8388608"),
    "im2col_c5": (1046053869, "row `im2col_rows_kernel<3>` grid 6422528"),
    "linear_fwd_8192x4096x4096": (1208263337, "row `sgemm_tile_kernel<Tile<256, 128, 32, 64, 64, 2, 1, 1>, 0, 2>` grid 524288"),
}


VERBOSE = False    # --all-extras: name the profile row behind every traffic figure


def roofline(bound, work, seconds, traffic_key=None, **more):
    """The roofline object of one workload: `work` algorithmic FLOPs (bound "mfma") or bytes (bound
    "hbm") per launch over the measured seconds per launch, against the published peak."""
    if bound == "mfma":
        achieved, peak, unit, key = work / seconds / 1e12, MFMA_PEAK_TFLOPS, "TFLOP/s", "algorithmic_flops_per_launch"
    else:
        achieved, peak, unit, key = work / seconds / 1e9, HBM_PEAK_GBPS, "GB/s", "algorithmic_bytes_per_launch"
    traffic, source = MEASURED_TRAFFIC.get(traffic_key, (None, None))
    r = {"bound": bound, "achieved": round(achieved, 3 if bound == "mfma" else 1), "peak": peak, "unit": unit,
         "frac": round(achieved / peak, 4), "traffic": traffic, key: work}
    if source and VERBOSE:
        r["traffic_source"] = "profiles/all_kernels_hbm_traffic_pmc.md, " + source
    r.update(more)
    return r


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the other BASELINE configs")
    ap.add_argument("--all-extras", action="store_true",
                    help="also time the workloads outside BASELINE.json (short K, streaming kernels, 1 x 1 convolution, "
                         "linear layer) and name the profile row of every traffic figure")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 256 MiB device copy kernel 3 times (reference point for "
                         "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE counters) and exit")
    ap.add_argument("--latency-floor", action="store_true",
                    help="only time 1024 x 1024 x K products for K = 32 .. 1024 and a one-workgroup kernel "
                         "(what config 1's time is made of: a fixed part and a part per k) and exit")
    args = ap.parse_args()
    global VERBOSE
    VERBOSE = args.all_extras
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (single-GPU hot path); --gpus must be 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    import cake_on_cpu_amd as cake
    from cake_on_cpu_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    lib = cake.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        src = torch.ones((64 << 20,), dtype=torch.float32, device=dev)   # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_each_way": src.numel() * 4, "launches": 3}))
        return 0
    info = cake.device_info()
    stream = torch.cuda.current_stream(dev).cuda_stream

    def dev_uniform(shape, seed):
        t = torch.empty(shape, dtype=torch.float32, device=dev)
        cake.fill_uniform(t, seed)
        return t

    def time_steps(launch, steps, warmup, settle_ms=0.0, each=False):
        """W warm-ups, then K launches between two synchronisations.  Returns the wall time of the
        K launches and the average and least launch duration by HIP events on the launch stream:
        one event pair around the K launches (their duration is the region's over K: a pair costs
        several microseconds of its own, too much to put around a launch of twenty), or with
        `each` a pair per launch, which also gives the least.
        settle_ms > 0 keeps launching warm-ups until that much GPU time has passed, so that a
        sub-millisecond kernel is timed at settled clocks like the long ones are."""
        for _ in range(warmup):
            launch()
        torch.cuda.synchronize()
        if settle_ms > 0:
            t_end = time.perf_counter() + settle_ms * 1e-3
            while time.perf_counter() < t_end:
                for _ in range(20):
                    launch()
                torch.cuda.synchronize()
        pairs = steps if each else 1
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(pairs)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if each:
            for a, b in evs:
                a.record()
                launch()
                b.record()
        else:
            evs[0][0].record()
            for _ in range(steps):
                launch()
            evs[0][1].record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        kernel = [a.elapsed_time(b) * 1e-3 * pairs / steps for a, b in evs]
        return wall, float(np.mean(kernel)), float(np.min(kernel))

    ROTATE = 4

    def time_rotating(launch_on, steps, warmup, settle_ms):
        """`launch_on(i)` launches on operand i of ROTATE.  Returns the average launch duration with
        every launch on operand 0 and with consecutive launches on different operands."""
        same = time_steps(lambda: launch_on(0), steps, warmup, settle_ms)[1]
        turn = [0]

        def next_one():
            launch_on(turn[0] % ROTATE)
            turn[0] += 1
        return same, time_steps(next_one, steps, warmup, settle_ms)[1]

    def rotating_operand(elems, seed):
        """ROTATE operands of `elems` floats in one allocation; operand 0 is the stream `seed`."""
        whole = torch.empty((ROTATE * elems,), dtype=torch.float32, device=dev)
        for r in range(ROTATE):
            cake.fill_uniform(whole[r * elems:(r + 1) * elems], seed if r == 0 else 1000 * r + seed)
        return whole

    if args.latency_floor:
        m = 1024
        a1, b1 = dev_uniform((m, m), 11), dev_uniform((m, m), 12)
        c1 = torch.zeros((m, m), dtype=torch.float32, device=dev)
        one = torch.zeros((64,), dtype=torch.float32, device=dev)
        rows = []

        def best_of(launch):
            return min(time_steps(launch, 50, 20, settle_ms=50.0)[1] for _ in range(3))

        rows.append({"kernel": "fill_uniform_kernel, one workgroup",
                     "us": round(best_of(lambda: _lib.check(lib.cake_hip_fill_uniform(one.data_ptr(), 64, 1, stream), "fill")) * 1e6, 2)})
        ks = (32, 64, 128, 256, 512, 768, 1024)
        for k in ks:
            # dense 1024 x k and k x 1024 operands at the front of the buffers
            def launch(k=k):
                _lib.check(lib.cake_hip_sgemm(a1.data_ptr(), b1.data_ptr(), c1.data_ptr(), m, m, k, cake.NA, 0, None,
                                              stream, None), "cake_hip_sgemm")
            pl = cake.plan(m, m, k)
            rows.append({"K": k, "us": round(best_of(launch) * 1e6, 2), "kernel": cake.KERNEL_NAMES[pl.kernel],
                         "tile": f"{pl.tile_m}x{pl.tile_n}x{pl.tile_k}", "workgroups": pl.grid})
        # least squares over the K that run the same kernel as K = 1024
        same = [r for r in rows if r.get("tile") == rows[-1]["tile"] and r.get("kernel") == rows[-1]["kernel"]]
        xs, ys = np.array([r["K"] for r in same], float), np.array([r["us"] for r in same], float)
        slope, fixed = np.polyfit(xs, ys, 1) if len(same) >= 2 else (float("nan"), float("nan"))
        peak_ns_per_k = 2.0 * m * m / (MFMA_PEAK_TFLOPS * 1e12) * 1e9
        print(json.dumps({"latency_floor_1024x1024xK": rows, "fit_over_K": [int(x) for x in xs],
                          "fixed_us": round(float(fixed), 2), "ns_per_k": round(float(slope) * 1e3, 2),
                          "ns_per_k_at_mfma_peak": round(peak_ns_per_k, 2)}))
        return 0

    # ---------------------------------------------------------------- config 2
    n = 8192
    A, B = dev_uniform((n, n), 1), dev_uniform((n, n), 2)
    Cm = torch.zeros((n, n), dtype=torch.float32, device=dev)
    pa, pb, pc = A.data_ptr(), B.data_ptr(), Cm.data_ptr()

    def sgemm_step():
        _lib.check(lib.cake_hip_sgemm(pa, pb, pc, n, n, n, cake.NA, 0, None, stream, None), "cake_hip_sgemm")

    wall, k_avg, k_min = time_steps(sgemm_step, args.steps, args.warmup, each=True)
    flops = 2.0 * n * n * n
    value = flops * args.steps / wall / 1e12
    achieved = flops / k_avg / 1e12
    plan = cake.plan(n, n, n)

    # cheap guard against a fast wrong answer: a few rows against fp64
    import oracle
    rows = torch.tensor([0, 1, 4097, n - 1], device=dev)
    C64, S = oracle.gemm_f64(np.ascontiguousarray(A[rows].cpu().numpy()), B.cpu().numpy())
    check_err = oracle.max_rel_err(np.ascontiguousarray(Cm[rows].cpu().numpy()), C64, S)

    out = {
        "metric": METRIC,
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "cake_sgemm C=A*B, M=K=N=8192, row-major fp32, uniform[-1,1) seeds 1/2 (BASELINE configs[1])",
            "tile": f"{plan.tile_m}x{plan.tile_n}x{plan.tile_k}",
            "wave_tile": f"{plan.wave_m}x{plan.wave_n}",
            "schedule": cake.SCHED_NAMES[plan.sched],
            "split_k": plan.split_k,
            "workgroups": plan.grid,
            "device": info.arch.decode(),
            "cus": info.cus,
        },
        "roofline": roofline("mfma", flops, k_avg, "sgemm_8192",
                             kernel=f"sgemm_tile_kernel<Tile<{plan.tile_m},{plan.tile_n},{plan.tile_k},{plan.wave_m},{plan.wave_n},...>,0,0>",
                             avg_launch_ms=round(k_avg * 1e3, 4), min_launch_ms=round(k_min * 1e3, 4)),
        "check": {"max_rel_err_sampled_rows": check_err, "tolerance": 1e-4},
    }

    # ------------------------------------------------------------ other configs
    p_cores = oracle.physical_cores()
    cpu_cx = oracle.query_cntx()

    def cpu_leg(run, work, unit, sample, repeats=3):
        """The CPU restatement of the reference's call on this host's physical cores: one warm-up,
        then the median of `repeats` runs; `run` returns the seconds the call itself reports."""
        if args.no_cpu:
            return None
        run()
        secs = float(np.median([run() for _ in range(repeats)]))
        scale = 1e12 if unit == "TFLOP/s" else 1e9
        return {"value": round(work / secs / scale, 4), "unit": unit, "cores": p_cores, "kind": "port",
                "seconds": round(secs, 5), "sample": sample}

    def more_extras():
        extras = other_extras
        # a 1 x 1 layer: planes read in place (no staged copy, no tap table), NCHW output
        Pb, Pc, Ph, Po = 32, 256, 14, 1024
        pin, pw = dev_uniform((Pb, Pc, Ph, Ph), 6), dev_uniform((Po, Pc), 7)
        po = torch.empty((Pb, Po, Ph, Ph), dtype=torch.float32, device=dev)
        pws_bytes = lib.cake_hip_conv2d_workspace(Pb, Pc, Ph, Ph, Po, 1, 1, 1, 0)
        pws = torch.empty((max(1, (pws_bytes + 3) // 4),), dtype=torch.float32, device=dev)
        pfl = 2.0 * Po * Pc * (Pb * Ph * Ph)
        pby = 4.0 * (Pb * Pc * Ph * Ph + Po * Pc + Pb * Po * Ph * Ph)
        _, avg, _ = time_steps(lambda: _lib.check(
            lib.cake_hip_conv2d(pin.data_ptr(), pw.data_ptr(), po.data_ptr(), Pb, Pc, Ph, Ph, Po, 1, 1, 1, 0, 1,
                                pws.data_ptr(), stream, None), "conv2d"), 50, 5, 40.0)
        extras.append({"workload": "conv 1x1, batch 32, 256->1024 ch, 14x14, NCHW output",
                       "us": round(avg * 1e6, 2), "tflops": round(pfl / avg / 1e12, 2),
                       "roofline": roofline("mfma", pfl, avg, "conv_1x1_14x14", algorithmic_bytes_per_launch=pby)})
        del pin, po, pws

        # the linear layer (src/linear.cpp): batch 8192, 4096 -> 4096 features, with bias
        Lm, Lk, Ln = 8192, 4096, 4096
        lx, lw, lb = dev_uniform((Lm, Lk), 11), dev_uniform((Ln, Lk), 12), dev_uniform((Ln,), 13)
        lg = dev_uniform((Lm, Ln), 14)
        ly = torch.empty((Lm, Ln), dtype=torch.float32, device=dev)
        lgx, lgw = torch.empty_like(lx), torch.empty_like(lw)
        lgb = torch.empty_like(lb)
        lfl = 2.0 * Lm * Ln * Lk
        _, avg, _ = time_steps(lambda: _lib.check(
            lib.cake_hip_linear_forward(lx.data_ptr(), lw.data_ptr(), lb.data_ptr(), ly.data_ptr(), Lm, Ln, Lk,
                                        stream, None), "linear_forward"), 20, 3, 40.0)
        extras.append({"workload": "linear forward, batch 8192, 4096->4096, bias (weights read as they lie, no transposed copy)",
                       "ms": round(avg * 1e3, 4), "tflops": round(lfl / avg / 1e12, 2),
                       "roofline": roofline("mfma", lfl, avg, "linear_fwd_8192x4096x4096")})
        _, avg, _ = time_steps(lambda: _lib.check(
            lib.cake_hip_linear_backward(lg.data_ptr(), lx.data_ptr(), lw.data_ptr(), lgx.data_ptr(), lgw.data_ptr(),
                                         lgb.data_ptr(), Lm, Ln, Lk, stream, None), "linear_backward"), 20, 3, 40.0)
        extras.append({"workload": "linear backward, same layer (two products, one transpose, bias sums)",
                       "ms": round(avg * 1e3, 4), "tflops": round(2 * lfl / avg / 1e12, 2),
                       "roofline": roofline("mfma", 2 * lfl, avg)})
        del lx, lg, ly, lgx
        # a small batch: the weights are streamed once as they lie, no transposed copy
        Sm, Sk, Sn = 16, 16384, 16384
        sx, sw, sb = dev_uniform((Sm, Sk), 15), rotating_operand(Sn * Sk, 16), dev_uniform((Sn,), 17)
        sy = torch.empty((Sm, Sn), dtype=torch.float32, device=dev)
        sby = 4.0 * (Sm * Sk + Sn * Sk + Sn + Sm * Sn)
        same, avg = time_rotating(lambda i: _lib.check(
            lib.cake_hip_linear_forward(sx.data_ptr(), sw.data_ptr() + 4 * Sn * Sk * i, sb.data_ptr(), sy.data_ptr(), Sm, Sn, Sk,
                                        stream, None), "linear_forward"), 50, 5, 40.0)
        extras.append({"workload": "linear forward, batch 16, 16384->16384, bias",
                       "us": round(avg * 1e6, 2), "us_same_buffer": round(same * 1e6, 2),
                       "tflops": round(2.0 * Sm * Sn * Sk / avg / 1e12, 2), "kernel": "sgemm_fewrows_nt_kernel",
                       "roofline": roofline("hbm", sby, avg, "linear_fwd_16x16384x16384",
                                            timed_on=f"{ROTATE} rotating weight matrices",
                                            frac_same_buffer=round(sby / same / 1e9 / HBM_PEAK_GBPS, 4))})

        # The copies of the path: pack_A / pack_B / pack_C / unpack_C (8192^2 operands in the reference's
        # panel layout for m_r = 6, n_r = 16; each call builds its two index tables first) and im2col
        # of config 5's input.  Algorithmic bytes: every element read once and written once.
        import ctypes as C
        Pn, Pp = 8192, 8
        pcx = cake.CpuCntx(1.0, 6, 16, 48 << 10, 2 << 20, 105 << 20, 8)
        pdims = cake.init_block_dims(Pn, Pn, Pn, Pp, pcx, cake.KMN)
        plain = dev_uniform((Pn, Pn), 21)
        sizes = {"a": cake.cake_sgemm_packed_A_size(Pn, Pn, Pp, pdims, pcx, cake.KMN), "b": cake.cake_sgemm_packed_B_size(Pn, Pn, Pp, pdims, pcx),
                 "c": cake.cake_sgemm_packed_C_size(Pn, Pn, Pp, pdims, pcx, cake.KMN)}
        packed = torch.empty((max(sizes.values()) // 4,), dtype=torch.float32, device=dev)
        back = torch.empty((Pn, Pn), dtype=torch.float32, device=dev)
        bd, bc = C.byref(pdims), C.byref(pcx)
        calls = (("pack_A", "a", lambda: lib.cake_hip_pack_a(plain.data_ptr(), packed.data_ptr(), Pn, Pn, Pp, bd, bc, cake.KMN, stream, None)),
                 ("pack_B", "b", lambda: lib.cake_hip_pack_b(plain.data_ptr(), packed.data_ptr(), Pn, Pn, Pp, bd, bc, cake.KMN, stream, None)),
                 ("pack_C", "c", lambda: lib.cake_hip_pack_c(plain.data_ptr(), packed.data_ptr(), Pn, Pn, Pp, bd, bc, cake.KMN, stream, None)),
                 ("unpack_C", "c", lambda: lib.cake_hip_unpack_c(back.data_ptr(), packed.data_ptr(), Pn, Pn, Pp, bd, bc, cake.KMN, stream, None)))
        for name, which, call in calls:
            _, avg, _ = time_steps(lambda: _lib.check(call(), name), 20, 3, 20.0)
            pby = 4.0 * Pn * Pn + sizes[which]
            extras.append({"workload": f"{name} of an 8192 x 8192 operand (index tables included)", "us": round(avg * 1e6, 2),
                           "roofline": roofline("hbm", pby, avg, {"pack_A": "pack_a_8192", "pack_B": "pack_b_8192", "pack_C": "pack_c_8192",
                                                                  "unpack_C": "unpack_c_8192"}[name])})
        del plain, packed, back
        Bn, Cc, H = 32, 256, 56
        iin = dev_uniform((Bn, Cc, H, H), 22)
        icols = torch.empty((Cc * 9, Bn * H * H), dtype=torch.float32, device=dev)
        other_a, other_b = torch.empty((8192, 8192), dtype=torch.float32, device=dev), torch.empty((8192, 8192), dtype=torch.float32, device=dev)
        iby = 4.0 * (iin.numel() + icols.numel())
        im = lambda: _lib.check(lib.cake_hip_im2col(iin.data_ptr(), icols.data_ptr(), Bn, Cc, H, H, 3, 3, 1, 1, stream, None), "im2col")
        _, alone, _ = time_steps(im, 20, 3, 20.0)
        # ... and with a 256 MB copy between the launches, so that neither the input nor the end of the
        # previous launch's columns wait in the memory-side cache: what the kernel costs inside a convolution
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(20)]
        for a, b in evs:
            other_b.copy_(other_a)
            a.record()
            im()
            b.record()
        torch.cuda.synchronize()
        between = float(np.mean([a.elapsed_time(b) for a, b in evs])) * 1e-3
        extras.append({"workload": "im2col of config 5's input (32 x 256 x 56 x 56, 3 x 3, pad 1): 925 MB of columns",
                       "us": round(between * 1e6, 2), "us_in_a_loop_of_its_own": round(alone * 1e6, 2),
                       "roofline": roofline("hbm", iby, between, "im2col_c5", timed_on="launches with a 256 MB copy between them")})
        del iin, icols, other_a, other_b

    if not args.no_extras:

        def gemm_extra(name, M, N, K, traffic_key=None, streaming_kernel=None, cpu=False, bound="hbm", rotate=None):
            """rotate: "A" or "B" -- the operand that is streamed once, timed on ROTATE different copies."""
            a = rotating_operand(M * K, 1) if rotate == "A" else dev_uniform((M, K), 1)
            b = rotating_operand(K * N, 2) if rotate == "B" else dev_uniform((K, N), 2)
            c = torch.zeros((M, N), dtype=torch.float32, device=dev)
            pc = c.data_ptr()

            def launch_on(i):
                pa = a.data_ptr() + (4 * M * K * i if rotate == "A" else 0)
                pb = b.data_ptr() + (4 * K * N * i if rotate == "B" else 0)
                _lib.check(lib.cake_hip_sgemm(pa, pb, pc, M, N, K, cake.NA, 0, None, stream, None), name)
            same = None
            if rotate:
                same, avg = time_rotating(launch_on, 50, 5, 40.0)
            else:
                _, avg, _ = time_steps(lambda: launch_on(0), 50, 5, 40.0)
            pl = cake.plan(M, N, K)
            fl = 2.0 * M * N * K
            by = 4.0 * (M * K + K * N + M * N)
            e = {"workload": name, "us": round(avg * 1e6, 2), "tflops": round(fl / avg / 1e12, 2),
                 "compulsory_GBps": round(by / avg / 1e9, 1), "kernel_family": cake.KERNEL_NAMES[pl.kernel]}
            more = {}
            if same is not None:
                e["us_same_buffer"] = round(same * 1e6, 2)
                more = {"timed_on": f"{ROTATE} rotating operands", "frac_same_buffer": round(by / same / 1e9 / HBM_PEAK_GBPS, 4)}
            if streaming_kernel:   # few rows or columns: bound by reading the large operand once
                e["kernel"] = streaming_kernel   # (or, from 49 rows on, by the matrix pipe)
                e["roofline"] = (roofline("hbm", by, avg, traffic_key, **more) if bound == "hbm" else
                                 roofline("mfma", fl, avg, traffic_key, algorithmic_bytes_per_launch=by))
            else:
                e.update({"tile": f"{pl.tile_m}x{pl.tile_n}x{pl.tile_k}", "split_k": pl.split_k,
                          "schedule": cake.SCHED_NAMES[pl.sched]})
                e["roofline"] = roofline("mfma", fl, avg, traffic_key, algorithmic_bytes_per_launch=by)
            if cpu:
                Ah, Bh = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
                dims = {}

                def run():
                    _, secs, x = oracle.cake_sgemm(Ah, Bh, p_cores, cpu_cx, return_time=True)
                    dims["x"] = x
                    return secs
                e["cpu_baseline"] = cpu_leg(run, fl, "TFLOP/s", "")
                if e["cpu_baseline"]:
                    x = dims["x"]
                    e["cpu_baseline"]["sample"] = (f"full product, reference default schedule "
                                                   f"{oracle.SCHED_NAMES[x.sch]}, m_c={x.m_c}, n_c={x.n_c}; median of 3")
            del a, b, c
            return e

        baseline_extras, other_extras = [], []
        baseline_extras.append(gemm_extra("configs[0] sgemm 1024^3", 1024, 1024, 1024, "sgemm_1024", cpu=True))
        baseline_extras.append(gemm_extra("configs[2] sgemm tall-skinny M=65536 K=1024 N=128", 65536, 128, 1024,
                                          "sgemm_tall_skinny", cpu=True))
        if args.all_extras:
            other_extras.append(gemm_extra("sgemm short K, many tiles: M=256 K=64 N=100352", 256, 100352, 64, "shortk_256x64x100352"))
            other_extras.append(gemm_extra("sgemm mid K on 256 x 128 tiles walked by resident workgroups: M=8192 K=256 N=8192",
                                           8192, 8192, 256, "resident_8192x256x8192", bound="mfma"))
            other_extras.append(gemm_extra("sgemm K = 100, 64 x 64 tiles walked stage by stage: M=3000 K=100 N=3000", 3000, 3000, 100,
                                           "staged_3000x100x3000", bound="mfma"))
            other_extras.append(gemm_extra("sgemm 16 rows: M=16 K=16384 N=16384", 16, 16384, 16384, "fewrows_nn",
                                           "sgemm_fewrows_nn_kernel + splitk_reduce_kernel", rotate="B"))
            other_extras.append(gemm_extra("sgemm 16 columns: M=16384 K=16384 N=16", 16384, 16, 16384, "fewrows_nt",
                                           "transpose_kernel (B into 16 rows) + sgemm_fewrows_nt_kernel", rotate="A"))
            other_extras.append(gemm_extra("sgemm 64 rows: M=64 K=16384 N=16384", 64, 16384, 16384, "fewrows_nn_64rows",
                                           "sgemm_fewrows_nn_kernel<4, 2> + splitk_reduce_kernel", bound="mfma"))
            other_extras.append(gemm_extra("sgemm 32 columns (a low-rank projection): M=16384 K=4096 N=32", 16384, 32, 4096,
                                           "narrow_tile_32cols",
                                           "sgemm_tile_kernel<Tile<128, 32, 32, 32, 32, 2, 1, 1>, 0, 0> in 4 K slices + splitk_reduce_kernel"))

        m = 16384
        Ag, xg = rotating_operand(m * m, 1), dev_uniform((m,), 3)
        yg = torch.zeros((m,), dtype=torch.float32, device=dev)
        gbytes = 4.0 * (m * m + m + m)
        gemv_cpu = None
        if not args.no_cpu:
            # cake_sgemv as examples/cake_gemv.cpp runs it: column-major A, m_r = 8, y accumulates
            Agh, xgh = oracle.uniform((m, m), 1), oracle.uniform(m, 3)
            gcx = oracle.query_cntx()
            gcx.mr = 8
            gemv_cpu = cpu_leg(lambda: oracle.cake_sgemv(Agh, xgh, p_cores, gcx, M=m, K=m, return_time=True)[1], gbytes, "GB/s",
                               "full 16384^2 cake_sgemv, column-major A (the reference's layout); median of 3")
            del Agh
        for col, label, key in ((0, "configs[3] sgemv 16384^2, row-major A", "sgemv_16384_rowmajor"),
                                (1, "configs[3] sgemv 16384^2, column-major A (cake_sgemv's layout)", "sgemv_16384_colmajor")):
            same, avg = time_rotating(lambda i: _lib.check(
                lib.cake_hip_sgemv(Ag.data_ptr() + 4 * m * m * i, xg.data_ptr(), yg.data_ptr(), m, m, col, 0, stream, None),
                "sgemv"), 60, 12, 40.0)
            baseline_extras.append({"workload": label, "us": round(avg * 1e6, 2), "us_same_buffer": round(same * 1e6, 2),
                                    "GBps": round(gbytes / avg / 1e9, 1),
                                    "roofline": roofline("hbm", gbytes, avg, key, timed_on=f"{ROTATE} rotating 1 GiB matrices",
                                                         frac_same_buffer=round(gbytes / same / 1e9 / HBM_PEAK_GBPS, 4)),
                                    "cpu_baseline": gemv_cpu if col else None})
        del Ag

        Bn, Cc, H = 32, 256, 56
        inp, wt = dev_uniform((Bn, Cc, H, H), 5), dev_uniform((Cc, Cc, 3, 3), 4)
        oc = torch.empty((Cc, Bn * H * H), dtype=torch.float32, device=dev)
        ws_bytes = lib.cake_hip_conv2d_workspace(Bn, Cc, H, H, Cc, 3, 3, 1, 1)
        ws = torch.empty(((ws_bytes + 3) // 4,), dtype=torch.float32, device=dev)
        cfl = 2.0 * Cc * (Cc * 9) * (Bn * H * H)
        cby = 4.0 * (Bn * Cc * H * H + Cc * Cc * 9 + Bn * Cc * H * H)      # input + weights + output
        conv_cpu = None
        if not args.no_cpu:
            # the reference's sequence for one image (examples/cake_conv.cpp:1007-1066): im_2_col of the
            # zero-padded CHW image, then cake_sgemm (which packs both operands); 2 of the 32 images
            imgs = oracle.uniform((2, Cc, H, H), 5)
            wh = oracle.uniform((Cc, Cc * 9), 4)
            padded = np.zeros((2, Cc, H + 2, H + 2), np.float32)
            padded[:, :, 1:-1, 1:-1] = imgs

            def conv_cpu_run():
                total = 0.0
                for b in range(2):
                    t0 = time.perf_counter()
                    cols = oracle.im_2_col(padded[b], 3, 3, H, H)
                    total += time.perf_counter() - t0
                    total += oracle.cake_sgemm(wh, cols, p_cores, cpu_cx, sch=oracle.KMN, return_time=True)[1]
                return total
            conv_cpu = cpu_leg(conv_cpu_run, cfl * 2 / Bn, "TFLOP/s",
                               "2 of the 32 images: im_2_col + cake_sgemm(KMN) per image, as examples/cake_conv.cpp; median of 3")
        # output written as NCHW by the GEMM's epilogue on both paths
        for fn, label, key in ((lib.cake_hip_conv2d, "input read where it lies (no column matrix)", "conv_c5_gather"),
                               (lib.cake_hip_conv2d_im2col, "im2col kernel, then GEMM (the reference's two steps)",
                                "conv_c5_two_step")):
            _, avg, _ = time_steps(lambda: _lib.check(
                fn(inp.data_ptr(), wt.data_ptr(), oc.data_ptr(), Bn, Cc, H, H, Cc, 3, 3, 1, 1, 1,
                   ws.data_ptr(), stream, None), "conv2d"), 20, 3, 40.0)
            baseline_extras.append({"workload": f"configs[4] conv 3x3 s1 p1, batch 32, 256->256, 56x56, NCHW out: {label}",
                                    "ms": round(avg * 1e3, 4), "tflops": round(cfl / avg / 1e12, 2),
                                    "roofline": roofline("mfma", cfl, avg, key, algorithmic_bytes_per_launch=cby),
                                    "cpu_baseline": conv_cpu if fn == lib.cake_hip_conv2d_im2col else None})
        del inp, oc, ws
        if args.all_extras:
            more_extras()
        # the BASELINE configs last: the end of a long line is what a log keeps
        out["extras"] = other_extras + baseline_extras

    # -------------------------------------------------------------- CPU baseline
    if not args.no_cpu:
        p, cx = p_cores, cpu_cx
        Ah, Bh = oracle.uniform((n, n), 1), oracle.uniform((n, n), 2)
        oracle.cake_sgemm(Ah[:2048, :2048].copy(), Bh[:2048, :2048].copy(), p, cx)   # warm-up
        _, secs, dims = oracle.cake_sgemm(Ah, Bh, p, cx, return_time=True)
        out["cpu_baseline"] = {
            "value": round(flops / secs / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": p,
            "kind": "port",
            "sample": f"one full 8192^3 cake_sgemm (plan+pack+compute+unpack, schedule "
                      f"{oracle.SCHED_NAMES[dims.sch]}, m_c=k_c={dims.m_c}, n_c={dims.n_c}) after a 2048^3 warm-up; "
                      f"{secs:.2f} s",
        }
    else:
        out["cpu_baseline"] = None

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
