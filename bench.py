#!/usr/bin/env python3
"""Headline benchmark: int4 x fp16 matvec at K(N)=5120, S=20480, M=1, g=128 on one
MI355X, through the C ABI of libint4mm_hip.so.

A step is one matvec over one set of packed weights.  Seven distinct weight sets
(390 MB, more than the 256 MB last-level cache) are used in rotation so that
every step streams its weights from HBM.  The timed region is K steps captured
in one HIP graph (no host work between kernels), replayed until about 2000 launches
have run, bracketed by synchronisation (ms_per_step = wall / (replays x K));
HIP events recorded on the launch stream around the same region give the average
kernel duration used for the roofline figure.  The int4 matmul at M=2048 is
measured the same way and reported beside it, and the torch-CPU
dequantise-then-matmul baseline is timed on the host on a bounded sample.

Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA

# HBM bytes per launch of i4::matvec_kernel<4,false,2,false>, from two counter runs of this script
# (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, with --calibrate-copy; commands and per-dispatch
# readings in profiles/matvec_int4_K5120_S20480.md): FETCH_SIZE 27 640.6 KiB x 2.000 (a 256 MiB
# copy reads 131 089.7) + WRITE_SIZE 1 000.0 KiB x 1.000 (the same copy writes 262 144.0)
MATVEC_TRAFFIC_BYTES = 57_631_949
# the same for i4::matmul_kernel_pipe<4,false,4,4,true,true> at M=2048, from the same two runs
# (profiles/matmul_int4_M2048_K5120_S20480.md): 192 782.5 KiB x 2.000 + 149 164.9 KiB x 1.000
MATMUL_TRAFFIC_BYTES = 547_563_418


def matvec_bytes(K, S, g, bits=4):
    return K * bits // 32 * S * 4 + 2 * (K // g) * S * 2 + 2 * K + 2 * S


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=700)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-gemm", action="store_true", help="skip the M=2048 matmul leg")
    ap.add_argument("--no-helpers", action="store_true", help="skip the pack / unpack / dequantise leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 256 MiB device-to-device copy five times (a kernel of known HBM "
                         "traffic, used to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the matvec/matmul shard "
              "by output columns without any exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from int4matmul_kernels_amd import capi
    from oracle import oracle as O

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    K, S, g, NSETS = 5120, 20480, 128, 7
    steps, warmup = max(1, args.steps), max(0, args.warmup)

    # ---- seeded synthetic workload (the headline matvec shape); set 0 is the oracle's problem
    p = O.make_problem(K=K, S=S, M=1, bits=4, group_size=g, seed=0)
    gen = torch.Generator(device="cpu").manual_seed(0)
    sets = []
    for i in range(NSETS):
        if i == 0:
            m, sc, ze = (torch.from_numpy(p["matrix"]), torch.from_numpy(p["scales"]), torch.from_numpy(p["zeros"]))
        else:
            m = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, S), dtype=torch.int32, generator=gen)
            sc = torch.empty((K // g, S)).uniform_(0.001, 0.02, generator=gen).half()
            ze = torch.empty((K // g, S)).uniform_(0.0, 15.0, generator=gen).half()
        sets.append((m.to(dev), sc.to(dev), ze.to(dev)))
    x = torch.from_numpy(p["states"]).to(dev)
    xneg = -x                                   # alternate sign so that outs does not grow
    outs = [torch.zeros((1, 1, S), dtype=torch.float16, device=dev) for _ in range(NSETS)]
    ws = capi.new_workspace(S)

    def step(i):
        m, sc, ze = sets[i % NSETS]
        xi = x if (i // NSETS) % 2 == 0 else xneg
        capi.matvec(4, outs[i % NSETS], m, xi, sc, ze, g, None, ws)

    # ---- correctness of the measured path against the oracle (set 0, fresh outs)
    chk = torch.zeros((1, 1, S), dtype=torch.float16, device=dev)
    capi.matvec(4, chk, sets[0][0], x, sets[0][1], sets[0][2], g, None, ws)
    torch.cuda.synchronize()
    w32 = O.dequantize_matrix_fp32(4, p["matrix"], p["scales"], p["zeros"], g)
    want = O.matmul_fp32(p["states"][0], w32)
    err = O.max_rel_error(want, chk.cpu().numpy()[0])
    assert err < 1e-2, f"matvec disagrees with the oracle: max relative error {err}"

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(warmup):
            step(i)
        stream.synchronize()
        # K steps in one graph: back-to-back kernels, no host work in the timed region
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(steps):
                step(i)
        graph.replay()                            # untimed: first replay uploads the graph
        stream.synchronize()
        # the timed region: the K-step graph replayed back to back often enough (about 2000 launches in
        # all) that the per-step figure is the steady state whatever K is -- a single replay of a short
        # graph would carry the graph's own launch latency
        replays = max(1, -(-2000 // steps))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(replays):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    launches = replays * steps
    wall_s = (t1 - t0) / replays                  # wall clock of one K-step pass
    ev_us = e0.elapsed_time(e1) * 1e3 / launches  # average launch duration, HIP events on the launch stream
    nbytes = matvec_bytes(K, S, g)
    value = nbytes * steps / wall_s / 1e9
    achieved = nbytes / (ev_us * 1e-6) / 1e9

    result = {
        "metric": "int4 GEMV GB/s & us (N=5120,S=20480,M=1); int4 GEMM TFLOP/s at M=2048",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": wall_s * 1e3 / steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "int4 dense matvec K(N)=5120 S=20480 M=1 B=1 group=128, "
                               f"{NSETS} weight sets in rotation (cold HBM)",
                   "bytes_per_step": nbytes, "us_per_step": round(wall_s * 1e6 / steps, 3),
                   "graph_replays_timed": replays,
                   "max_rel_err_vs_fp32_oracle": float(f"{err:.3e}")},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MATVEC_TRAFFIC_BYTES,
                     "kernel": "i4::matvec_kernel<4,false,...>", "avg_launch_us": round(ev_us, 3)},
    }

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        result["calibration"] = {"kernel": "torch device copy", "bytes_read": 256 << 20, "bytes_written": 256 << 20}

    # ---- the matmul half of the metric: M=2048, same weights (the headline matmul shape)
    if not args.no_gemm:
        M = 2048
        xs = torch.randn((1, M, K), generator=torch.Generator(device="cpu").manual_seed(1)).half().to(dev)
        om = torch.zeros((1, M, S), dtype=torch.float16, device=dev)
        m, sc, ze = sets[0]
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        def timed(fn, warm=50, batches=7, reps=10):
            """median over `batches` of the mean launch time of `reps` back-to-back launches, after
            `warm` untimed ones: coming from a lighter phase, the first ~40 launches of a kernel
            that fills the GPU run up to 10 % slower than the steady state (the clocks settle)"""
            with torch.cuda.stream(stream):
                for _ in range(warm):
                    fn()
                stream.synchronize()
                us = []
                for _ in range(batches):
                    e0.record(stream)
                    for _ in range(reps):
                        fn()
                    e1.record(stream)
                    stream.synchronize()
                    us.append(e0.elapsed_time(e1) * 1e3 / reps)
            return sorted(us)[len(us) // 2]

        ws_mm = capi.new_matmul_workspace(1, M, K, S)      # (room to split the last round of tiles along K)
        mm_us = timed(lambda: capi.matmul(4, om, m, xs, sc, ze, g, None, ws_mm))
        flops = 2.0 * M * K * S
        tf = flops / (mm_us * 1e-6) / 1e12
        # spot check: 16 rows against the fp32 oracle
        rows = np.linspace(0, M - 1, 16).astype(int)
        got = om[0, rows].cpu().numpy()
        want_mm = O.matmul_fp32(xs[0, rows].cpu().numpy(), w32)
        mm_err = O.max_rel_error(want_mm, got)
        assert mm_err < 1e-2, f"matmul disagrees with the oracle: {mm_err}"
        # yardstick: the vendor library's plain fp16 GEMM of the same shape and data
        # on this GPU (fp16 weights already in HBM, no dequantisation)
        w16_dev = torch.from_numpy(O.dequantize_matrix(4, p["matrix"], p["scales"], p["zeros"], g)).to(dev)
        with torch.cuda.stream(stream):
            lib_us = timed(lambda: torch.matmul(xs[0], w16_dev))
        del w16_dev
        # the shader clock the power management leaves this kernel (rocm-smi sampled every 0.1 s while it is
        # launched back to back for two seconds): the 2.5 PFLOP/s peak assumes 2.4 GHz on all 256 compute units
        from int4matmul_kernels_amd.harness import shader_clock_under_load
        sclk = shader_clock_under_load(lambda: capi.matmul(4, om, m, xs, sc, ze, g, None, ws_mm), 2.0)
        peak_at_clock = MFMA_FP16_PEAK_TFLOPS * sclk / 2400.0 if sclk else None
        result["gemm"] = {"workload": "int4 dense matmul M=2048 K(N)=5120 S=20480 group=128",
                          "vendor_fp16_gemm_same_shape": {"us": round(lib_us, 2),
                                                          "tflops": round(flops / (lib_us * 1e-6) / 1e12, 1)},
                          "us": round(mm_us, 2), "tflops": round(tf, 1),
                          "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_FP16_PEAK_TFLOPS,
                                       "unit": "TFLOP/s", "frac": round(tf / MFMA_FP16_PEAK_TFLOPS, 4),
                                       "traffic": MATMUL_TRAFFIC_BYTES,
                                       "sclk_mhz_under_load": sclk,
                                       "peak_at_clock": round(peak_at_clock, 1) if peak_at_clock else None,
                                       "frac_at_clock": round(tf / peak_at_clock, 4) if peak_at_clock else None},
                          "max_rel_err_vs_fp32_oracle": float(f"{mm_err:.3e}")}

        # ---- the few-row products in between (a batch of decoding requests): 2, 8 and 64 rows, same weights
        few = {}
        for rows in (2, 8, 64):
            xr = xs[:, :rows].contiguous()
            orow = torch.zeros((1, rows, S), dtype=torch.float16, device=dev)
            ws_r = capi.new_matmul_workspace(1, rows, K, S)
            us = timed(lambda: capi.matmul(4, orow, m, xr, sc, ze, g, None, ws_r), warm=50, batches=7, reps=20)
            got_r = orow[0].cpu().numpy()
            err_r = O.max_rel_error(O.matmul_fp32(xr[0].cpu().numpy(), w32), got_r)
            assert err_r < 1e-2, f"{rows}-row product disagrees with the oracle: {err_r}"
            nb = matvec_bytes(K, S, g) + 2 * rows * (K + S) - 2 * (K + S)
            few[f"rows_{rows}"] = {"us": round(us, 2), "GB/s": round(nb / (us * 1e-6) / 1e9, 1),
                                   "frac_of_hbm_peak": round(nb / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                   "max_rel_err_vs_fp32_oracle": float(f"{err_r:.3e}")}
        result["few_rows"] = {"workload": "int4 dense, K(N)=5120 S=20480 group=128, 2, 8 and 64 rows of states "
                                          "(weights warm in the last-level cache)", **few}

        # ---- the integer helpers either side of the products (pack, unpack, dequantise), HBM-bound: int4 at
        # K = S = 16384, every array larger than the last-level cache; algorithmic bytes = inputs read + outputs written
        if not args.no_helpers:
            Kh = Sh = 16384
            gen = torch.Generator(device=dev).manual_seed(5)
            codes_sk = torch.randint(0, 16, (Sh, Kh), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
            keep = (torch.rand((Sh, Kh // 32, 32), generator=gen, device=dev).argsort(dim=2) < 16).to(torch.uint8).reshape(Sh, Kh)
            m_sp = torch.zeros((Kh // 16, Sh), dtype=torch.int32, device=dev)
            msk = torch.zeros((Kh // 32, Sh), dtype=torch.int32, device=dev)
            codes_ks = codes_sk.t().contiguous()
            m_de = torch.zeros((Kh // 8, Sh), dtype=torch.int32, device=dev)
            out8 = torch.empty((Kh, Sh), dtype=torch.uint8, device=dev)
            w16h = torch.empty((Kh, Sh), dtype=torch.float16, device=dev)
            sch = (torch.rand((Kh // 128, Sh), generator=gen, device=dev) * 0.02).half()
            zeh = (torch.rand((Kh // 128, Sh), generator=gen, device=dev) * 15).half()
            n = Kh * Sh
            legs = {"sparse_pack": (lambda: capi.sparse_pack(m_sp, msk, codes_sk, keep), 2 * n + n // 4 + n // 8),
                    "dense_pack": (lambda: capi.dense_pack(4, m_de, codes_ks), n + n // 2),
                    "unpack": (lambda: capi.unpack(4, out8, None, m_de, None), n // 2 + n),
                    "dequantize": (lambda: capi.dequantize(4, w16h, m_de, sch, zeh, 128, None), n // 2 + 2 * n + 4 * (Kh // 128) * Sh),
                    "plain_copy_same_size": (lambda: out8.copy_(codes_ks), 2 * n)}
            helpers = {}
            for name, (fn, nb) in legs.items():
                us = timed(fn, warm=5, batches=5, reps=5)
                helpers[name] = {"us": round(us, 1), "GB/s": round(nb / (us * 1e-6) / 1e9, 1),
                                 "frac_of_hbm_peak": round(nb / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
            result["helpers"] = {"workload": "int4, K(N)=S=16384 (16:32 pack: uint8 codes and mask [S, K] -> packed words and "
                                             "mask words), cold HBM", **helpers}
            del codes_sk, keep, codes_ks, out8, w16h

    # ---- CPU baseline: torch dequantise + fp32 matmul on the host (reported only)
    if not args.no_cpu:
        from oracle import cpu_baseline

        r = cpu_baseline.time_matvec(p, budget_s=15.0)
        cpu_err = O.max_rel_error(want, r["result"])
        result["cpu_baseline"] = {
            "value": round(nbytes / r["best_s"] / 1e9, 3), "unit": "GB/s", "cores": r["threads"], "kind": "port",
            "sample": f"the full K=5120 S=20480 matvec, best of {r['reps']} repetitions "
                      f"(dequantise {r['dequant_s'] * 1e3:.0f} ms + fp32 matmul {r['matmul_s'] * 1e3:.1f} ms)",
            "us_per_step": round(r["best_s"] * 1e6, 1), "host_cpus": os.cpu_count(),
            "max_rel_err_vs_fp32_oracle": float(f"{cpu_err:.3e}")}

    print(json.dumps(result))


if __name__ == "__main__":
    main()
