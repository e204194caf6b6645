"""In-kernel timeline of the dense int4 matvec: where a launch spends its time.

``python -m int4matmul_kernels_amd.matvec_timeline [K S [group]]`` runs the
instrumented variant of ``matvec_kernel`` (same code, plus a 100 MHz wall-clock
reading per wave at seven points) on cold weights -- seven weight sets in
rotation, more than the last-level cache holds -- and prints, in microseconds
after the first wave's entry, the minimum / median / 90th percentile / maximum
over all waves of: entry, first requests issued, staging barrier passed, each
64-row unit consumed, workgroup reduction done, end (outputs or hand-over slots
written).  It also prints how the workgroups were spread over the compute units
and when the workgroups of each K split ended.

The instrumented variant is selected by passing the address of a device buffer
through ``int4mm_tune`` key 9 (0 switches it off again); the product path is not
affected when the key is 0.
"""
from __future__ import annotations

import sys

import numpy as np
import torch

from . import capi

STAMPS = 16
WAVE_SLOTS = 8
NAMES = ["entry", "first requests issued", "staging barrier passed"] + [f"unit {i} consumed" for i in range(9)] + \
        ["workgroup reduced", "end"]


def run(K=5120, S=20480, g=128, reps=4, nsets=7, dev="cuda"):
    gen = torch.Generator(device="cpu").manual_seed(0)
    sets = []
    for _ in range(nsets):
        m = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, S), dtype=torch.int32, generator=gen).to(dev)
        sc = torch.empty((K // g, S)).uniform_(0.001, 0.02, generator=gen).half().to(dev)
        ze = torch.empty((K // g, S)).uniform_(0.0, 15.0, generator=gen).half().to(dev)
        sets.append((m, sc, ze))
    x = torch.randn((1, 1, K), generator=gen).half().to(dev)
    outs = torch.zeros((1, 1, S), dtype=torch.float16, device=dev)
    ws = capi.new_workspace(S)
    max_wgs = (S // 64) * 32                              # narrowest strips x most K splits
    tl = torch.zeros((max_wgs, WAVE_SLOTS, STAMPS), dtype=torch.int64, device=dev)
    acc = []
    try:
        for rep in range(reps + 1):
            for i, (m, sc, ze) in enumerate(sets):        # the traced launch comes after six others: cold weights
                last = i == nsets - 1
                if last:
                    tl.zero_()
                    torch.cuda.synchronize()
                capi.tune(9, tl.data_ptr() if last else 0)
                capi.matvec(4, outs, m, x, sc, ze, g, None, ws)
            torch.cuda.synchronize()
            capi.tune(9, 0)
            if rep == 0:
                continue                                   # warm-up
            a = tl.cpu().numpy()
            live = a[:, :, 0] != 0
            t0 = a[:, :, 0][live].min()
            rel = np.where(a[:, :, :14] == 0, np.nan, (a[:, :, :14] - t0) / 100.0)
            rows = []
            for k in range(14):
                v = rel[:, :, k][live]
                v = v[~np.isnan(v)]
                rows.append((v.min(), np.percentile(v, 50), np.percentile(v, 90), v.max()) if len(v) else (np.nan,) * 4)
            acc.append(rows)
            if rep == 1:
                hw = a[:, :, 15][live]
                xcc = (hw >> 32) & 0xF
                key = xcc * 4096 + ((hw >> 8) & 0xFF)      # (XCC, SE / SH / CU bits of HW_ID)
                uniq, cnt = np.unique(key, return_counts=True)
                wg_live = live.any(axis=1)
                wgs = int(wg_live.sum())
                print(f"{wgs} workgroups, {int(live.sum())} waves on {len(uniq)} compute units; waves per compute unit "
                      f"min {cnt.min()} max {cnt.max()}")
                end = np.full(a.shape[0], np.nan)
                end[wg_live] = np.nanmax(np.where(live, rel[:, :, 13], np.nan)[wg_live], axis=1)
                # workgroups are numbered split-major: split = index // strips; find strips from the live count
                idx = np.nonzero(wg_live)[0]
                first_gap = np.nonzero(np.diff(idx) > 1)[0]
                print(f"workgroup end times (us): median {np.nanmedian(end[wg_live]):.2f}, "
                      f"90th percentile {np.nanpercentile(end[wg_live], 90):.2f}, max {np.nanmax(end[wg_live]):.2f}"
                      + ("" if len(first_gap) == 0 else " (non-contiguous workgroup numbering)"))
                # by accelerator die (XCC id of the workgroup's first wave) and by K split (workgroups are
                # numbered split-major: index = split * strips + strip)
                wg_xcc = ((a[:, 0, 15] >> 32) & 0xF)[wg_live]
                e = end[wg_live]
                print("  by die:   " + "  ".join(f"{x}: {np.median(e[wg_xcc == x]):.2f} / {e[wg_xcc == x].max():.2f}"
                                                 for x in np.unique(wg_xcc)) + "   (median / max)")
                for k, name in ((0, "entry"), (1, "first requests issued"), (3, "unit 0 consumed")):
                    v = rel[:, 0, k][wg_live]
                    print(f"            {name}, median by die: " + "  ".join(
                        f"{x}: {np.nanmedian(v[wg_xcc == x]):.2f}" for x in np.unique(wg_xcc)))
                hw0 = a[:, 0, 15][wg_live]
                wg_cu = ((hw0 >> 32) & 0xF) * 4096 + ((hw0 >> 8) & 0xFF)
                cu_end = np.array([e[wg_cu == c].max() for c in np.unique(wg_cu)])
                print(f"  compute units by the end of their last workgroup: min {cu_end.min():.2f}, median "
                      f"{np.median(cu_end):.2f}, 90th percentile {np.percentile(cu_end, 90):.2f}, max {cu_end.max():.2f}")
                shape = dict(kv.split("=") for kv in capi.describe_launch("vec", 4, 1, 1, K, S, g).split() if "=" in kv
                             and kv.split("=")[0] in ("strips", "splits"))
                strips, splits = int(shape["strips"]), int(shape["splits"])
                if splits * strips == wgs and splits > 1:
                    sp = idx // strips
                    print("  by split: " + "  ".join(f"{k}: {np.median(e[sp == k]):.2f} / {e[sp == k].max():.2f}"
                                                     for k in range(splits)))
    finally:
        capi.tune(9, 0)
    acc = np.array(acc).mean(axis=0)
    print(f"int4 dense matvec K={K} S={S} group={g}: microseconds after the first wave's entry "
          f"(min / median / p90 / max over waves, mean of {reps} cold launches)")
    for k, n in enumerate(NAMES):
        if np.isnan(acc[k][0]):
            continue
        print(f"  {n:24s} {acc[k][0]:6.2f} {acc[k][1]:6.2f} {acc[k][2]:6.2f} {acc[k][3]:6.2f}")


if __name__ == "__main__":
    args = [int(v) for v in sys.argv[1:]]
    run(*args[:3])
