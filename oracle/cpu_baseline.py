"""CPU baseline for bench.py: torch-CPU dequantise + fp32 matmul of the same
seeded workload, timed on the host's cores.

TEST / MEASUREMENT INFRASTRUCTURE ONLY.  The reference has no CPU path; this is
the stand-in its harness implies (kernel_test.py:138-157 builds the dequantised
matrix with torch ops, :251-252 multiplies it in fp32): unpack the int32 words
with shifts and masks, ``(q.half() - zeros) * scales`` in fp16 like the
reference's roundings, widen to fp32, ``states.float() @ W``.
"""
from __future__ import annotations

import time

import numpy as np
import torch


def dequant_int4_torch(matrix: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, group_size: int):
    """int32 [K/8, S] -> fp32 [K, S] on the CPU with torch ops."""
    R, S = matrix.shape
    shifts = torch.arange(0, 32, 4, dtype=torch.int32).view(1, 8, 1)
    q = (matrix.view(R, 1, S) >> shifts) & 0xF                      # [R, 8, S]
    q = q.reshape(R * 8, S).to(torch.float16)
    G = scales.shape[0]
    z = zeros.view(G, 1, S).expand(G, group_size, S).reshape(-1, S)[: R * 8]
    s = scales.view(G, 1, S).expand(G, group_size, S).reshape(-1, S)[: R * 8]
    return ((q - z) * s).float()


def time_matvec(problem: dict, budget_s: float = 15.0, max_reps: int = 5):
    """Returns dict(best_s, dequant_s, matmul_s, reps, threads)."""
    m = torch.from_numpy(np.ascontiguousarray(problem["matrix"]))
    sc = torch.from_numpy(np.ascontiguousarray(problem["scales"]))
    ze = torch.from_numpy(np.ascontiguousarray(problem["zeros"]))
    x = torch.from_numpy(np.ascontiguousarray(problem["states"])).float().view(-1, problem["K"])
    g = problem["group_size"]
    best = (float("inf"), 0.0, 0.0)
    reps = 0
    t_start = time.perf_counter()
    y = None
    while reps < max_reps and (reps < 2 or time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        w = dequant_int4_torch(m, sc, ze, g)
        t1 = time.perf_counter()
        y = x @ w
        t2 = time.perf_counter()
        if t2 - t0 < best[0]:
            best = (t2 - t0, t1 - t0, t2 - t1)
        reps += 1
        del w
    return dict(best_s=best[0], dequant_s=best[1], matmul_s=best[2], reps=reps,
                threads=torch.get_num_threads(), result=y.numpy())
