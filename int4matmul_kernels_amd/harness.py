"""Accuracy + timing harness of the quantized products on an MI355X.

Plays the role of the reference's `kernel_test.py` (generation of test
matrices `:160-236`, call convention `:254-259`, error metric `:261-262`, pass
rule `:344-348`, timing loop `:290-309`, markdown table `:359-391`) through the
drop-in `int4matmul` extension module, with three differences: matrices are
packed on the device by the library's own packers (the expected values come from
the unpacked codes, in plain torch arithmetic), each row also reports the
roofline figure of the kernel (GB/s for M = 1, TFLOP/s otherwise), and launches
are additionally timed with HIP events.

    python -m int4matmul_kernels_amd.harness                 # the standard configurations
    python -m int4matmul_kernels_amd.harness --quick         # small shapes only
    python -m int4matmul_kernels_amd.harness --config 4,5120,20480,2048,128,0
    python -m int4matmul_kernels_amd.harness --only C3,C3t --clocks 3    # + shader clock under load
    python -m int4matmul_kernels_amd.harness --only C3,C4m --exponent-every 40   # one group in 40 in exponent mode

A configuration is bits,K,S,M,group,sparse[,B].
"""
import argparse
import time

import torch

import int4matmul_kernels_amd as pkg
from int4matmul_kernels_amd import capi

DEV = "cuda"

# name, bits, K, S, M, group, sparse, B
STANDARD = [
    ("C1", 4, 1024, 1024, 1, 64, False, 1),
    ("C2", 4, 5120, 20480, 1, 128, False, 1),
    ("C2t", 4, 20480, 5120, 1, 128, False, 1),
    ("C3", 4, 5120, 20480, 2048, 128, False, 1),
    ("C3t", 4, 20480, 5120, 2048, 128, False, 1),
    ("C3s", 4, 128, 128, 2048, 128, False, 1),
    ("C4v", 4, 16384, 16384, 1, 64, True, 1),
    ("C4m", 4, 5120, 20480, 2048, 64, True, 1),
    ("C5v3", 3, 5120, 20480, 1, 128, False, 1),
    ("C5m3", 3, 5120, 20480, 2048, 128, False, 1),
    ("C5v2", 2, 5120, 20480, 1, 128, False, 1),
    ("C5m2", 2, 5120, 20480, 2048, 128, False, 1),
]
QUICK = [
    ("q4", 4, 1024, 1024, 1, 64, False, 1),
    ("q4m", 4, 512, 512, 256, 128, False, 1),
    ("q3", 3, 1024, 512, 70, 64, False, 2),
    ("q2", 2, 512, 1024, 1, -1, False, 3),
    ("q4s", 4, 1024, 512, 1, 64, True, 1),
    ("q4sm", 4, 512, 512, 300, 64, True, 1),
]


def make_case(bits, K, S, M, group, sparse, B, seed=0, exponent_every=0):
    """Synthetic problem: codes U{0..2^bits-1}, scales U(0.001, 0.02) (int4) or
    U(0.004, 0.08), zeros U(0, 15) for int4 and the mid-code constant otherwise,
    states N(0, 1); generated on the CPU with a fixed seed, packed on the device.
    `exponent_every` = n > 0: every n-th group of every column gets a negative scale, which switches
    that (group, column) to the exponent quantisation (matmul.cuh:414-428)."""
    gen = torch.Generator().manual_seed(seed)
    codes = torch.randint(0, 1 << bits, (K, S), generator=gen, dtype=torch.int32).to(torch.uint8)
    G = 1 if group < 0 else (K + group - 1) // group
    lo, hi = (0.001, 0.02) if bits == 4 else (0.004, 0.08)
    scales = (torch.rand((G, S), generator=gen) * (hi - lo) + lo).half()
    if bits == 4:
        zeros = (torch.rand((G, S), generator=gen) * 15.0).half()
    else:
        zeros = torch.full((G, S), ((1 << bits) - 1) / 2.0).half()
    if exponent_every > 0:
        scales[exponent_every - 1::exponent_every] *= -1
    states = torch.randn((B, M, K), generator=gen).half()
    codes_d = codes.to(DEV)
    mask = None
    if sparse:
        # a random 16 of every 32 consecutive K per column
        keys = torch.rand((S, K // 32, 32), generator=gen)
        keep = torch.zeros((S, K // 32, 32), dtype=torch.uint8)
        keep.scatter_(2, keys.argsort(dim=2)[:, :, :16], 1)
        keep_d = keep.reshape(S, K).to(DEV)
        matrix = torch.zeros((K // 16, S), dtype=torch.int32, device=DEV)
        mask = torch.zeros((K // 32, S), dtype=torch.int32, device=DEV)
        capi.sparse_pack(matrix, mask, codes_d.t().contiguous(), keep_d)
    else:
        matrix = torch.zeros((K * bits // 32, S), dtype=torch.int32, device=DEV)
        capi.dense_pack(bits, matrix, codes_d)
    keep_ks = keep_d.t().contiguous() if sparse else None            # [K, S], 1 = kept
    return dict(bits=bits, K=K, S=S, M=M, B=B, group=group, matrix=matrix, mask=mask,
                scales=scales.to(DEV), zeros=zeros.to(DEV), states=states.to(DEV), codes=codes_d, keep=keep_ks)


def reference_matrices(c):
    """(fp16 weights as the reference's decode defines them, fp32 weights dequantised in fp32),
    both from the UNPACKED codes and mask the case was generated with, in plain torch arithmetic
    (kernel_test.py:138-157) -- nothing of the library's pack, unpack or dequantise is involved, so
    a packing or decoding bug that the product kernels shared with the helpers would fail the gate"""
    K = c["K"]
    g = K if c["group"] < 0 else c["group"]
    rows = torch.arange(K, device=DEV) // g
    q = c["codes"]
    s16, z16 = c["scales"][rows], c["zeros"][rows]
    w16 = (q.half() - z16) * s16                                     # two fp16 roundings
    w32 = (q.float() - z16.float()) * s16.float()
    expo = s16 < 0
    if bool(expo.any()):
        # exponent mode (matmul.cuh:127-136): +-2^(low bits) * (-scale) + zero, rounded once
        low = (q & ((1 << (c["bits"] - 1)) - 1)).to(torch.int32)
        iv = torch.where((q >> (c["bits"] - 1)) & 1 == 1, -1.0, 1.0).double() * torch.pow(2.0, low.double())
        we = iv * (-s16.double()) + z16.double()
        w16 = torch.where(expo, we.half(), w16)
        w32 = torch.where(expo, we.float(), w32)
    if c["keep"] is not None:
        w16 = w16 * c["keep"].half()
        w32 = w32 * c["keep"].float()
    return w16, w32


def mean_rel_error(truth, cand):
    """the reference's metric: nanmean(|(cand - truth) / truth|)"""
    return ((cand.float() - truth) / truth).abs().nanmean().item()


def algorithmic_bytes(c):
    n = c["matrix"].numel() * 4 + c["scales"].numel() * 2 + c["zeros"].numel() * 2 + 2 * c["K"] + 2 * c["S"]
    if c["mask"] is not None:
        n += c["mask"].numel() * 4
    return n


def shader_clock_under_load(call, seconds):
    """Median shader clock (MHz) that `rocm-smi --showclocks` reports while `call` is launched
    back to back for `seconds`: what the GPU's power management leaves of its peak clock under
    this kernel.  None when the tool gives no reading."""
    import re
    import subprocess
    import threading

    readings, stop = [], threading.Event()

    def sample():
        while not stop.is_set():
            try:
                text = subprocess.run(["rocm-smi", "--showclocks", "--csv"], capture_output=True, text=True,
                                      timeout=5).stdout
            except (OSError, subprocess.SubprocessError):
                return
            header = text.strip().splitlines()[0].split(",") if text.strip() else []
            cols = [i for i, h in enumerate(header) if h.startswith("sclk clock speed")]
            for line in text.strip().splitlines()[1:2]:
                cells = line.split(",")
                for i in cols:
                    m = re.search(r"(\d+)Mhz", cells[i]) if i < len(cells) else None
                    if m:
                        readings.append(int(m.group(1)))
            time.sleep(0.1)

    th = threading.Thread(target=sample)
    th.start()
    t0 = time.time()
    while time.time() - t0 < seconds:
        for _ in range(20):
            call()
        torch.cuda.synchronize()
    stop.set()
    th.join()
    readings = sorted(readings[1:])                       # the first one may predate the load
    return readings[len(readings) // 2] if readings else None


def run_case(name, c, ext, repeats=100, trials=5, cold=False, clocks=0.0):
    B, M, K, S = c["B"], c["M"], c["K"], c["S"]
    w16, w32 = reference_matrices(c)
    truth = c["states"].float() @ w32

    def quant():
        outs = torch.zeros((B, M, S), dtype=torch.float16, device=DEV)
        ext.quant_matmul(c["bits"], outs, c["matrix"], c["states"], c["scales"], c["zeros"], c["group"], c["mask"])
        return outs

    def fp16():
        return c["states"] @ w16

    err_q = mean_rel_error(truth, quant())
    err_h = mean_rel_error(truth, fp16())
    ok = err_q <= 0.1 or not (err_h == err_h)          # the reference's pass rule
    out = {"name": name, "err_quant": err_q, "err_fp16": err_h, "ok": ok}
    for label, fn in (("fp16", fp16), ("quant", quant)):
        # reference-style wall clock: trials x repeats launches including the output allocation
        fn()
        torch.cuda.synchronize()
        walls = []
        for _ in range(trials):
            t0 = time.time()
            for _ in range(repeats):
                fn()
            torch.cuda.synchronize()
            walls.append((time.time() - t0) / repeats)
        out[label + "_wall_us"] = sum(walls) / len(walls) * 1e6
    # kernel-only: HIP events around back-to-back launches into one output buffer.  `cold`: the
    # matvec rotates over enough copies of its weights (about 400 MB, more than the 256 MB
    # last-level cache) that every launch streams them from HBM
    outs = torch.zeros((B, M, S), dtype=torch.float16, device=DEV)
    copies = [(c["matrix"], c["scales"], c["zeros"], c["mask"])]
    if cold and M * B == 1:
        while len(copies) * algorithmic_bytes(c) < 400e6:
            copies.append(tuple(None if t is None else t.clone() for t in copies[0]))
    state = {"i": 0}

    def call():
        m, sc, ze, mk = copies[state["i"] % len(copies)]
        state["i"] += 1
        ext.quant_matmul(c["bits"], outs, m, c["states"], sc, ze, c["group"], mk)
    n = 200 if M == 1 else 20
    for _ in range(5):
        call()
    torch.cuda.synchronize()
    batches = []
    for _ in range(5):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            call()
        e1.record()
        torch.cuda.synchronize()
        batches.append(e0.elapsed_time(e1) * 1e3 / n)
    us = sorted(batches)[len(batches) // 2]
    out["quant_event_us"] = us
    if M * B == 1:
        out["rate"] = "%.0f GB/s" % (algorithmic_bytes(c) / us / 1e3)
    else:
        out["rate"] = "%.1f TFLOP/s" % (2.0 * B * M * K * S / us / 1e6)
    if clocks > 0:
        out["sclk_mhz"] = shader_clock_under_load(call, clocks)
        out["fp16_sclk_mhz"] = shader_clock_under_load(fp16, clocks) if M > 1 else None
    return out


def table(rows, cases):
    head = ["case", "B", "S", "N", "M", "", "weights", "states", "Time (us)", "kernel (us)", "rate", "mean rel err", ""]
    body = []
    for r, (name, bits, K, S, M, group, sparse, B) in zip(rows, cases):
        sp = "16:32" if sparse else ""
        body.append([name, B, S, K, M, sp, "fp16", "fp16", "%.2f" % r["fp16_wall_us"], "", "", "%.2e" % r["err_fp16"], ""])
        body.append([name, B, S, K, M, sp, "int%d" % bits, "fp16", "%.2f" % r["quant_wall_us"],
                     "%.2f" % r["quant_event_us"], r["rate"], "%.2e" % r["err_quant"], "ok" if r["ok"] else "FAIL"])
    cols = list(zip(*([head] + [[str(x) for x in b] for b in body])))
    widths = [max(len(x) for x in col) + 2 for col in cols]
    lines = ["|" + "|".join(h.center(w) for h, w in zip(head, widths)) + "|",
             "|" + "|".join(("-" * (w - 2)).center(w) for w in widths) + "|"]
    for b in body:
        lines.append("|" + "|".join(str(x).rjust(w - 1) + " " for x, w in zip(b, widths)) + "|")
    return "\n".join(lines)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--quick", action="store_true", help="small shapes only")
    ap.add_argument("--config", action="append", default=[], help="bits,K,S,M,group,sparse[,B]")
    ap.add_argument("--repeats", type=int, default=100)
    ap.add_argument("--cold", action="store_true", help="M = 1: rotate over copies of the weights so that every launch reads HBM")
    ap.add_argument("--clocks", type=float, default=0.0, metavar="SECONDS",
                    help="also run each case for SECONDS and report the shader clock rocm-smi shows meanwhile")
    ap.add_argument("--only", default="", help="comma-separated names of standard configurations to run")
    ap.add_argument("--exponent-every", type=int, default=0, metavar="N",
                    help="every N-th quantisation group of every column in exponent mode (a negative scale)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("the harness needs a GPU")
    ext = pkg.load_extension()
    cases = QUICK if args.quick else STANDARD
    if args.only:
        cases = [c for c in STANDARD if c[0] in args.only.split(",")]
    if args.config:
        cases = []
        for i, spec in enumerate(args.config):
            v = [int(x) for x in spec.split(",")]
            cases.append(("u%d" % i, v[0], v[1], v[2], v[3], v[4], bool(v[5]), v[6] if len(v) > 6 else 1))
    rows = []
    for case in cases:
        name, bits, K, S, M, group, sparse, B = case
        c = make_case(bits, K, S, M, group, sparse, B, exponent_every=args.exponent_every)
        rows.append(run_case(name, c, ext, repeats=args.repeats, cold=args.cold, clocks=args.clocks))
        print("%-5s int%d K=%d S=%d M=%d B=%d g=%d %s: %.2f us, %s, mean rel err %.2e %s%s" % (
            name, bits, K, S, M, B, group, "16:32" if sparse else "dense", rows[-1]["quant_event_us"],
            rows[-1]["rate"], rows[-1]["err_quant"], "ok" if rows[-1]["ok"] else "FAIL",
            ", shader clock under load %s MHz (vendor fp16 GEMM: %s)" % (rows[-1]["sclk_mhz"], rows[-1]["fp16_sclk_mhz"])
            if args.clocks > 0 else ""), flush=True)
        del c
        torch.cuda.empty_cache()
    print()
    print(table(rows, cases))
    if not all(r["ok"] for r in rows):
        raise SystemExit("a case exceeded the 10 % mean relative error gate")
    return rows


if __name__ == "__main__":
    main()
