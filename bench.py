#!/usr/bin/env python3
"""Headline benchmark: fp32 min-plus SRGEMM at M=N=K=4096 on one MI355X.

One step = one APSP repeated-squaring pass D_out = min(D, D (x) D) on a seeded
4096 x 4096 distance matrix (column-major, 10 % edges, +inf elsewhere), i.e.
one SRGEMM with A = B = C = D, alpha = beta = semiring one (0.0f), additive
identity +inf, ping-pong output buffers.  Inputs are resident in HBM before
the timed region.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size N] [--kernel auto]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_VECTOR_PEAK_TFLOPS = 157.3   # MI355X published FP32 vector peak (FMA, dual rate)
# a min-plus term is one add and half a 3-input min: 1.5 vector instructions
# for 2 ops, against 2 flops per lane-slot for FMA => at most 2/3 of the peak
SEMIRING_CEILING_TOPS = FP32_VECTOR_PEAK_TFLOPS * (2.0 / 1.5) / 2.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--size", type=int, default=4096)
    ap.add_argument("--kernel", default="auto")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="also run one plain device copy of this many MiB (a known-size kernel "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this library runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(no collectives, no sharding in this build).", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import cuasr_amd
    from cuasr_amd import inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    cuasr_amd.load()  # raises if the HIP library is not built (no fallback)
    n = args.size
    dev = torch.device("cuda:0")
    D0_host = inputs.graph_distances(2024, n, density=0.10, lo=1.0, hi=100.0)  # column-major
    # column-major n x n on the device = transpose view of a row-major buffer
    d_in = torch.from_numpy(np.ascontiguousarray(D0_host.T)).to(dev).t()
    bufs = [torch.empty(n, n, device=dev).t() for _ in range(2)]
    inf = float("inf")

    def squaring(src, dst):
        # D_out = min(D (x) D, D): alpha = beta = 0.0f (the min-plus "one"), identity +inf
        cuasr_amd.srgemm("minimum", "plus", src, src, src, dst, 0.0, 0.0, inf, 0.0, kernel=args.kernel)

    def run(steps, start):
        cur = start
        for i in range(steps):
            dst = bufs[i & 1]
            squaring(cur, dst)
            cur = dst
        return cur

    run(args.warmup, d_in)
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    cur = d_in
    ev[0].record()
    for i in range(args.steps):
        dst = bufs[i & 1]
        squaring(cur, dst)
        ev[i + 1].record()
        cur = dst
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms = [ev[i].elapsed_time(ev[i + 1]) for i in range(args.steps)]
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    ops = 2.0 * n * n * n
    value = ops * args.steps / wall / 1e9
    achieved_tops = ops / (avg_kernel_ms * 1e-3) / 1e12

    if args.copy_calibration:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    desc_kernel = args.kernel
    if args.kernel == "auto":
        d = cuasr_amd.make_desc("minimum", "plus", "f32", d_in, d_in, d_in, bufs[0], 0.0, 0.0, inf, 0.0)
        desc_kernel = (cuasr_amd.load().cuasr_amd_selected_kernel(d) or b"?").decode()

    out = {
        "metric": "fp32 min-plus SRGEMM GOPS at 4096^3 (2 ops/term)" if n == 4096
                  else f"fp32 min-plus SRGEMM GOPS at {n}^3 (2 ops/term)",
        "value": round(value, 1), "unit": "GOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"APSP repeated-squaring step, min-plus SRGEMM fp32, M=N=K={n}, column-major, "
                               "D_out = min(D, D (x) D), 10% edges U[1,100), rest +inf, alpha=beta=0.0f (semiring one)",
                   "m": n, "n": n, "k": n, "kernel_family": desc_kernel},
        "roofline": {
            "bound": "valu", "achieved": round(achieved_tops, 3), "peak": FP32_VECTOR_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved_tops / FP32_VECTOR_PEAK_TFLOPS, 4), "traffic": None,
            "kernel_ms_avg": round(avg_kernel_ms, 4), "kernel_ms_min": round(min(kernel_ms), 4),
            "note": "achieved = 2*M*N*K per launch / mean launch duration (HIP events on the launch stream). "
                    "peak = published FP32 vector peak (counts FMA as 2 flops). A min-plus term needs 1.5 vector "
                    "instructions for its 2 ops, so no min-plus code can exceed 2/3 of that peak.",
            "semiring_ceiling_tops": round(SEMIRING_CEILING_TOPS, 1),
            "frac_of_semiring_ceiling": round(achieved_tops / SEMIRING_CEILING_TOPS, 4),
        },
    }

    if not args.no_cpu:
        # CPU baseline: the oracle (a port of the reference host SRGEMM, OpenMP over
        # 32x32 output blocks) on the host cores, running the whole repeated-squaring
        # job (log2(n) squarings) on the same input.  Its final matrix also checks
        # the GPU's, bit for bit.
        import oracle
        threads = oracle.max_threads()
        squarings = max(1, int(np.ceil(np.log2(n))))
        oracle.srgemm("minimum", "plus", D0_host[:64], D0_host, D0_host[:64], 0.0, 0.0, np.inf)  # warm-up
        t1 = time.perf_counter()
        host = D0_host
        for _ in range(squarings):
            host = oracle.srgemm("minimum", "plus", host, host, host, 0.0, 0.0, np.inf)
        cpu_s = time.perf_counter() - t1
        final = run(squarings, d_in)
        torch.cuda.synchronize()
        got = final.cpu().numpy()
        exact = bool(np.ascontiguousarray(got).tobytes() == np.ascontiguousarray(host).tobytes())
        out["cpu_baseline"] = {
            "value": round(squarings * ops / cpu_s / 1e9, 2), "unit": "GOPS", "cores": threads,
            "kind": "port",
            "sample": f"{squarings} repeated squarings of the same {n}x{n} input (M=N=K={n} each), "
                      f"{cpu_s:.2f} s wall on {threads} OpenMP threads",
            "gpu_final_matrix_bit_exact_vs_oracle": exact,
        }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
