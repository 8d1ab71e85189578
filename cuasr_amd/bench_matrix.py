"""Benchmark matrix: every pre-tuned semiring x element type x layout x size, one SRGEMM each.

The counterpart of the reference's generated benchmark files (bench/device/simt_sm50.py emits one
case per semiring, layout pair and tile shape; bench/device/harness.h:157-181 runs N = 256 .. 4096
in powers of two with alpha = beta = the multiplicative identity and reports 2 * N^3 / t).  Tile
shapes are the library's business here, so the matrix is semiring x type x layout x size.

    python -m cuasr_amd.bench_matrix [--sizes 256,512,1024,2048,4096] [--dtypes f32,f64]
                                     [--layouts nn,nt,tn,tt] [--kernel auto] [--json out.jsonl]

Layouts name A and B as the reference does (n = column-major, t = row-major); C and D are
column-major.  Prints a table of TOPS (2 ops per term) and, with --json, one JSON object per case.
"""
import argparse
import ctypes
import json
import sys

SEMIRINGS = [("plus", "multiplies"), ("minimum", "plus"), ("maximum", "plus"), ("minimum", "multiplies"),
             ("maximum", "multiplies"), ("minimum", "maximum"), ("maximum", "minimum"), ("logical_or", "logical_and")]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", default="256,512,1024,2048,4096")
    ap.add_argument("--dtypes", default="f32,f64")
    ap.add_argument("--layouts", default="nn,nt,tn,tt")
    ap.add_argument("--kernel", default="auto")
    ap.add_argument("--json", default=None)
    args = ap.parse_args()

    import numpy as np
    import torch
    import cuasr_amd
    from cuasr_amd import inputs

    if not torch.cuda.is_available():
        sys.exit("bench_matrix: no GPU visible")
    cuasr_amd.load()
    sizes = [int(x) for x in args.sizes.split(",")]
    layouts = args.layouts.split(",")
    sink = open(args.json, "w") if args.json else None
    # the clock takes ~100 ms of load to ramp up: keep the chip busy for a while before the first case
    warm = torch.rand(4096, 4096, device="cuda")
    t_end = torch.cuda.Event(enable_timing=True)
    t_start = torch.cuda.Event(enable_timing=True)
    t_start.record()
    while True:
        for _ in range(20):
            cuasr_amd.srgemm("minimum", "plus", warm, warm, warm, warm.clone(), 0.0, 0.0, float("inf"), 0.0)
        t_end.record()
        torch.cuda.synchronize()
        if t_start.elapsed_time(t_end) > 300.0:
            break
    for dt in args.dtypes.split(","):
        npd, tdt = {"f32": (np.float32, torch.float32), "f64": (np.float64, torch.float64)}[dt]
        print(f"\n{dt}: TOPS (2 ops per term), layouts of A and B = {' '.join(layouts)}; C, D column-major; kernel = {args.kernel}")
        print("| add-mult | " + " | ".join(f"N={n}" for n in sizes) + " |")
        print("|---|" + "---|" * len(sizes))
        data = {}
        for n in sizes:
            # one buffer per operand and size; a layout is only a way of reading it
            data[n] = [torch.from_numpy(inputs.uniform(901 + i, n, n, -1.0, 1.0, npd, "C")).cuda() for i in range(3)]
            data[n].append(torch.empty(n, n, dtype=tdt, device="cuda"))
        for add, mult in SEMIRINGS:
            ident = cuasr_amd.op_identity(add, dt, True)
            one = cuasr_amd.op_identity(mult, dt, True)
            cells = []
            for n in sizes:
                A0, B0, C0, D0 = data[n]
                reps = max(10, min(200, int(1e12 / (2.0 * n ** 3))))
                per_layout = []
                for lay in layouts:
                    A = A0.t() if lay[0] == "n" else A0
                    B = B0.t() if lay[1] == "n" else B0
                    C, D = C0.t(), D0.t()
                    # the descriptor is built once: at the small sizes a launch is shorter than building it
                    desc = cuasr_amd.make_desc(add, mult, dt, A, B, C, D, one, one, ident, one, 1, args.kernel)
                    ref, launch = ctypes.byref(desc), cuasr_amd.load().cuasr_amd_srgemm
                    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

                    def run():
                        if launch(ref, stream) != 0:
                            raise RuntimeError(f"cuasr_amd_srgemm failed for {add}-{mult} {dt} {n} {lay}")
                    for _ in range(max(3, reps // 4)):
                        run()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(reps):
                        run()
                    e1.record()
                    torch.cuda.synchronize()
                    ms = e0.elapsed_time(e1) / reps
                    tops = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
                    per_layout.append(tops)
                    if sink:
                        fam = (cuasr_amd.load().cuasr_amd_selected_kernel(desc) or b"?").decode() if args.kernel == "auto" else args.kernel
                        sink.write(json.dumps({"add": add, "mult": mult, "dtype": dt, "n": n, "layout": lay, "ms": round(ms, 5),
                                               "tops": round(tops, 2), "kernel_family": fam}) + "\n")
                cells.append(" ".join(f"{t:.1f}" for t in per_layout))
            print(f"| {add}-{mult} | " + " | ".join(cells) + " |", flush=True)
    if sink:
        sink.close()


if __name__ == "__main__":
    main()
