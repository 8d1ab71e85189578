"""Benchmark matrix: every pre-tuned semiring x element type x layout x size, one SRGEMM each.

The counterpart of the reference's generated benchmark files (bench/device/simt_sm50.py emits one
case per semiring, layout pair and tile shape; bench/device/harness.h:157-181 runs N = 256 .. 4096
in powers of two with alpha = beta = the multiplicative identity and reports 2 * N^3 / t).  Tile
shapes are the library's business here, so the matrix is semiring x type x layout x size.

    python -m cuasr_amd.bench_matrix [--sizes 256,512,1024,2048,4096] [--dtypes f32,f64]
                                     [--layouts nn,nt,tn,tt] [--kernel auto] [--json out.jsonl] [--bitwise]

Layouts name A and B as the reference does (n = column-major, t = row-major); C and D are
column-major.  Prints a table of TOPS (2 ops per term) and, with --json, one JSON object per case.

    python -m cuasr_amd.bench_matrix --tune [...]

times every case on every kernel family that accepts it as well (the reference's generator sweeps
tile shapes per semiring for this purpose, test/device/simt_sm50.py:193-367) and lists the cases
where the library's own choice (kernel = auto) is more than 3 % slower than the best forced
family: the table the selection rules in csrc/abi.hip are checked against.
"""
import argparse
import ctypes
import json
import sys

SEMIRINGS = [("plus", "multiplies"), ("minimum", "plus"), ("maximum", "plus"), ("minimum", "multiplies"),
             ("maximum", "multiplies"), ("minimum", "maximum"), ("maximum", "minimum"), ("logical_or", "logical_and")]
# the pairs on bits (the reference's user-defined example is xor-and, examples/01_userdefined_semiring): integer types only
BITWISE = [("bit_xor", "bit_and"), ("bit_or", "bit_and")]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", default="256,512,1024,2048,4096")
    ap.add_argument("--dtypes", default="f32,f64", help="any of f32, f64, f16, i8")
    ap.add_argument("--layouts", default="nn,nt,tn,tt")
    ap.add_argument("--kernel", default="auto")
    ap.add_argument("--json", default=None)
    ap.add_argument("--tune", action="store_true", help="also time every forced kernel family; list where auto loses")
    ap.add_argument("--bitwise", action="store_true", help="add xor-and and or-and on bits (dtypes i32, u32, i8)")
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
    losses = []
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
        # (f16: binary16 throughout; i8: int8 A and B, int32 C and D)
        npd, tdt = {"f32": (np.float32, torch.float32), "f64": (np.float64, torch.float64), "f16": (np.float16, torch.float16),
                    "i8": (np.int32, torch.int32), "i32": (np.int32, torch.int32), "u32": (np.uint32, torch.int32)}[dt]
        integer = dt in ("i8", "i32", "u32")
        if args.bitwise and not integer:
            sys.exit("bench_matrix: --bitwise needs integer dtypes (i32, u32, i8)")
        print(f"\n{dt}: TOPS (2 ops per term), layouts of A and B = {' '.join(layouts)}; C, D column-major; kernel = {args.kernel}")
        print("| add-mult | " + " | ".join(f"N={n}" for n in sizes) + " |")
        print("|---|" + "---|" * len(sizes))
        data = {}
        for n in sizes:
            # one buffer per operand and size; a layout is only a way of reading it
            # (seeds further apart than a matrix has elements: the generator is counter-based, and seed s + d gives the
            # stream of seed s moved on by d words -- B would be A moved down by d rows)
            if dt == "i8":
                data[n] = [torch.from_numpy(inputs.integers(901 + (i << 40), n, n, -128, 127, np.int8, "C")).cuda() for i in range(2)]
                data[n].append(torch.from_numpy(inputs.integers(901 + (2 << 40), n, n, -1000, 1000, np.int32, "C")).cuda())
            elif integer:
                # random words for the pairs on bits; (small values would suit the arithmetic pairs, which this table
                # times on the floating-point types)
                data[n] = [torch.from_numpy(inputs.words32(901 + (i << 40), n, n, "C").view(np.int32)).cuda() for i in range(3)]
            else:
                data[n] = [torch.from_numpy(inputs.uniform(901 + (i << 40), n, n, -1.0, 1.0, npd, "C")).cuda() for i in range(3)]
            data[n].append(torch.empty(n, n, dtype=tdt, device="cuda"))
        for add, mult in (BITWISE if args.bitwise else SEMIRINGS):
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
                    def time_family(kernel):
                        # the descriptor is built once: at the small sizes a launch is shorter than building it
                        desc = cuasr_amd.make_desc(add, mult, dt, A, B, C, D, one, one, ident, one, 1, kernel)
                        ref, lib = ctypes.byref(desc), cuasr_amd.load()
                        if lib.cuasr_amd_srgemm_can_implement(ref) != 0:
                            return None, None
                        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

                        def run():
                            if lib.cuasr_amd_srgemm(ref, stream) != 0:
                                raise RuntimeError(f"cuasr_amd_srgemm failed for {add}-{mult} {dt} {n} {lay} {kernel}")
                        # the clock follows the kernel that ran last: give it this kernel for 25 ms before timing
                        w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        w0.record()
                        while True:
                            for _ in range(max(3, reps // 4)):
                                run()
                            w1.record()
                            torch.cuda.synchronize()
                            if w0.elapsed_time(w1) > 25.0:
                                break
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record()
                        for _ in range(reps):
                            run()
                        e1.record()
                        torch.cuda.synchronize()
                        ms = e0.elapsed_time(e1) / reps
                        fam = (lib.cuasr_amd_selected_kernel(desc) or b"?").decode() if kernel == "auto" else kernel
                        return 2.0 * n ** 3 / (ms * 1e-3) / 1e12, fam

                    tops, fam = time_family(args.kernel)
                    if tops is None:
                        raise RuntimeError(f"kernel = {args.kernel} cannot run {add}-{mult} {dt} {n} {lay}")
                    per_layout.append(tops)
                    record = {"add": add, "mult": mult, "dtype": dt, "n": n, "layout": lay, "ms": round(2.0 * n ** 3 / tops / 1e9, 5),
                              "tops": round(tops, 2), "kernel_family": fam}
                    if args.tune:
                        forced = {}
                        for k in ("valu", "direct", "streamk", "mfma"):
                            t, _ = time_family(k)
                            if t is not None:
                                forced[k] = round(t, 2)
                        record["forced"] = forced
                        # the first case after a change of kernel runs on a clock that is still settling:
                        # the library's own choice is timed once more, after the others, and the better time counts
                        again, _ = time_family(args.kernel)
                        tops = max(tops, again)
                        per_layout[-1] = tops
                        record["tops"], record["ms"] = round(tops, 2), round(2.0 * n ** 3 / tops / 1e9, 5)
                        best = max(forced, key=forced.get) if forced else None
                        if best and forced[best] > 1.03 * tops:
                            losses.append((forced[best] / tops, f"{add}-{mult} {dt} N={n} {lay}: auto ({fam}) {tops:.1f}, {best} {forced[best]:.1f}"))
                    if sink:
                        sink.write(json.dumps(record) + "\n")
                cells.append(" ".join(f"{t:.1f}" for t in per_layout))
            print(f"| {add}-{mult} | " + " | ".join(cells) + " |", flush=True)
    if sink:
        sink.close()
    if args.tune:
        print(f"\ncases where kernel = auto is more than 3 % behind the best forced family: {len(losses)}")
        for _, line in sorted(losses, reverse=True):
            print("  " + line)


if __name__ == "__main__":
    main()
