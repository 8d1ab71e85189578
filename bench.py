#!/usr/bin/env python3
"""Semiring-GEMM benchmark on one MI355X.  Prints ONE JSON line.

Default workload (the headline metric): fp32 min-plus SRGEMM at M=N=K=4096.
One step = one APSP repeated-squaring pass D_out = min(D, D (x) D) on a seeded
4096 x 4096 distance matrix (column-major, 10 % edges, +inf elsewhere), i.e.
one SRGEMM with A = B = C = D, alpha = beta = semiring one (0.0f), additive
identity +inf, ping-pong output buffers.  Inputs are resident in HBM before
the timed region.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload apsp] [--size N] [--kernel auto]

Other workloads (same JSON shape; one step = one SRGEMM on fixed inputs):
    maxplus_f64, maxmin_f64   fp64, M=N=K=8192, column-major, U[-1,1), beta = one with a seeded C
    splitk                    fp32 min-plus, M=N=256, K=65536, --slices S (two kernels per step);
                              --serial runs the serial form (the reference's SplitKSerial = true)
    xorand_u32                GF(2) product on bit-packed uint32 words, 4096^3
    plustimes_f32             fp32 plus-times on the matrix cores, 4096^3, N(0,1)
    plustimes_f64             fp64 plus-times on the matrix cores, 4096^3, N(0,1)
    srgemm                    any --add / --mult / --dtype / --layouts at --size (the reference's benchmark matrix)
    functor                   kernels built from user functors (cuasr/gemm/kernel/functor_srgemm.h), fp32 at --size^3:
                              runs cuasr_amd/lib/functor_bench, a program of its own because such kernels are compiled
                              in the user's translation unit; `value` is the pair that computes min-plus through fminf
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
FP32_VECTOR_PEAK = 157.3   # TFLOP/s, FMA counted as 2 flops (also the fp32 matrix-core peak)
FP64_VECTOR_PEAK = 78.6    # also the fp64 matrix-core peak
INT8_MATRIX_PEAK = 5000.0  # TOP/s, dense int8 on the matrix cores
F16_MATRIX_PEAK = 2500.0   # TFLOP/s, dense binary16 on the matrix cores
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the dominant kernel come from profiles/traffic.json, which the profiling
# run writes (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what the same counter reads for
# a plain copy of known size): {"<workload>:<m>x<n>x<k>": {"bytes": ..., "kernel": ..., "commit": ...}}.
# An entry is used only for the kernel family it was measured on.
def measured_traffic(workload, m, n, k, family):
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            e = json.load(f).get(f"{workload}:{m}x{n}x{k}")
    except (OSError, ValueError):
        return None
    if not e or e.get("kernel_family") != family:
        return None
    return e


def settle(step, torch, min_ms=200.0, cap_ms=1500.0):
    """Launch until the clock has settled: at least min_ms of GPU time and three consecutive launches
    within 1 % of each other (the engine clock ramps over the first tens of milliseconds of load)."""
    total, last = 0.0, []
    i = 0
    while total < cap_ms:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        step(i)
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_time(e1)
        total += ms
        last = (last + [ms])[-3:]
        i += 1
        if total >= min_ms and len(last) == 3 and max(last) <= 1.01 * min(last):
            break
    return i


def timed(step, steps, torch):
    """steps launches, HIP events on the launch stream around each: (wall seconds, [ms per launch])."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        step(i)
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]


class PowerSampler:
    """Reads the board's power sensor (hwmon power1_input, microwatts) every 20 ms in a thread; summary() averages
    the readings of the second half of the interval, where the sensor's own averaging has caught up with the load."""

    def __init__(self):
        import glob
        import threading
        hw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
        self.path = next((os.path.join(h, "power1_input") for h in hw if os.path.exists(os.path.join(h, "power1_input"))), None)
        cap = next((os.path.join(h, "power1_cap") for h in hw if os.path.exists(os.path.join(h, "power1_cap"))), None)
        self.cap = self._read(cap) if cap else None
        self.samples, self.stop = [], False
        self.thread = threading.Thread(target=self._run, daemon=True)

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return int(f.read().strip())
        except (OSError, ValueError):
            return None

    def _run(self):
        while not self.stop:
            v = self._read(self.path) if self.path else None
            if v is not None:
                self.samples.append((time.perf_counter(), v))
            time.sleep(0.02)

    def __enter__(self):
        self.t0 = time.perf_counter()
        self.thread.start()
        return self

    def __exit__(self, *exc):
        self.t1 = time.perf_counter()
        self.stop = True
        self.thread.join()

    def summary(self):
        mid = 0.5 * (self.t0 + self.t1)
        late = [v for t, v in self.samples if t >= mid]
        if not late:
            return {"avg_w": None, "samples": 0, "note": "no power sensor reading (hwmon power1_input) during the timed region"}
        return {"avg_w": round(sum(late) / len(late) / 1e6, 1), "cap_w": round(self.cap / 1e6, 1) if self.cap else None,
                "samples": len(late), "sensor": self.path,
                "note": "board power over the second half of the timed region (hwmon power1_input every 20 ms; the first "
                        "card's sensor: on a host with several cards it may not be the one that ran the kernels)"}


def build_workload(args, np, torch, cuasr_amd, inputs):
    """Returns a dict: step(i) launches one step; metadata for the JSON line; sample() for the CPU leg."""
    dev = torch.device("cuda:0")
    inf = float("inf")

    def col_major(host):  # column-major m x n on the device = transpose view of a row-major buffer
        return torch.from_numpy(np.ascontiguousarray(host.T)).to(dev).t()

    def row_major(host):
        return torch.from_numpy(np.ascontiguousarray(host)).to(dev)

    w = args.workload
    if w == "apsp":
        n = args.size or 4096
        D0 = inputs.graph_distances(2024, n, density=0.10, lo=1.0, hi=100.0)
        d_in = col_major(D0)
        bufs = [torch.empty(n, n, device=dev).t() for _ in range(2)]
        state = {"cur": d_in}
        squarings = max(1, int(np.ceil(np.log2(n))))

        def reset():
            state["cur"] = d_in

        def step(i):
            if i % squarings == 0:   # a new job: the timed steps are whole runs of log2(n) squarings of the input graph
                state["cur"] = d_in
            dst = bufs[i & 1]
            cuasr_amd.srgemm("minimum", "plus", state["cur"], state["cur"], state["cur"], dst, 0.0, 0.0, inf, 0.0,
                             kernel=args.kernel)
            state["cur"] = dst

        desc = cuasr_amd.make_desc("minimum", "plus", "f32", d_in, d_in, d_in, bufs[0], 0.0, 0.0, inf, 0.0)
        return dict(step=step, reset=reset, state=state, m=n, n=n, k=n, dtype="f32", desc=desc, host=(D0,),
                    metric=f"fp32 min-plus SRGEMM GOPS at {n}^3 (2 ops/term)",
                    workload=f"APSP repeated-squaring step, min-plus SRGEMM fp32, M=N=K={n}, column-major, "
                             "D_out = min(D, D (x) D), 10% edges U[1,100), rest +inf, alpha=beta=0.0f (semiring one); "
                             f"consecutive steps square the previous result, a new job from the input graph every {squarings} steps",
                    bound="valu", peak=FP32_VECTOR_PEAK, instr_per_term=1.5)

    if w in ("maxplus_f64", "maxmin_f64"):
        n = args.size or 8192
        add, mult = ("maximum", "plus") if w == "maxplus_f64" else ("maximum", "minimum")
        one = 0.0 if w == "maxplus_f64" else inf
        A = inputs.uniform(301, n, n, -1.0, 1.0, np.float64)
        B = inputs.uniform(302, n, n, -1.0, 1.0, np.float64)
        C = inputs.uniform(303, n, n, -1.0, 1.0, np.float64)
        dA, dB, dC = col_major(A), col_major(B), col_major(C)
        dD = torch.empty(n, n, dtype=torch.float64, device=dev).t()

        def step(i):
            cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, one, one, -inf, one, dtype="f64", kernel=args.kernel)

        desc = cuasr_amd.make_desc(add, mult, "f64", dA, dB, dC, dD, one, one, -inf, one)
        return dict(step=step, m=n, n=n, k=n, dtype="f64", desc=desc, host=(add, mult, A, B, C, one, one, -np.inf),
                    result=lambda: dD.cpu().numpy(),
                    metric=f"fp64 {add[:3]}-{mult} SRGEMM GOPS at {n}^3 (2 ops/term)",
                    workload=f"fp64 {add}-{mult} SRGEMM, M=N=K={n}, column-major, U[-1,1), beta = one with a seeded C",
                    bound="valu", peak=FP64_VECTOR_PEAK, instr_per_term=2.0)

    if w == "splitk":
        m = n = args.size or 256
        k = 65536
        A = inputs.uniform(401, m, k, 0.0, 10.0, order="C")   # K contiguous in A and B
        B = inputs.uniform(402, k, n, 0.0, 10.0, order="F")
        C = inputs.uniform(403, m, n, 0.0, 10.0, order="C")
        dA, dB, dC = row_major(A), col_major(B), row_major(C)
        dD = torch.empty(m, n, device=dev)
        ws = torch.empty(cuasr_amd.splitk_workspace_bytes(m, n, args.slices, "f32") // 4, dtype=torch.float32, device=dev)

        run = cuasr_amd.srgemm_splitk_serial if args.serial else cuasr_amd.srgemm_splitk

        def step(i):
            run("minimum", "plus", dA, dB, dC, dD, args.slices, ws, 0.0, 0.0, inf, 0.0)

        import ctypes
        rdesc = cuasr_amd.make_desc("minimum", "plus", "f32", dA, dB, dC, dD, 0.0, 0.0, inf, 0.0, args.slices)

        def reduce_step(i):   # the reduction kernel alone, on the partial tiles the last step left in the workspace
            st = cuasr_amd.load().cuasr_amd_reduce_splitk(ctypes.byref(rdesc), ctypes.c_void_p(ws.data_ptr()),
                                                          ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            assert st == 0, st

        form = "serial-form split-K (ordered chain of epilogues)" if args.serial else "split-K"
        return dict(step=step, m=m, n=n, k=k, dtype="f32", desc=None, host=("minimum", "plus", A, B, C, 0.0, 0.0, np.inf),
                    result=lambda: dD.cpu().numpy(), reduce_step=reduce_step,
                    metric=f"fp32 min-plus {form} SRGEMM GOPS at {m}x{n}x{k}, {args.slices} slices (2 ops/term)",
                    workload=f"{form} min-plus SRGEMM fp32, M=N={m}, K={k}, K contiguous in A and B, U[0,10), "
                             f"{args.slices} slices: partial tiles to a workspace, then a reduction kernel",
                    bound="valu", peak=FP32_VECTOR_PEAK, instr_per_term=1.5, slices=args.slices)

    if w == "xorand_u32":
        n = args.size or 4096
        A, B = inputs.words32(501, n, n), inputs.words32(502, n, n)
        C = np.zeros((n, n), dtype=np.uint32, order="F")
        dA, dB, dC = (col_major(x.view(np.int32)) for x in (A, B, C))
        dD = torch.empty(n, n, dtype=torch.int32, device=dev).t()

        def step(i):
            cuasr_amd.srgemm("bit_xor", "bit_and", dA, dB, dC, dD, 0xFFFFFFFF, 0, 0, 0xFFFFFFFF, dtype="u32", kernel=args.kernel)

        desc = cuasr_amd.make_desc("bit_xor", "bit_and", "u32", dA, dB, dC, dD, 0xFFFFFFFF, 0, 0, 0xFFFFFFFF)
        return dict(step=step, m=n, n=n, k=n, dtype="u32", desc=desc, host=("bit_xor", "bit_and", A, B, C, 0xFFFFFFFF, 0, 0),
                    result=lambda: dD.cpu().numpy(),
                    metric=f"uint32 xor-and SRGEMM GOPS at {n}^3 (2 ops/term)",
                    workload=f"GF(2) xor-and SRGEMM on bit-packed uint32 words, M=N=K={n}, column-major, random words",
                    bound="valu", peak=FP32_VECTOR_PEAK, instr_per_term=1.0)  # one v_bitop3_b32 per term

    if w == "plustimes_f32":
        n = args.size or 4096
        A, B = inputs.normal(601, n, n), inputs.normal(602, n, n)
        C = np.zeros((n, n), dtype=np.float32, order="F")
        dA, dB, dC = col_major(A), col_major(B), col_major(C)
        dD = torch.empty(n, n, device=dev).t()

        def step(i):
            cuasr_amd.srgemm("plus", "multiplies", dA, dB, dC, dD, 1.0, 0.0, 0.0, 1.0, kernel=args.kernel)

        desc = cuasr_amd.make_desc("plus", "multiplies", "f32", dA, dB, dC, dD, 1.0, 0.0, 0.0, 1.0)
        return dict(step=step, m=n, n=n, k=n, dtype="f32", desc=desc, host=("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0),
                    result=lambda: dD.cpu().numpy(),
                    metric=f"fp32 plus-times SRGEMM GFLOP/s at {n}^3 (2 flops/term)",
                    workload=f"plus-times SRGEMM fp32 on the matrix cores, M=N=K={n}, column-major, N(0,1), C = 0",
                    bound="mfma", peak=FP32_VECTOR_PEAK, instr_per_term=None)

    if w == "plustimes_f64":
        n = args.size or 4096
        A = inputs.normal(611, n, n).astype(np.float64, order="F")
        B = inputs.normal(612, n, n).astype(np.float64, order="F")
        C = np.zeros((n, n), dtype=np.float64, order="F")
        dA, dB, dC = col_major(A), col_major(B), col_major(C)
        dD = torch.empty(n, n, dtype=torch.float64, device=dev).t()

        def step(i):
            cuasr_amd.srgemm("plus", "multiplies", dA, dB, dC, dD, 1.0, 0.0, 0.0, 1.0, dtype="f64", kernel=args.kernel)

        desc = cuasr_amd.make_desc("plus", "multiplies", "f64", dA, dB, dC, dD, 1.0, 0.0, 0.0, 1.0)
        return dict(step=step, m=n, n=n, k=n, dtype="f64", desc=desc, host=("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0),
                    metric=f"fp64 plus-times SRGEMM GFLOP/s at {n}^3 (2 flops/term)",
                    workload=f"plus-times SRGEMM fp64 on the matrix cores, M=N=K={n}, column-major, N(0,1), C = 0",
                    bound="mfma", peak=FP64_VECTOR_PEAK, instr_per_term=None)

    if w == "fwgemm":
        # one step of all-pairs shortest paths WITH predecessor tracking: the library snapshots dist (and
        # its transpose) into the workspace and runs the min-plus product that records the first k of
        # every improvement
        n = args.size or 4096
        D0 = inputs.graph_distances(2024, n, density=0.10, lo=1.0, hi=100.0)
        d0 = col_major(D0)
        dist = torch.empty(n, n, device=dev).t()
        parent = torch.empty(n, n, dtype=torch.int32, device=dev).t()
        ws = torch.empty(cuasr_amd.apsp_workspace_bytes(n, "f32") // 4, dtype=torch.float32, device=dev)
        squarings = max(1, int(np.ceil(np.log2(max(2, n - 1)))))

        def restart():
            dist.copy_(d0)
            parent.fill_(-1)

        def step(i):
            if i % squarings == 0:   # a new job every `squarings` steps, so every job's first (improving) steps are timed
                restart()
            cuasr_amd.apsp_squaring(dist, parent, ws, iterations=1)

        return dict(step=step, reset=restart, m=n, n=n, k=n, dtype="f32", desc=None, host=(D0,), family="fwgemm_tile",
                    fw=dict(dist=dist, parent=parent, ws=ws, squarings=squarings),
                    metric=f"fp32 min-plus product with predecessor tracking GOPS at {n}^3 (2 ops/term)",
                    workload=f"APSP repeated-squaring step with predecessor tracking (cpu_fwgemm_naive semantics), fp32, "
                             f"M=N=K={n}, column-major, 10% edges U[1,100), rest +inf; a step = snapshot of dist and its "
                             f"transpose into the workspace + product; a new job (dist, parent reset) every {squarings} steps",
                    bound="valu", peak=FP32_VECTOR_PEAK, instr_per_term=1.5)

    if w == "apsp_blocked":
        # a whole all-pairs shortest-path job with predecessor tracking by blocked Floyd-Warshall:
        # one step = reset dist and parent, then the n / 128 block steps (2 * n^3 operations in all)
        n = args.size or 4096
        dt = args.dtype if args.dtype == "f64" else "f32"
        D0 = inputs.graph_distances(2024, n, density=0.10, lo=1.0, hi=100.0)
        if dt == "f64":
            D0 = D0.astype(np.float64)
        d0 = col_major(D0)
        dist = torch.empty(n, n, dtype=d0.dtype, device=dev).t()
        parent = torch.empty(n, n, dtype=torch.int32, device=dev).t()
        ws = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(n, dt), dtype=torch.uint8, device=dev)

        def step(i):
            dist.copy_(d0)
            parent.fill_(-1)
            cuasr_amd.apsp_blocked(dist, parent, ws)

        bits = "fp64" if dt == "f64" else "fp32"
        return dict(step=step, m=n, n=n, k=n, dtype=dt, desc=None, host=(D0,), family="fwgemm_tile + fw_close_dist",
                    fw=dict(dist=dist, parent=parent),
                    metric=f"{bits} all-pairs shortest paths with predecessors, blocked Floyd-Warshall, GOPS at n={n} "
                           "(2 ops/term, 2*n^3 per job)",
                    workload=f"whole APSP job with predecessor tracking by blocked Floyd-Warshall (128-vertex blocks), {bits}, "
                             f"n={n}, column-major, 10% edges U[1,100), rest +inf; a step = reset of dist and parent + "
                             f"{(n + 127) // 128} block steps",
                    bound="valu", peak=FP64_VECTOR_PEAK if dt == "f64" else FP32_VECTOR_PEAK,
                    instr_per_term=2.0 if dt == "f64" else 1.5)

    if w == "srgemm":
        # any operator pair / element type / layout combination at one size: the reference's
        # benchmark matrix (bench/device/harness.h:157-181 counts 2 * N^3 / t the same way)
        n = args.size or 4096
        add, mult, dt = args.add, args.mult, args.dtype
        npd = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "u32": np.uint32, "f16": np.float16, "i8": np.int32}[dt]
        la, lb, lc = ["F" if c == "c" else "C" for c in args.layouts]
        if dt == "i8":
            # int8 operands over their whole range, int32 C and D
            A, B = (inputs.integers(701 + i, n, n, -128, 127, np.int8, o) for i, o in enumerate((la, lb)))
            C = inputs.integers(703, n, n, -100000, 100000, np.int32, lc)
        elif dt == "f16" and mult != "multiplies":
            # distances of a few units: sums stay well inside binary16's range and still round
            A, B, C = (inputs.uniform(701 + i, n, n, 0.5, 100.0, npd, o) for i, o in enumerate((la, lb, lc)))
        elif dt in ("f32", "f64", "f16"):
            A, B, C = (inputs.uniform(701 + i, n, n, -1.0, 1.0, npd, o) for i, o in enumerate((la, lb, lc)))
        elif dt == "u32":
            A, B, C = (inputs.words32(701 + i, n, n, o) for i, o in enumerate((la, lb, lc)))
        else:
            A, B, C = (inputs.integers(701 + i, n, n, 0, 8, npd, o) for i, o in enumerate((la, lb, lc)))
        ident = cuasr_amd.op_identity(add, dt, True)
        one = cuasr_amd.op_identity(mult, dt, True)
        up = lambda X: (col_major if X.flags.f_contiguous else row_major)(X.view(np.int32) if dt == "u32" else X)
        dA, dB, dC = up(A), up(B), up(C)
        tdt = {"f32": torch.float32, "f64": torch.float64, "i32": torch.int32, "u32": torch.int32, "f16": torch.float16, "i8": torch.int32}[dt]
        dD = torch.empty(n, n, dtype=tdt, device=dev)
        dD = dD.t() if lc == "F" else dD

        if args.kernel == "vendor":
            # a yardstick, not this library: the vendor BLAS behind PyTorch on the same device operands
            # (plus-times only; the int8 product has no fused source term there, so it reads no C)
            if not (add == "plus" and mult == "multiplies" and dt in ("f32", "f64", "f16", "i8")):
                raise SystemExit("bench.py: --kernel vendor times the vendor BLAS, which has plus-times on f32, f64, f16, i8 only")

            def step(i):
                if dt == "i8":
                    torch._int_mm(dA, dB, out=dD)
                else:
                    torch.addmm(dC, dA, dB, out=dD)

            desc = None
        else:
            def step(i):
                cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, one, one, ident, one, dtype=dt, kernel=args.kernel)

            desc = cuasr_amd.make_desc(add, mult, dt, dA, dB, dC, dD, one, one, ident, one, kernel=args.kernel)
        # (binary16 plus-times runs on the matrix cores, with float accumulation, only when asked to)
        matrix = add == "plus" and mult == "multiplies" and (dt in ("f32", "f64", "i8") or (dt == "f16" and args.kernel in ("mfma", "vendor")))
        return dict(step=step, m=n, n=n, k=n, dtype=dt, desc=desc, host=(add, mult, A, B, C, one, one, ident),
                    result=lambda: dD.cpu().numpy(),
                    metric=f"{dt} {add}-{mult} SRGEMM GOPS at {n}^3 (2 ops/term)",
                    workload=f"{add}-{mult} SRGEMM {dt}, M=N=K={n}, layouts (A, B, C) = {args.layouts} "
                             "(c = column-major, r = row-major), beta = one with a seeded C"
                             + (" -- timed on the vendor BLAS behind PyTorch, as a yardstick" if args.kernel == "vendor" else ""),
                    bound="mfma" if matrix else "valu",
                    peak=FP64_VECTOR_PEAK if dt == "f64" else INT8_MATRIX_PEAK if (dt == "i8" and matrix)
                    else F16_MATRIX_PEAK if (dt == "f16" and matrix) else FP32_VECTOR_PEAK,
                    instr_per_term=None)

    raise SystemExit(f"bench.py: unknown workload {w!r}")


FUNCTOR_BENCH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cuasr_amd", "lib", "functor_bench")


def functor_lines(size, steps, warmup):
    """Kernels built from user functors (cuasr/gemm/kernel/functor_srgemm.h) are compiled in the user's translation
    unit, so they are measured by a program of their own, cuasr_amd/lib/functor_bench (built from
    cuasr_amd/functor_bench.hip by `python -m cuasr_amd.build`): its JSON lines, parsed."""
    import subprocess
    if not os.path.exists(FUNCTOR_BENCH):
        raise SystemExit("bench.py: cuasr_amd/lib/functor_bench is not built (python -m cuasr_amd.build)")
    r = subprocess.run([FUNCTOR_BENCH, str(size), str(steps), str(warmup)], capture_output=True, text=True, timeout=600)
    if r.returncode != 0:
        raise SystemExit(f"bench.py: functor_bench failed ({r.returncode}): {r.stderr[-500:]}")
    return [json.loads(line) for line in r.stdout.splitlines() if line.startswith("{")]


def extra_configs(np, torch, cuasr_amd, inputs, oracle, base_args):
    """The other BASELINE configs, timed in the same process (a few launches each) and checked against the
    oracle on a sample: [{workload, ms, tops, frac, kernel_family, bit_exact | within_tolerance}]."""
    out = []

    def ns(**kw):
        a = argparse.Namespace(**vars(base_args))
        a.kernel, a.size, a.serial = "auto", 0, False
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    def family_of(wl, fallback):
        if wl["desc"] is None:
            return fallback
        return (cuasr_amd.load().cuasr_amd_selected_kernel(wl["desc"]) or b"?").decode()

    def measure(wl, budget_ms=60.0):
        step = wl["step"]
        # the oracle's check of the config before left the GPU idle: let the clock come back first
        settle(step, torch, min_ms=60.0, cap_ms=400.0)
        _, first = timed(step, 2, torch)
        steps = int(max(3, min(300, budget_ms / max(min(first), 1e-3))))
        _, ms = timed(step, steps, torch)
        return sum(ms) / len(ms), steps

    def entry(wl, ms, steps, family, **check):
        tops = 2.0 * wl["m"] * wl["n"] * wl["k"] / (ms * 1e-3) / 1e12
        e = {"workload": wl["workload"], "ms": round(ms, 4), "launches": steps, "tops": round(tops, 2),
             "frac": round(tops / wl["peak"], 4), "peak": wl["peak"], "bound": wl["bound"], "kernel_family": family}
        e.update(check)
        return e

    def rows_of(X, rows):
        return np.ascontiguousarray(X[:rows]) if X.flags.c_contiguous else np.asfortranarray(X[:rows])

    # C1: min-plus f32 1024^3, column-major (the srgemm workload: beta = one with a seeded C)
    wl = build_workload(ns(workload="srgemm", add="minimum", mult="plus", dtype="f32", layouts="ccc", size=1024), np, torch, cuasr_amd, inputs)
    ms, steps = measure(wl)
    add, mult, A, B, C, alpha, beta, ident = wl["host"]
    wl["step"](0)
    torch.cuda.synchronize()
    want = oracle.srgemm(add, mult, A, B, C, alpha, beta, ident)
    out.append(entry(wl, ms, steps, family_of(wl, "?"), bit_exact=bool(wl["result"]().tobytes() == np.ascontiguousarray(want).tobytes())))

    # C3: fp64 max-plus and max-min 8192^3; a 512 x 512 block against the oracle
    for w in ("maxplus_f64", "maxmin_f64"):
        wl = build_workload(ns(workload=w), np, torch, cuasr_amd, inputs)
        ms, steps = measure(wl, 150.0)
        add, mult, A, B, C, alpha, beta, ident = wl["host"]
        r0, c0 = 3 * 512 + 17, 9 * 512 + 5
        want = oracle.srgemm(add, mult, np.asfortranarray(A[r0:r0 + 512, :]), np.asfortranarray(B[:, c0:c0 + 512]),
                             np.asfortranarray(C[r0:r0 + 512, c0:c0 + 512]), alpha, beta, ident)
        got = wl["result"]()[r0:r0 + 512, c0:c0 + 512]
        out.append(entry(wl, ms, steps, family_of(wl, "?"), bit_exact=bool(np.asfortranarray(got).tobytes() == np.asfortranarray(want).tobytes()),
                         checked="512 x 512 block of the output"))
        del wl
        torch.cuda.empty_cache()

    # C4: split-K 256 x 256 x 65536, 8 and 64 slices; the reduction kernel on its own as well
    want = None
    for slices in (8, 16, 32, 64):
        wl = build_workload(ns(workload="splitk", slices=slices), np, torch, cuasr_amd, inputs)
        ms, steps = measure(wl)
        add, mult, A, B, C, alpha, beta, ident = wl["host"]
        if want is None:
            want = oracle.srgemm(add, mult, A, B, C, alpha, beta, ident)
        red_step = wl["reduce_step"]
        _, rms = timed(red_step, 50, torch)
        rms = sorted(rms)[len(rms) // 2]
        red_bytes = (slices + 2) * wl["m"] * wl["n"] * 4      # S partial tiles + C read, D written
        out.append(entry(wl, ms, steps, "valu (64x64x32 staged tile) + reduce_splitk_kernel",
                         bit_exact=bool(wl["result"]().tobytes() == np.ascontiguousarray(want).tobytes()),
                         split_k_slices=slices, reduce_kernel_ms=round(rms, 5), reduce_kernel_bytes=red_bytes,
                         reduce_kernel_gbs=round(red_bytes / (rms * 1e-3) / 1e9, 1),
                         reduce_note="partial tiles of this size stay in the last-level caches: an effective rate, not an HBM rate"))

    # C5a: xor-and on bit-packed uint32 words, 4096^3; the first 256 rows against the oracle
    wl = build_workload(ns(workload="xorand_u32"), np, torch, cuasr_amd, inputs)
    ms, steps = measure(wl)
    add, mult, A, B, C, alpha, beta, ident = wl["host"]
    want = oracle.srgemm(add, mult, rows_of(A, 256), B, rows_of(C, 256), alpha, beta, ident)
    got = wl["result"]().view(np.uint32)[:256]
    out.append(entry(wl, ms, steps, family_of(wl, "?"), bit_exact=bool(np.asfortranarray(got).tobytes() == np.asfortranarray(want).tobytes()),
                     checked="first 256 rows of the output"))

    # C5b: plus-times f32 on the matrix cores, 4096^3; |d - r| <= 1e-5 * sum |a||b| on the first 256 rows
    wl = build_workload(ns(workload="plustimes_f32"), np, torch, cuasr_amd, inputs)
    ms, steps = measure(wl)
    add, mult, A, B, C, alpha, beta, ident = wl["host"]
    want = oracle.srgemm(add, mult, rows_of(A, 256), B, rows_of(C, 256), alpha, beta, ident).astype(np.float64)
    bound = 1e-5 * (np.abs(A[:256]).astype(np.float64) @ np.abs(B).astype(np.float64))
    got = wl["result"]()[:256].astype(np.float64)
    out.append(entry(wl, ms, steps, family_of(wl, "?"), within_tolerance=bool((np.abs(got - want) <= bound).all()),
                     tolerance="|d - r| <= 1e-5 * sum_k |a||b|, first 256 rows"))
    del wl
    torch.cuda.empty_cache()

    # Half precision (the reference names it as an aim, README.md:11): min-plus on binary16, 4096^3, column-major;
    # the first 64 rows against the oracle, which rounds every sum to binary16 as the device does
    wl = build_workload(ns(workload="srgemm", add="minimum", mult="plus", dtype="f16", layouts="ccc", size=4096), np, torch, cuasr_amd, inputs)
    ms, steps = measure(wl)
    add, mult, A, B, C, alpha, beta, ident = wl["host"]
    want = oracle.srgemm(add, mult, rows_of(A, 64), B, rows_of(C, 64), alpha, beta, ident)
    got = wl["result"]()[:64]
    out.append(entry(wl, ms, steps, family_of(wl, "?"), bit_exact=bool(np.asfortranarray(got).tobytes() == np.asfortranarray(want).tobytes()),
                     checked="first 64 rows of the output",
                     note="packed binary16 instructions issue at half the rate of 4-byte ones: two terms per instruction, the same vector peak"))
    del wl
    torch.cuda.empty_cache()

    # binary16 plus-times with float accumulation on the matrix cores (the reference's ElementAccumulator = float for
    # half operands; by request only: kernel = mfma), 4096^3, A row-major and B column-major; the first 256 rows
    # against a double-precision product: one binary16 rounding of the result plus the error of a float sum
    wl = build_workload(ns(workload="srgemm", add="plus", mult="multiplies", dtype="f16", layouts="rcr", size=4096, kernel="mfma"),
                        np, torch, cuasr_amd, inputs)
    ms, steps = measure(wl)
    add, mult, A, B, C, alpha, beta, ident = wl["host"]
    a64, b64 = A[:256].astype(np.float64), B.astype(np.float64)
    want = float(alpha) * (a64 @ b64) + float(beta) * C[:256].astype(np.float64)
    bound = 2.0 ** -11 * np.abs(want) + 1e-5 * (np.abs(a64) @ np.abs(b64)) + 1e-7
    got = wl["result"]()[:256].astype(np.float64)
    out.append(entry(wl, ms, steps, "mfma", within_tolerance=bool((np.abs(got - want) <= bound).all()),
                     tolerance="|d - r| <= 2^-11 |r| + 1e-5 * sum_k |a||b| against a double-precision product, first 256 rows",
                     note="float accumulation: not bit-identical to the all-binary16 sums the library computes by default (65 TFLOP/s on the vector ALU)"))
    del wl
    torch.cuda.empty_cache()

    # int8 operands with int32 accumulation (the element types of the reference's dp4a cores,
    # default_srmma_core_simt.h:747-757), plus-times on the matrix cores, 4096^3, A row-major and B column-major
    # (both k-contiguous); the first 256 rows against the oracle
    wl = build_workload(ns(workload="srgemm", add="plus", mult="multiplies", dtype="i8", layouts="rcr", size=4096), np, torch, cuasr_amd, inputs)
    ms, steps = measure(wl)
    add, mult, A, B, C, alpha, beta, ident = wl["host"]
    want = oracle.srgemm(add, mult, rows_of(A, 256), B, rows_of(C, 256), int(alpha), int(beta), int(ident))
    got = wl["result"]()[:256]
    out.append(entry(wl, ms, steps, family_of(wl, "?"), bit_exact=bool(np.ascontiguousarray(got).tobytes() == np.ascontiguousarray(want).tobytes()),
                     checked="first 256 rows of the output"))
    del wl
    torch.cuda.empty_cache()

    # Kernels built from user functors (none of the library's operators): fp32 at 4096^3 for a functor pair that
    # computes min-plus (compared bit for bit, by the program itself, with the tuned min-plus kernel, which the
    # headline's check pins against the oracle), one spelled as the reference spells its minimum, one no library
    # operator computes; the quarter-size tile at 1024^3; split-K 256 x 256 x 65536
    for line in functor_lines(4096, 10, 5):
        e = {"workload": line["workload"], "ms": line["ms"], "tops": line["tops"], "frac": round(line["tops"] / 157.3, 4),
             "peak": 157.3, "bound": "valu", "kernel_family": "functor_srgemm_kernel (built from the user's functors by hipcc)"}
        if line.get("bit_identical_to_tuned_min_plus") is not None:
            e["bit_exact"] = bool(line["bit_identical_to_tuned_min_plus"])
            e["checked"] = "whole matrix against the library's tuned min-plus kernel on the same operands"
        out.append(e)

    # All-pairs shortest paths with predecessors on top of SRGEMM (README.md:338-342 of the reference,
    # cpu_fwgemm_naive): a whole job at n = 4096 by blocked Floyd-Warshall, counted as 2 n^3 operations, and the
    # same kind of graph at n = 1024 against the oracle's blocked iteration, dist and parent bit for bit
    wl = build_workload(ns(workload="apsp_blocked"), np, torch, cuasr_amd, inputs)
    ms, steps = measure(wl, 80.0)
    nc = 1024
    Dc = inputs.graph_distances(2024, nc, density=0.10, lo=1.0, hi=100.0)
    hd, hp = Dc.copy(order="F"), np.full((nc, nc), -1, dtype=np.int32, order="F")
    oracle.apsp_blocked(hd, hp, 128)
    gd = torch.from_numpy(np.ascontiguousarray(Dc.T)).to("cuda:0").t()
    gp = torch.full((nc, nc), -1, dtype=torch.int32, device="cuda:0").t()
    gws = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(nc, "f32"), dtype=torch.uint8, device="cuda:0")
    cuasr_amd.apsp_blocked(gd, gp, gws)
    torch.cuda.synchronize()
    exact = bool(np.ascontiguousarray(gd.cpu().numpy()).tobytes() == np.ascontiguousarray(hd).tobytes() and (gp.cpu().numpy() == hp).all())
    out.append(entry(wl, ms, steps, "fw_diagonal + fwgemm_pair + fwgemm_tile (closing the next diagonal block)",
                     bit_exact=exact, checked=f"dist and parent of the same job at n = {nc}"))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="apsp",
                    choices=["apsp", "maxplus_f64", "maxmin_f64", "splitk", "xorand_u32", "plustimes_f32", "plustimes_f64",
                             "srgemm", "fwgemm", "apsp_blocked", "functor"])
    ap.add_argument("--add", default="minimum", help="workload srgemm: the semiring's add operator")
    ap.add_argument("--mult", default="plus", help="workload srgemm: the semiring's multiply operator")
    ap.add_argument("--dtype", default="f32", choices=["f32", "f64", "i32", "u32", "f16", "i8"], help="workload srgemm")
    ap.add_argument("--layouts", default="ccc", help="workload srgemm: layouts of A, B, C (c = column-major, r = row-major)")
    ap.add_argument("--size", type=int, default=0, help="override the workload's M=N (and K where it is square)")
    ap.add_argument("--slices", type=int, default=64, help="split-K slices (workload splitk)")
    ap.add_argument("--serial", action="store_true", help="workload splitk: the serial form (SplitKSerial = true)")
    ap.add_argument("--kernel", default="auto",
                    help="a kernel family of the library, or (workload srgemm, plus-times) vendor: the vendor BLAS as a yardstick")
    ap.add_argument("--no-power", dest="power", action="store_false",
                    help="do not read the board's power sensor during the timed region (the reading settles over about a "
                         "second of load: give --steps that much work for a figure to quote)")
    ap.add_argument("--power", dest="power", action="store_true", help="(the default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="headline only: do not time the other configs (extra.configs)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="also run one plain device copy of this many MiB (a known-size kernel "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this library runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(no collectives, no sharding in this build).", file=sys.stderr)
        sys.exit(2)

    if args.workload == "functor":
        # measured by a program of its own (the kernels are built in the user's translation unit); --steps / --warmup
        # are launches per functor pair
        n = args.size or 4096
        lines = functor_lines(n, args.steps, args.warmup)
        head = lines[0]
        print(json.dumps({
            "metric": f"fp32 min-plus SRGEMM GOPS at {n}^3 (2 ops/term) on a kernel built from user functors, 1 GPU",
            "value": round(head["tops"] * 1e3, 1), "unit": "GOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": head["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic", "config": {"workload": head["workload"], "m": n, "n": n, "k": n,
                                            "kernel_family": "functor_srgemm_kernel (built from the user's functors by hipcc)"},
            "roofline": {"bound": "valu", "achieved": head["tops"], "peak": 157.3, "unit": "TOPS", "frac": round(head["tops"] / 157.3, 4),
                         "traffic": None},
            "bit_identical_to_tuned_min_plus": head.get("bit_identical_to_tuned_min_plus"),
            "extra": {"functor_pairs": lines}}), flush=True)
        return

    import numpy as np
    import torch
    import cuasr_amd
    from cuasr_amd import inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    cuasr_amd.load()  # raises if the HIP library is not built (no fallback)
    wl = build_workload(args, np, torch, cuasr_amd, inputs)
    step = wl["step"]
    m, n, k = wl["m"], wl["n"], wl["k"]

    settled = settle(step, torch)      # whatever --warmup says: a short warm-up must not time the clock ramp
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    if "reset" in wl:
        wl["reset"]()
    if args.power:
        with PowerSampler() as power:
            wall, kernel_ms = timed(step, args.steps, torch)
    else:
        wall, kernel_ms = timed(step, args.steps, torch)
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    ops = 2.0 * m * n * k
    value = ops * args.steps / wall / 1e9
    achieved_tops = ops / (avg_kernel_ms * 1e-3) / 1e12

    if args.copy_calibration:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    family = wl.get("family", args.kernel)
    if args.kernel == "auto" and wl["desc"] is not None:
        family = (cuasr_amd.load().cuasr_amd_selected_kernel(wl["desc"]) or b"?").decode()

    roof = {
        "bound": wl["bound"], "achieved": round(achieved_tops, 3), "peak": wl["peak"], "unit": "TFLOP/s",
        "frac": round(achieved_tops / wl["peak"], 4),
        "traffic": None,
        "kernel_ms_avg": round(avg_kernel_ms, 4), "kernel_ms_min": round(min(kernel_ms), 4),
        "note": "achieved = 2*M*N*K per launch / mean launch duration (HIP events on the launch stream); "
                "peak = published vector / matrix peak of the element type (FMA = 2 flops).",
    }
    traffic = measured_traffic(args.workload, m, n, k, family)
    if traffic:
        roof["traffic"] = traffic["bytes"]
        roof["traffic_source"] = f"profiles/traffic.json: {traffic.get('kernel', '?')} at commit {traffic.get('commit', '?')}"
    if wl["instr_per_term"]:
        # a semiring term that needs i vector instructions for its 2 ops cannot beat peak / i
        ceiling = wl["peak"] / wl["instr_per_term"]
        roof["semiring_ceiling_tops"] = round(ceiling, 1)
        roof["frac_of_semiring_ceiling"] = round(achieved_tops / ceiling, 4)
        roof["note"] += f" A term of this semiring costs {wl['instr_per_term']} vector instructions, an FMA 1: " \
                        "semiring_ceiling = peak / that."
    out = {
        "metric": wl["metric"], "value": round(value, 1), "unit": "GOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_launches": settled, "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": wl["dtype"], "data": "synthetic",
        "config": {"workload": wl["workload"], "m": m, "n": n, "k": k, "kernel_family": family},
        "roofline": roof,
    }
    if "slices" in wl:
        out["config"]["split_k_slices"] = wl["slices"]
    if args.power:
        out["power"] = power.summary()

    if not args.no_cpu:
        # CPU baseline: the oracle (a port of the reference host SRGEMM, OpenMP over 32x32 output
        # blocks) on the host cores, on a bounded sample of the same workload; its result also
        # checks the GPU's.
        import oracle
        threads = oracle.max_threads()
        if args.workload == "apsp":
            D0 = wl["host"][0]
            squarings = max(1, int(np.ceil(np.log2(n))))
            oracle.srgemm("minimum", "plus", D0[:64], D0, D0[:64], 0.0, 0.0, np.inf)  # warm-up
            t1 = time.perf_counter()
            host = D0
            for _ in range(squarings):
                host = oracle.srgemm("minimum", "plus", host, host, host, 0.0, 0.0, np.inf)
            cpu_s = time.perf_counter() - t1
            wl["reset"]()
            for i in range(squarings):
                step(i)
            torch.cuda.synchronize()
            got = wl["state"]["cur"].cpu().numpy()
            exact = bool(np.ascontiguousarray(got).tobytes() == np.ascontiguousarray(host).tobytes())
            out["cpu_baseline"] = {
                "value": round(squarings * ops / cpu_s / 1e9, 2), "unit": "GOPS", "cores": threads, "kind": "port",
                "sample": f"{squarings} repeated squarings of the same {n}x{n} input (M=N=K={n} each), "
                          f"{cpu_s:.2f} s wall on {threads} OpenMP threads",
                "gpu_final_matrix_bit_exact_vs_oracle": exact,
            }
        elif args.workload == "apsp_blocked":
            # the oracle's blocked iteration on a smaller graph of the same kind (the CPU needs
            # minutes at full size); the GPU runs that graph too and must match it bit for bit
            nc = min(n, 2048)
            Dc = inputs.graph_distances(2024, nc, density=0.10, lo=1.0, hi=100.0)
            if wl["dtype"] == "f64":
                Dc = Dc.astype(np.float64)
            hd, hp = Dc.copy(order="F"), np.full((nc, nc), -1, dtype=np.int32, order="F")   # (a copy: the oracle works in place)
            t1 = time.perf_counter()
            oracle.apsp_blocked(hd, hp, 128)
            cpu_s = time.perf_counter() - t1
            gd = torch.from_numpy(np.ascontiguousarray(Dc.T)).to("cuda:0").t()
            gp = torch.full((nc, nc), -1, dtype=torch.int32, device="cuda:0").t()
            gws = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(nc, wl["dtype"]), dtype=torch.uint8, device="cuda:0")
            cuasr_amd.apsp_blocked(gd, gp, gws)
            torch.cuda.synchronize()
            exact = bool(np.ascontiguousarray(gd.cpu().numpy()).tobytes() == np.ascontiguousarray(hd).tobytes()
                         and (gp.cpu().numpy() == hp).all())
            out["cpu_baseline"] = {
                "value": round(2.0 * nc ** 3 / cpu_s / 1e9, 2), "unit": "GOPS", "cores": threads, "kind": "port",
                "sample": f"the same job at n={nc} ({cpu_s:.2f} s wall on {threads} OpenMP threads)",
                "gpu_dist_and_parent_bit_exact_vs_oracle": exact,
            }
        elif args.workload == "fwgemm":
            D0, fw = wl["host"][0], wl["fw"]
            rows = int(min(n, max(32, 0.5e11 / (2.0 * n * k))))  # the literal scan runs at a few GOPS
            hd, hp = np.asfortranarray(D0[:rows]), np.full((rows, n), -1, dtype=np.int32, order="F")
            t1 = time.perf_counter()
            oracle.fwgemm(np.asfortranarray(D0[:rows]), D0, hd, hp)
            cpu_s = time.perf_counter() - t1
            wl["reset"]()
            step(1)  # one squaring from the initial graph (index 1: no restart)
            torch.cuda.synchronize()
            gd, gp = fw["dist"].cpu().numpy()[:rows], fw["parent"].cpu().numpy()[:rows]
            exact = bool(np.ascontiguousarray(gd).tobytes() == np.ascontiguousarray(hd).tobytes() and (gp == hp).all())
            out["cpu_baseline"] = {
                "value": round(2.0 * rows * n * k / cpu_s / 1e9, 2), "unit": "GOPS", "cores": threads, "kind": "port",
                "sample": f"the first {rows} rows of the first squaring ({rows} x {n} x {k}), {cpu_s:.2f} s wall on "
                          f"{threads} OpenMP threads",
                "gpu_rows_bit_exact_vs_oracle": exact,
            }
        else:
            add, mult, A, B, C, alpha, beta, ident = wl["host"]
            rows = int(min(m, max(32, 1.0e12 / (2.0 * n * k))))
            sub = lambda X: np.ascontiguousarray(X[:rows]) if X.flags.c_contiguous else np.asfortranarray(X[:rows])
            As, Cs = sub(A), sub(C)
            t1 = time.perf_counter()
            oracle.srgemm(add, mult, As, B, Cs, alpha, beta, ident)
            cpu_s = time.perf_counter() - t1
            out["cpu_baseline"] = {
                "value": round(2.0 * rows * n * k / cpu_s / 1e9, 2), "unit": "GOPS", "cores": threads, "kind": "port",
                "sample": f"the first {rows} rows of the output ({rows} x {n} x {k}), {cpu_s:.2f} s wall on "
                          f"{threads} OpenMP threads",
            }
    if args.workload == "apsp" and not args.size and not args.no_extra and args.kernel == "auto":
        import oracle
        del wl
        torch.cuda.empty_cache()
        out["extra"] = {"configs": extra_configs(np, torch, cuasr_amd, inputs, oracle, args),
                        "note": "the other BASELINE configs at full size, same process, mean launch time by HIP events; "
                                "frac = tops / peak of the element type's vector (valu) or matrix (mfma) unit"}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
