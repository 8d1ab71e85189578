"""Builds cuasr_amd/lib/libcuasr_amd.so for gfx950 with hipcc (cross-compiles
without a GPU).  Usage: ``python -m cuasr_amd.build [-j N]``."""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libcuasr_amd.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# packed-fp32 code generation is switched off for every device object
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


# the vector-ALU tiles may assume NaN-free data: it lets min/max map to single
# (3-input) instructions without re-canonicalising every accumulator
PER_FILE = {"valu_": ["-fno-honor-nans"], "mfma_f32": ["-fno-honor-nans"], "direct_": ["-fno-honor-nans"],
            "fwgemm": ["-fno-honor-nans"]}


def _compile(src):
    obj = os.path.join(OBJ, src[:-4] + ".o")
    extra = [f for k, v in PER_FILE.items() if src.startswith(k) for f in v]
    cmd = [HIPCC] + FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return obj, err


def generate():
    """The hand-scheduled main loops of the direct-to-LDS tile: asm text written by csrc/gen_direct_asm.py."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_direct_asm", os.path.join(CSRC, "gen_direct_asm.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.generate(os.path.join(CSRC, "gen")) + mod.generate_mfma(os.path.join(CSRC, "gen")) + mod.generate_mfma64(os.path.join(CSRC, "gen")) + mod.generate_narrow(os.path.join(CSRC, "gen")) + mod.generate_fwgemm_merge(os.path.join(CSRC, "gen"))


def build(jobs=None, verbose=True):
    generate()
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        results = list(ex.map(_compile, sources()))
    for obj, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    objs = [o for o, _ in results]
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


def build_functor_bench():
    """cuasr_amd/functor_bench.hip -> cuasr_amd/lib/functor_bench: the throughput of kernels built from user functors
    (what `bench.py --workload functor` runs), compiled the way a user's translation unit is."""
    root = os.path.dirname(HERE)
    out = os.path.join(LIB_DIR, "functor_bench")
    cmd = [HIPCC] + [f for f in FLAGS if f != "-fPIC"] + ["-I", os.path.join(root, "include"), os.path.join(HERE, "functor_bench.hip"),
                                                          "-L", LIB_DIR, "-lcuasr_amd", "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath,$ORIGIN", "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on functor_bench.hip:\n" + r.stderr[-4000:])
    return out


if __name__ == "__main__":
    j = int(sys.argv[sys.argv.index("-j") + 1]) if "-j" in sys.argv else None
    print(build(j))
    print(build_functor_bench())
