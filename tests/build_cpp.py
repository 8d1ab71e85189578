"""Builds the C++ test programs under tests/cpp (test infrastructure: they include the checker's headers from
oracle/include, which the library never does).  Usage: ``python tests/build_cpp.py``; ``__graft_entry__.build()``
and the tests that run the programs call ``build_all()`` / ``build(name)``."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CPP = os.path.join(HERE, "cpp")
LIB_DIR = os.path.join(ROOT, "cuasr_amd", "lib")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.environ.get("HIPCC", os.path.join(ROCM, "bin", "hipcc"))
INCLUDES = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "oracle", "include")]
LINK = ["-L", LIB_DIR, "-lcuasr_amd", "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath,$ORIGIN/../../cuasr_amd/lib"]
# what a translation unit that builds kernels from its own functors is compiled with: no contraction of a
# functor's a * b + c into a fused multiply-add (the host reference does not fuse), no packed-fp32 instructions
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]

# name -> (source, compiler); "host" programs are plain C++ (g++), "hip" ones hold device code (hipcc)
PROGRAMS = {
    "test_device_api": ("test_device_api.cpp", "host"),
    "host_splitk_models": ("host_splitk_models.cpp", "host-only"),
    "test_user_functor": ("test_user_functor.hip", "hip"),
    "test_reference_call_sites": ("test_reference_call_sites.hip", "hip"),
}


def path(name):
    return os.path.join(CPP, name)


def build(name):
    src, kind = PROGRAMS[name]
    src, out = os.path.join(CPP, src), path(name)
    if kind == "hip":
        cmd = [HIPCC] + HIP_FLAGS + INCLUDES + [src] + LINK + ["-o", out]
        subprocess.check_call(cmd, stderr=subprocess.DEVNULL)
    else:
        # the operator templates need only the HIP runtime API header
        cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O1", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROCM, "include")]
        cmd += INCLUDES + [src]
        if kind == "host":
            cmd += LINK + ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64"]
        subprocess.check_call(cmd + ["-o", out])
    return out


def build_all():
    return [build(name) for name in PROGRAMS if os.path.exists(os.path.join(CPP, PROGRAMS[name][0]))]


def ensure(name):
    """The program's path, built first if it is not there."""
    return path(name) if os.path.exists(path(name)) else build(name)


if __name__ == "__main__":
    for out in (build_all() if len(sys.argv) < 2 else [build(n) for n in sys.argv[1:]]):
        print(out)
