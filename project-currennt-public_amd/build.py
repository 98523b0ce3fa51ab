"""Builds libcurrennt_hip.so (gfx950) from csrc/*.hip with hipcc.  Pure build logic, no GPU needed."""
import concurrent.futures as cf
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcurrennt_hip.so")
BIN_DIR = os.path.join(HERE, "bin")
HOST_DRIVER = os.path.join(BIN_DIR, "run_stack")
HOST_DRIVERS = ["run_stack", "run_graph"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


# Per-file additions.  The weight update is specified operation by operation (every product and sum rounded
# on its own, as the reference's host and device code do), so its file is compiled without contraction into
# fused multiply-adds; HIP's __fmul_rn / __fadd_rn are plain operators and do not prevent it.
EXTRA_FLAGS = {"optimizer.hip": ["-ffp-contract=off"]}


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    cmd = [HIPCC] + FLAGS + EXTRA_FLAGS.get(os.path.basename(src), []) + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, r.returncode, r.stdout + r.stderr


def build_library(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = []
    with cf.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        for src, obj, rc, out in ex.map(_compile, srcs):
            filtered = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
            if rc != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
            if verbose and filtered.strip():
                print(filtered)
            objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    build_host_driver()
    return LIB_PATH


def build_host_driver():
    """C++ layer shells (host/layers.hpp) + the drivers that run them, linked against the C-ABI library."""
    os.makedirs(BIN_DIR, exist_ok=True)
    for name in HOST_DRIVERS:
        cmd = [HIPCC, "-O2", "-std=c++17", "-Wall", "-x", "c++", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
               os.path.join(HERE, "host", name + ".cpp"), "-o", os.path.join(BIN_DIR, name), "-L" + LIB_DIR,
               "-lcurrennt_hip", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/../lib", "-Wl,-rpath,/opt/rocm/lib"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("host driver build failed:\n" + r.stdout + r.stderr)
    return HOST_DRIVER


if __name__ == "__main__":
    print(build_library())
