"""Builds libglades_hip.so (HIP kernels + C ABI) and libglades_host.so (the C++ class API on
top of it) for gfx950, in-tree.  `python glades-ml_amd/build.py` or build_all() from Python."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libglades_hip.so")
HOST_LIB = os.path.join(HERE, "libglades_host.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
             "-Wno-option-ignored", "-Wno-unused-result", "-Wno-inline-asm"]

# Exact mode repeats the reference's fp32 arithmetic operation by operation: a product must be
# rounded before it is added, so nothing in that file may be contracted into a fused multiply-add
# (hipcc contracts by default, across the inlined __fmul_rn / __fadd_rn helpers too).
PER_FILE_FLAGS = {"exact_kernel.hip": ["-ffp-contract=off"]}


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + "\n")
        raise RuntimeError("build failed: " + cmd[-1])
    # the host pass does not know the packed-fp32 feature and says so: harmless
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if "error" in out:
        sys.stderr.write(out + "\n")
    return out


def build_all(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    objs = [os.path.join(OBJ, f[:-4] + ".o") for f in srcs]

    def one(pair):
        src, obj = pair
        return _run([HIPCC] + HIP_FLAGS + PER_FILE_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(6, len(srcs))) as ex:
        outs = list(ex.map(one, zip(srcs, objs)))
    if verbose:
        for o in outs:
            if o:
                print(o)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    host_srcs = sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp")) if os.path.isdir(HOST) else []
    if host_srcs:
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", os.path.join(HERE, "..", "include"),
              "-pthread", "-o", HOST_LIB] + host_srcs + ["-L", HERE, "-lglades_hip", "-Wl,-rpath,$ORIGIN"])
        # driver of the C++ class API used by tests/test_host_api.py (built here, run on the GPU box)
        # CPU checker of the restated float routines against this machine's C library (tests/test_libm_exact.py)
        libm_src = os.path.join(HERE, "..", "tests", "libm_check.cpp")
        if os.path.exists(libm_src):
            os.makedirs(os.path.join(HERE, "..", "tests", "bin"), exist_ok=True)
            _run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-fopenmp", "-o",
                  os.path.join(HERE, "..", "tests", "bin", "libm_check"), libm_src, "-lm"])
        check_src = os.path.join(HERE, "..", "tests", "host_api_check.cpp")
        if os.path.exists(check_src):
            bindir = os.path.join(HERE, "..", "tests", "bin")
            os.makedirs(bindir, exist_ok=True)
            _run(["g++", "-O2", "-std=c++17", "-Wall", "-pthread", "-I", HOST, "-I", os.path.join(HERE, "..", "include"),
                  "-o", os.path.join(bindir, "host_api_check"), check_src, "-L", HERE, "-lglades_host", "-lglades_hip",
                  "-Wl,-rpath,$ORIGIN/../../glades-ml_amd", "-Wl,-rpath-link," + HERE, "-L/opt/rocm/lib", "-Wl,-rpath-link,/opt/rocm/lib"])
    return LIB


if __name__ == "__main__":
    print(build_all(verbose=True))
