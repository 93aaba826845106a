"""Build liboptimus_mi355x.so (the C-ABI library) with hipcc for gfx950.

    python optimus-lm_amd/build.py

Cross-compiles without a GPU.  The library has no dependency on PyTorch: it exports plain
extern "C" functions over device pointers (see include/optimus_mi355x.h).
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "liboptimus_mi355x.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # scalar fp32 arithmetic only: no packed-fp32 instruction selection
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def lib_path():
    return os.path.join(LIBDIR, LIBNAME)


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = []
    procs = []
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    for s in srcs:
        o = os.path.join(objdir, os.path.basename(s)[:-4] + ".o")
        objs.append(o)
        cmd = [hipcc] + compile_flags + ["-c", s, "-o", o]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for s, p in procs:
        out, _ = p.communicate()
        # hipcc's host pass does not know the device-only target feature; that warning is noise
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            print(f"[build] FAILED {s}\n{out}", file=sys.stderr)
        elif verbose and out:
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path()] + objs
    subprocess.run(cmd, check=True)
    return lib_path()


if __name__ == "__main__":
    print(build(verbose=True))
