"""Compiles the HIP sources under csrc/ into liblten_hip.so (gfx950 only), in-tree, and the calibration kernels
under measure/ into a library of their own, liblten_hip_measure.so (used by bench.py and the profile commands only).

Usage: python light-tensor_amd/build.py [--verbose]
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblten_hip.so")
MEASURE_SRC = os.path.join(HERE, "measure", "measure.hip")
MEASURE_LIB = os.path.join(HERE, "liblten_hip_measure.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed fp32 instruction selection is switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no implicit fused multiply-add: the requantize step of the int8 path is an unfused multiply
    # then add, and the fp32 kernels ask for fma explicitly where they want it
    "-ffp-contract=off",
    "-Wno-unused-result",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose=False, extra_flags=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in sources():
        obj = os.path.join(CSRC, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc] + [f for f in HIPCC_FLAGS if f != "-shared"] + list(extra_flags) + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l or "error" in l]
        if p.returncode != 0:
            failed = True
            print("\n".join(lines), file=sys.stderr)
        elif verbose and lines:
            print("\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    cmd = [hipcc] + HIPCC_FLAGS + [MEASURE_SRC, "-o", MEASURE_LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        print(r.stdout, file=sys.stderr)
        raise RuntimeError("hipcc failed")
    return LIB


if __name__ == "__main__":
    print(build(verbose="--verbose" in sys.argv))
