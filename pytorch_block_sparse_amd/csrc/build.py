"""Compile libpbs_hip.so (the C-ABI HIP library) for gfx950 next to its sources.

Also libpbs_hip_check.so: the same library with the conservative progress protocol of the two barrier-free bf16
kernels (-DPBS_DDS16_PUBLISH_AFTER_WAIT -DPBS_DDSC_PUBLISH_AFTER_WAIT).  Only tests/test_gpu_wide_protocol.py loads it, to compare the two bit for bit.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libpbs_hip.so")
CHECK_LIB = os.path.join(HERE, "libpbs_hip_check.so")


def build(verbose=True):
    _compile(LIB, [], verbose)
    _compile(CHECK_LIB, ["-DPBS_DDS16_PUBLISH_AFTER_WAIT", "-DPBS_DDSC_PUBLISH_AFTER_WAIT"], verbose)
    return LIB


def _compile(lib, defines, verbose):
    cmd = [
        os.environ.get("HIPCC", "hipcc"),
        "-O3",
        "-std=c++17",
        "--offload-arch=gfx950",
        "-fPIC",
        "-shared",
        "-Xclang",
        "-target-feature",
        "-Xclang",
        "-packed-fp32-ops",
        *defines,
        "-o",
        lib,
        os.path.join(HERE, "pbs_hip.hip"),
    ]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, cwd=HERE, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass prints one harmless "not a recognized feature" line per compile step
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip() and verbose:
        print(out)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout)
    return lib


if __name__ == "__main__":
    build()
    sys.exit(0)
