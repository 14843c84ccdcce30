"""Compile libqtip_hip.so for gfx950 in-tree:  python -m qtip_amd.build"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRCS = [os.path.join(HERE, "csrc", f) for f in ("qtip_hip.hip", "qtip_rht.hip", "qtip_decoder.hip", "qtip_pack.hip")]
OUT = os.path.join(HERE, "libqtip_hip.so")

# packed fp32 VALU forms are switched off for every HIP translation unit
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + SRCS + ["-o", OUT + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    os.replace(OUT + ".tmp", OUT)
    return OUT


if __name__ == "__main__":
    build()
