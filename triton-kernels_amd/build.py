"""Builds lib/libema_hip.so (gfx950) from csrc/ with hipcc: the EMA scan (ema_abi.hip) and the
SSD forward stages (ssd_abi.hip).  Usage: python build.py"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = [os.path.join(HERE, "csrc", "ema_abi.hip"), os.path.join(HERE, "csrc", "ssd_abi.hip")]
OUT = os.path.join(HERE, "lib", "libema_hip.so")

FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-shared",
    "-fPIC",
    # packed FP32 VALU ops are kept off for every HIP translation unit of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose: bool = True) -> str:
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-o", OUT] + SRC
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(
        l for l in res.stderr.splitlines() if "is not a recognized feature for this target" not in l
    )
    if res.returncode != 0:
        sys.stderr.write(err + "\n")
        raise RuntimeError("hipcc failed")
    if verbose and err.strip():
        print(err)
    return OUT


if __name__ == "__main__":
    build()
