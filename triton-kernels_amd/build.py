"""Builds lib/libema_hip.so (gfx950) from csrc/ with hipcc: the EMA scan (ema_abi.hip) and the
SSD stages (ssd_abi.hip).  The translation units are compiled side by side and then linked.
Usage: python build.py"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = [os.path.join(HERE, "csrc", "ema_abi.hip"), os.path.join(HERE, "csrc", "ssd_abi.hip")]
OUT = os.path.join(HERE, "lib", "libema_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    # packed FP32 VALU ops are kept off for every HIP translation unit of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(
        l for l in res.stderr.splitlines() if "is not a recognized feature for this target" not in l
    )
    if res.returncode != 0:
        sys.stderr.write(err + "\n")
        raise RuntimeError("hipcc failed: " + " ".join(cmd))
    if verbose and err.strip():
        print(err)


def build(verbose: bool = True, extra_flags=(), out: str = OUT) -> str:
    os.makedirs(os.path.dirname(out), exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    tag = os.path.splitext(os.path.basename(out))[0]
    objs = [os.path.join(OBJ_DIR, tag + "_" + os.path.basename(s) + ".o") for s in SRC]
    with ThreadPoolExecutor(len(SRC)) as pool:
        list(pool.map(lambda so: _run([hipcc] + FLAGS + list(extra_flags) + ["-c", so[0], "-o", so[1]], verbose),
                      zip(SRC, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs, verbose)
    return out


# Development build with per-tile phase timestamps in the single-pass kernels (what
# `bench.py --stage tile_phases` loads); never the library the operators use.
TIMING_OUT = os.path.join(HERE, "lib", "libema_hip_timing.so")


if __name__ == "__main__":
    if "--timing" in sys.argv[1:]:
        build(extra_flags=["-DEMA_TIMING"], out=TIMING_OUT)
    else:
        build()
