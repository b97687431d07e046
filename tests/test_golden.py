"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from a float64
numpy evaluation of the definition): the oracle against them on the CPU, and the HIP
library against them on the GPU."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import ema_oracle as orc
from parity_util import announce, check_close

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def load(path):
    z = np.load(path)  # allow_pickle stays False
    t = {k: torch.from_numpy(z[k]) for k in ("A", "X", "dy", "y", "dx", "dA")}
    return t, int(z["chunk_size"]), bool(z["bf16"])


def test_fixture_files_present():
    assert len(GOLDEN) == 5


@pytest.mark.parametrize("path", GOLDEN, ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_reproduces_golden(path):
    """The float32 oracle (sequential and chunked) against the float64 vectors."""
    t, Q, _ = load(path)
    b, L, nh, d = t["X"].shape
    Xf, Af = orc.to_flat(t["X"], t["A"])
    dyf, _ = orc.to_flat(t["dy"], t["A"])
    y_ref, _ = orc.to_flat(t["y"], t["A"])
    dx_ref, _ = orc.to_flat(t["dx"], t["A"])
    dA_ref = t["dA"].permute(0, 2, 1).reshape(b * nh, L)
    check_close("ema_loop", orc.ema_loop(Xf, Af), y_ref, torch.float32)
    y, *_ = orc.combined_fwd(Af, Xf, Q)
    check_close("combined_fwd", y, y_ref, torch.float32)
    dx, ddA = orc.combined_bwd(dyf, Xf, Af, Q)
    check_close("combined_bwd dx", dx, dx_ref, torch.float32)
    check_close("combined_bwd dA", ddA.reshape(b * nh, -1)[:, :L], dA_ref, torch.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=lambda p: os.path.basename(p)[:-4])
def test_hip_reproduces_golden(path, device):
    """The autograd entry point, headed layout, against the float64 vectors."""
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    t, Q, bf16 = load(path)
    dtype = torch.bfloat16 if bf16 else torch.float32
    announce(f"golden {os.path.basename(path)} chunk={Q} {dtype}")
    A = t["A"].to(device).requires_grad_(True)
    X = t["X"].to(device, dtype).requires_grad_(True)
    y = ema_matmul_scan_combined(A, X, Q)
    y.backward(t["dy"].to(device, dtype))
    check_close("y", y, t["y"], dtype)
    check_close("dx", X.grad, t["dx"], dtype)
    check_close("dA", A.grad, t["dA"], dtype)
