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

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "ema_*.npz")))
GOLDEN_SSD = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "ssd_*.npz")))
GOLDEN_SEQ = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "emaseq_*.npz")))


def load(path):
    z = np.load(path)  # allow_pickle stays False
    t = {k: torch.from_numpy(z[k]) for k in ("A", "X", "dy", "y", "dx", "dA")}
    return t, int(z["chunk_size"]), bool(z["bf16"])


def test_fixture_files_present():
    assert len(GOLDEN) == 5 and len(GOLDEN_SSD) == 2 and len(GOLDEN_SEQ) == 1


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


# ---- Mamba-2 SSD and the sequence-level EMA forms (tests/golden/make_golden_ssd.py)


def _load_all(path):
    z = np.load(path)
    return {k: torch.from_numpy(z[k]) for k in z.files}


@pytest.mark.parametrize("path", GOLDEN_SSD, ids=lambda p: os.path.basename(p)[:-4])
def test_ssd_oracle_reproduces_golden(path):
    from oracle import ssd_oracle as S

    t = _load_all(path)
    Q = int(t["chunk_size"])
    y, fin = S.ssd_loop(t["x"], t["dt"], t["A"], t["B"], t["C"], t["D"], t["z"], t["init"])
    check_close("ssd_loop y", y, t["y"], torch.float32)
    check_close("ssd_loop final", fin, t["final"], torch.float32)
    y, fin = S.combined_fwd(t["x"], t["dt"], t["A"], t["B"], t["C"], Q, D=t["D"], z=t["z"], initial_states=t["init"])
    check_close("combined_fwd y", y, t["y"], torch.float32)
    check_close("combined_fwd final", fin, t["final"], torch.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN_SSD, ids=lambda p: os.path.basename(p)[:-4])
def test_ssd_hip_reproduces_golden(path, device):
    from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

    t = {k: v.to(device) for k, v in _load_all(path).items()}
    announce(f"golden {os.path.basename(path)}")
    y, fin = mamba_chunk_scan_combined_fwd(t["x"], t["dt"], t["A"], t["B"], t["C"], int(t["chunk_size"]), D=t["D"],
                                           z=t["z"], initial_states=t["init"], return_final_states=True)
    check_close("y", y, t["y"], torch.float32)
    check_close("final states", fin, t["final"], torch.float32)


@pytest.mark.parametrize("path", GOLDEN_SEQ, ids=lambda p: os.path.basename(p)[:-4])
def test_seq_oracle_reproduces_golden(path):
    t = _load_all(path)
    b, L, nh, d = t["x"].shape
    xf, pf = orc.to_flat(t["x"], t["p"])
    dzf, _ = orc.to_flat(t["dz"], t["p"])
    init, dfin = t["init"].reshape(b * nh, d), t["dfinal"].reshape(b * nh, d)
    z, fin = orc.ema_seq_loop(xf, pf, "probability", init)
    dx, dp, dinit = orc.ema_seq_loop_bwd(dzf, xf, pf, "probability", init, dfin)
    check_close("z", orc.from_flat(z, b, nh), t["z"], torch.float32)
    check_close("final", fin.reshape(b, nh, d), t["final"], torch.float32)
    check_close("dx", orc.from_flat(dx, b, nh), t["dx"], torch.float32)
    check_close("dp", dp.reshape(b, nh, L).permute(0, 2, 1), t["dp"], torch.float32)
    check_close("dinit", dinit.reshape(b, nh, d), t["dinit"], torch.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN_SEQ, ids=lambda p: os.path.basename(p)[:-4])
def test_seq_hip_reproduces_golden(path, device):
    from kernels.ema_seq import ema_seq_scan

    t = {k: v.to(device) for k, v in _load_all(path).items()}
    announce(f"golden {os.path.basename(path)}")
    x, p, init = (t[k].clone().requires_grad_() for k in ("x", "p", "init"))
    z, fin = ema_seq_scan(p, x, "probability", initial_states=init, return_final_states=True)
    ((z * t["dz"]).sum() + (fin * t["dfinal"]).sum()).backward()
    check_close("z", z, t["z"], torch.float32)
    check_close("final", fin, t["final"], torch.float32)
    check_close("dx", x.grad, t["dx"], torch.float32)
    check_close("dp", p.grad, t["dp"], torch.float32)
    check_close("dinit", init.grad, t["dinit"], torch.float32)
