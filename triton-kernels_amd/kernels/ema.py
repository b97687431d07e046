"""Probability-space entry point of the reference's first EMA implementation.

Mirrors the signature of ema_scan_combined, kernels/ema.py:370-375 of the reference: that
file's three sequential Triton kernels are replaced by the chunked-scan path, reached by the
change of variables A = log(1 - p), X = p * x (kernels/benchmarks/ema_bench.py:135-136)."""
import torch

from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

DEFAULT_CHUNK = 128


def ema_scan_combined(x, p):
    """z_t = (1 - p_t) * z_{t-1} + p_t * x_t with z_{-1} = 0.

    x: (B, L, D) float32 or bfloat16; p: (B, L, 1) in [0, 1).  Differentiable in x and p."""
    assert x.dim() == 3 and p.shape == (x.shape[0], x.shape[1], 1)
    assert x.is_contiguous()
    assert p.is_contiguous()
    pf = p.float()
    A = torch.log1p(-pf).squeeze(-1)
    X = (pf * x.float()).to(x.dtype) if x.dtype != torch.float32 else pf * x
    return ema_matmul_scan_combined(A, X, DEFAULT_CHUNK)
