"""Probability-space entry point of the reference's first EMA implementation.

Mirrors the signature of ema_scan_combined, kernels/ema.py:370-375 of the reference: that
file's three sequential Triton kernels are replaced by the chunked-scan path, reached by the
change of variables A = log(1 - p), X = p * x (kernels/benchmarks/ema_bench.py:135-136)."""
import torch

from kernels.ema_seq import ema_seq_scan


def ema_scan_combined(x, p):
    """z_t = (1 - p_t) * z_{t-1} + p_t * x_t with z_{-1} = 0, in one pass over x.

    x: (B, L, D) float32 or bfloat16; p: (B, L, 1) in [0, 1].  Differentiable in x and p (the
    reference's backward returns None, kernels/ema.py:366-367)."""
    assert x.dim() == 3 and p.shape == (x.shape[0], x.shape[1], 1)
    assert x.is_contiguous()
    assert p.is_contiguous()
    return ema_seq_scan(p.float().squeeze(-1), x, form="probability")
