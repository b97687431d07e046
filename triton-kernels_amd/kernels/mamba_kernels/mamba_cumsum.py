"""SSD stage 1: processed dt and the per-chunk cumsum of dt * A.

Mirrors _chunk_cumsum_fwd, kernels/mamba_kernels/mamba_cumsum.py:103-128 of the reference
(same positional signature, same return order); the Triton kernel is replaced by
ssd_chunk_cumsum_fwd of libema_hip.so."""
import math

import torch

from kernels import _lib


def _chunk_cumsum_fwd(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    batch, seqlen, nheads = dt.shape
    assert A.shape == (nheads,)
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
    dev = _lib.require_gpu(dt, A)
    if dt.dtype not in (torch.float32, torch.bfloat16):
        dt = dt.float()
    nchunks = math.ceil(seqlen / chunk_size)
    dt_out = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    dA_cumsum = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    Af = _lib.f32c(A)
    bias = None if dt_bias is None else _lib.f32c(dt_bias)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_cumsum_fwd(
                dt.data_ptr(), _lib.dtype_code(dt), dt.stride(0), dt.stride(1), dt.stride(2), Af.data_ptr(),
                None if bias is None else bias.data_ptr(), dA_cumsum.data_ptr(), dt_out.data_ptr(), batch, seqlen,
                nheads, chunk_size, int(bool(dt_softplus)), float(dt_limit[0]),
                float(min(dt_limit[1], 3.0e38)), _lib.stream_ptr(dev)),
            "ssd_chunk_cumsum_fwd")
    return dA_cumsum, dt_out
