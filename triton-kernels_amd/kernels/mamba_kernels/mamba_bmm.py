"""SSD stage 4: C B^T per chunk and group.

Mirrors _bmm_chunk_fwd, kernels/mamba_kernels/mamba_bmm.py:80-126 of the reference.  The whole
chunk_size x chunk_size block is computed also with causal=True (the reference then leaves the
strictly upper tiles unwritten)."""
import math

import torch

from kernels import _lib
from kernels.mamba_kernels._shapes import Plan


def _bmm_chunk_fwd(a, b, chunk_size, seq_idx=None, causal=False, output_dtype=None):
    has_groups = a.dim() == 4
    if not has_groups:
        batch, seqlen, k = a.shape
        a4, b4 = a.unsqueeze(2), b.unsqueeze(2)
        ngroups = 1
    else:
        batch, seqlen, ngroups, k = a.shape
        a4, b4 = a, b
    assert b.shape == a.shape
    plan = Plan(64, k)
    if plan.N != k:  # a short contraction axis is padded with zeros
        return _bmm_chunk_fwd(plan.bc(a), plan.bc(b), chunk_size, seq_idx=seq_idx, causal=causal,
                              output_dtype=a.dtype if output_dtype is None else output_dtype)
    dev = _lib.require_gpu(a, b)
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    if b4.dtype != a4.dtype:
        b4 = b4.to(a4.dtype)
    a4, sa = _lib.strided4(a4)
    b4, sb = _lib.strided4(b4)
    nchunks = math.ceil(seqlen / chunk_size)
    out_dtype = a.dtype if output_dtype is None else output_dtype
    kernel_out = torch.float32 if out_dtype != a4.dtype else out_dtype
    out = torch.empty(batch, nchunks, ngroups, chunk_size, chunk_size, device=dev, dtype=kernel_out)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_bmm_chunk_fwd(*sa, *sb, _lib.dtype_code(a4), out.data_ptr(), _lib.dtype_code(out), batch,
                                         seqlen, ngroups, k, chunk_size, *ids, _lib.stream_ptr(dev)),
            "ssd_bmm_chunk_fwd")
    if out.dtype != out_dtype:
        out = out.to(out_dtype)
    return out if has_groups else out.squeeze(2)
