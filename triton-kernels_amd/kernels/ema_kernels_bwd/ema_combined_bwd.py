"""Whole backward of the EMA chunked scan.

Mirrors kernels/ema_kernels_bwd/ema_combined_bwd.py:13-83 of the reference."""
import math

import torch

from kernels import _lib


def _ema_chunk_scan_combined_bwd(dout, x, A, chunk_size, dt_limit=(0.0, float("inf")), recompute_output=False):
    """dout, x: (B, L, T) or (b, L, nh, d); A: (B, L) or (b, L, nh) float32.

    Returns (dx, ddA) with ddA (N, nchunks, chunk_size) float32, ddA[n, c, q] = dL/dA at
    position c * chunk_size + q of sequence n; with recompute_output also the forward
    output."""
    dev = _lib.require_gpu(dout, x, A)
    x, x_args, batch, nh, seqlen, token_dim = _lib.seq_view(x)
    if dout.dtype != x.dtype:
        dout = dout.to(x.dtype)
    dout, d_args, *_ = _lib.seq_view(dout)
    a_args, a_batch, a_nh, a_len = _lib.decay_view(A)
    nchunks = math.ceil(seqlen / chunk_size)
    assert dout.shape == x.shape
    assert (a_batch, a_nh, a_len) == (batch, nh, seqlen)
    N = batch * nh
    dx = torch.empty(x.shape, device=dev, dtype=x.dtype)
    _, dx_args, *_ = _lib.seq_view(dx)
    ddA = torch.empty(N, nchunks, chunk_size, device=dev, dtype=torch.float32)
    if recompute_output:
        y = torch.empty(x.shape, device=dev, dtype=x.dtype)
        _, y_args, *_ = _lib.seq_view(y)
    else:
        y, y_args = None, [None, 0, 0, 0]
    L = _lib.lib()
    ws_bytes = L.ema_bwd_workspace_bytes(batch, nh, seqlen, token_dim, chunk_size)
    assert ws_bytes > 0, "unsupported shape"
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        st = L.ema_bwd(
            *d_args, *x_args, *a_args, _lib.dtype_code(x), *dx_args, ddA.data_ptr(), *y_args,
            ws.data_ptr(), ws_bytes, batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_chunk_scan_combined_bwd")
    return (dx, ddA) if not recompute_output else (dx, ddA, y)
