"""Whole backward of the EMA chunked scan.

Mirrors kernels/ema_kernels_bwd/ema_combined_bwd.py:13-83 of the reference."""
import math

import torch

from kernels import _lib


def _ema_chunk_scan_combined_bwd(dout, x, A, chunk_size, dt_limit=(0.0, float("inf")), recompute_output=False,
                                 prev128=None, kernel_events=None):
    """dout, x: (B, L, T) or (b, L, nh, d); A: (B, L) or (b, L, nh) float32.  prev128
    (optional) is the fifth return value of _ema_matmul_scan_combined_fwd(...,
    return_prev128=True); with it the backward does not re-read x to rebuild it.
    kernel_events: optional (start, stop) torch.cuda.Event pair recorded around the
    single-pass kernel.

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
    if prev128 is not None:
        assert prev128.shape == (N, math.ceil(seqlen / 128), token_dim)
        assert prev128.dtype == torch.float32 and prev128.is_contiguous()
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
    ws, ready = _lib.workspace(dev, ws_bytes, batch, nh, seqlen, token_dim)
    with torch.cuda.device(dev):
        st = L.ema_bwd(
            *d_args, *x_args, *a_args, None if prev128 is None else prev128.data_ptr(),
            _lib.dtype_code(x), *dx_args, ddA.data_ptr(), *y_args,
            ws.data_ptr(), ws.numel(), ready, batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
            *_lib.event_ptrs(kernel_events),
        )
    _lib.check(st, "_ema_chunk_scan_combined_bwd")
    return (dx, ddA) if not recompute_output else (dx, ddA, y)


def _ema_bwd_dx_dA_fused(x, dA_cumsum, dout, prev_states, dstates, recompute_output=False):
    """One pass over x and dout for a chunk size of 128: dx and the complete log-decay
    gradient (what the reference assembles from its dx, db, dC and ddAcs launchers,
    kernels/ema_kernels_bwd/ema_combined_bwd.py:70-79).

    x, dout: (B, L, T) or (b, L, nh, d); dA_cumsum: (N, C, 128); prev_states, dstates:
    (N, C, T).  Returns (dx, ddA (N, C, 128)[, y])."""
    dev = _lib.require_gpu(x, dA_cumsum, dout, prev_states, dstates)
    x, x_args, batch, nh, seqlen, token_dim = _lib.seq_view(x)
    dout, d_args, *_ = _lib.seq_view(dout)
    N = batch * nh
    nchunks = math.ceil(seqlen / 128)
    assert dout.shape == x.shape and dout.dtype == x.dtype
    assert dA_cumsum.shape == (N, nchunks, 128), "this kernel works on chunks of 128 rows"
    assert prev_states.shape == (N, nchunks, token_dim)
    assert dstates.shape == (N, nchunks, token_dim)
    cs, prev, g = _lib.f32c(dA_cumsum), _lib.f32c(prev_states), _lib.f32c(dstates)
    dx = torch.empty(x.shape, device=dev, dtype=x.dtype)
    _, dx_args, *_ = _lib.seq_view(dx)
    ddA = torch.empty(N, nchunks, 128, device=dev, dtype=torch.float32)
    if recompute_output:
        y = torch.empty(x.shape, device=dev, dtype=x.dtype)
        _, y_args, *_ = _lib.seq_view(y)
    else:
        y, y_args = None, [None, 0, 0, 0]
    L = _lib.lib()
    ws_bytes = L.ema_bwd_dx_dA_fused_workspace_bytes(batch, nh, seqlen, token_dim)
    assert ws_bytes > 0, "unsupported shape"
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        st = L.ema_bwd_dx_dA_fused(
            *x_args, *d_args, _lib.dtype_code(x), cs.data_ptr(), prev.data_ptr(), g.data_ptr(),
            *dx_args, ddA.data_ptr(), *y_args, ws.data_ptr(), ws_bytes, batch, nh, seqlen,
            token_dim, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_bwd_dx_dA_fused")
    return (dx, ddA) if not recompute_output else (dx, ddA, y)
