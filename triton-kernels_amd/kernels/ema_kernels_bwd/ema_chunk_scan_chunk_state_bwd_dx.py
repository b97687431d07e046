"""B3, gradient of the input: the transposed intra-chunk contraction on MFMA plus the
carried state gradient.

Mirrors kernels/ema_kernels_bwd/ema_chunk_scan_chunk_state_bwd_dx.py:208-262 of the
reference."""
import torch

from kernels import _lib


def _chunk_scan_chunk_state_bwd_dx(x, dA_cumsum, dout, dstates, D=None, seq_idx=None, dx=None):
    """x, dout: (B, L, T) or (b, L, nh, d); dA_cumsum: (N, C, Q); dstates: (N, C, T) -> dx."""
    if D is not None or seq_idx is not None:
        raise NotImplementedError("D and seq_idx are not supported by the EMA kernels")
    dev = _lib.require_gpu(x, dA_cumsum, dout, dstates)
    dout, d_args, batch, nh, seqlen, token_dim = _lib.seq_view(dout)
    _, nchunks, chunk_size = dA_cumsum.shape
    assert dstates.shape == (batch * nh, nchunks, token_dim)
    assert dout.shape == x.shape
    assert dA_cumsum.shape[0] == batch * nh and nchunks == -(-seqlen // chunk_size)
    user_dx = dx
    if dx is None or dx.dtype != dout.dtype or dx.stride(-1) != 1:
        dx = torch.empty(dout.shape, device=dev, dtype=dout.dtype)
    assert dx.shape == x.shape
    _, dx_args, *_ = _lib.seq_view(dx)
    cs = _lib.f32c(dA_cumsum)
    g = _lib.f32c(dstates)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_chunk_scan_chunk_state_bwd_dx(
            *d_args, _lib.dtype_code(dout), cs.data_ptr(), g.data_ptr(), *dx_args,
            batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_chunk_scan_chunk_state_bwd_dx")
    if user_dx is not None and user_dx is not dx:
        user_dx.copy_(dx)
        return user_dx
    return dx
