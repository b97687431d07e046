"""B1, gradient of the states entering each chunk.

Mirrors kernels/ema_kernels_bwd/ema_scan_bwd.py:132-153 of the reference."""
import torch

from kernels import _lib


def _ema_chunk_scan_bwd_dstates(dA_cumsum, dout, seq_idx=None, dtype=None):
    """dA_cumsum: (N, nchunks, chunk_size); dout: (B, L, T) or (b, L, nh, d)
    -> dprev_states (N, nchunks, T)."""
    if seq_idx is not None:
        raise NotImplementedError("seq_idx is not supported by the EMA kernels")
    dev = _lib.require_gpu(dout, dA_cumsum)
    dout, d_args, batch, nh, seqlen, token_dim = _lib.seq_view(dout)
    _, nchunks, chunk_size = dA_cumsum.shape
    assert dA_cumsum.shape == (batch * nh, nchunks, chunk_size)
    assert nchunks == -(-seqlen // chunk_size)
    dtype = dA_cumsum.dtype if dtype is None else dtype
    cs = _lib.f32c(dA_cumsum)
    ds = torch.empty(batch * nh, nchunks, token_dim, device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_chunk_scan_bwd_dstates(
            *d_args, _lib.dtype_code(dout), cs.data_ptr(), ds.data_ptr(),
            batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_chunk_scan_bwd_dstates")
    return ds if dtype == torch.float32 else ds.to(dtype)
