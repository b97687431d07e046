"""B4, log-decay gradient through the chunk-local states.

Mirrors kernels/ema_kernels_bwd/ema_chunk_state_bwd_db.py:122-152 of the reference; the
cumulative sum the reference runs with torch.cumsum afterwards happens inside the kernel."""
import torch

from kernels import _lib


def _ema_chunk_state_bwd_db(x, dA_cumsum, dstates, seq_idx=None, B=None, ngroups=1, raw_scale_gradient=False):
    """x: (B, L, T) or (b, L, nh, d); dA_cumsum: (N, C, Q); dstates: (N, C, T)
    -> ddA_cumsum (N, C, Q): slot m+1 holds the contribution of row m (slot 0 is 0), summed
    cumulatively along the chunk unless raw_scale_gradient."""
    if seq_idx is not None or B is not None:
        raise NotImplementedError("seq_idx and B are not supported by the EMA kernels")
    dev = _lib.require_gpu(x, dA_cumsum, dstates)
    x, x_args, batch, nh, seqlen, token_dim = _lib.seq_view(x)
    _, nchunks, chunk_size = dA_cumsum.shape
    assert dstates.shape == (batch * nh, nchunks, token_dim)
    assert dA_cumsum.shape[0] == batch * nh and nchunks == -(-seqlen // chunk_size)
    cs = _lib.f32c(dA_cumsum)
    g = _lib.f32c(dstates)
    ddA_cumsum = torch.empty(batch * nh, nchunks, chunk_size, device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_chunk_state_bwd_db(
            *x_args, _lib.dtype_code(x), cs.data_ptr(), g.data_ptr(), ddA_cumsum.data_ptr(),
            1 if raw_scale_gradient else 0, batch, nh, seqlen, token_dim, chunk_size,
            _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_chunk_state_bwd_db")
    return ddA_cumsum
