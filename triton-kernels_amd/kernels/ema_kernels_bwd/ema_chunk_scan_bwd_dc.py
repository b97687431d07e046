"""B5, log-decay gradient through the carried-state term of the chunk scan.

Mirrors kernels/ema_kernels_bwd/ema_chunk_scan_bwd_dc.py:115-147 of the reference."""
import torch

from kernels import _lib


def _ema_chunk_scan_bwd_dC(prev_states, dA_cumsum, dout, seq_idx=None, C=None, ngroups=1):
    """prev_states: (N, C, T); dA_cumsum: (N, C, Q); dout: (B, L, T) or (b, L, nh, d)
    -> ddA_cumsum (N, C, Q) with s[m] = exp(cs[m]) * <dout[m], prev>, before any cumsum."""
    if seq_idx is not None or C is not None:
        raise NotImplementedError("seq_idx and C are not supported by the EMA kernels")
    dev = _lib.require_gpu(prev_states, dA_cumsum, dout)
    dout, d_args, batch, nh, seqlen, token_dim = _lib.seq_view(dout)
    _, nchunks, chunk_size = dA_cumsum.shape
    assert prev_states.shape == (batch * nh, nchunks, token_dim)
    assert dA_cumsum.shape[0] == batch * nh and nchunks == -(-seqlen // chunk_size)
    cs = _lib.f32c(dA_cumsum)
    prev = _lib.f32c(prev_states)
    ddA_cumsum = torch.empty(batch * nh, nchunks, chunk_size, device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_chunk_scan_bwd_dc(
            *d_args, _lib.dtype_code(dout), prev.data_ptr(), cs.data_ptr(), ddA_cumsum.data_ptr(),
            batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_chunk_scan_bwd_dC")
    return ddA_cumsum
