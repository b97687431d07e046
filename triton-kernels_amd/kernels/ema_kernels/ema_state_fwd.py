"""F2, chunk-end states as a decay-weighted reduction over each chunk.

Mirrors kernels/ema_kernels/ema_state_fwd.py:130-163 of the reference."""
import math

import torch

from kernels import _lib


def _ema_chunk_state_fwd(x, A_cumsum, seq_idx=None, states=None, states_in_fp32=True):
    """x: (B, L, T) or (b, L, nh, d); A_cumsum: (N, nchunks, chunk_size) -> states (N, nchunks, T).

    The kernels keep chunk states in float32; with states_in_fp32=False the result is cast
    to x.dtype afterwards."""
    if seq_idx is not None:
        raise NotImplementedError("seq_idx is not supported by the EMA kernels")
    dev = _lib.require_gpu(x, A_cumsum)
    x, x_args, batch, nh, seqlen, token_dim = _lib.seq_view(x)
    _, nchunks_cs, chunk_size = A_cumsum.shape
    nchunks = math.ceil(seqlen / chunk_size)
    assert A_cumsum.is_contiguous()
    assert A_cumsum.shape == (batch * nh, nchunks, chunk_size)
    out = None
    if states is not None:
        assert states.shape == (batch * nh, nchunks, token_dim)
        if states.dtype == torch.float32 and states.is_contiguous():
            out = states
    if out is None:
        out = torch.empty((batch * nh, nchunks, token_dim), device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_chunk_state_fwd(
            *x_args, _lib.dtype_code(x), A_cumsum.data_ptr(), out.data_ptr(),
            batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_chunk_state_fwd")
    if states is not None and out is not states:
        states.copy_(out)
        return states
    return out if states_in_fp32 else out.to(x.dtype)
