"""F1, per-chunk cumulative sum of the log-decay.

Mirrors kernels/ema_kernels/ema_cumsum.py:66-80 of the reference."""
import math

import torch

from kernels import _lib


def ema_chunk_cumsum_fwd(A: torch.Tensor, chunk_size: int):
    """A: (B, L) or (b, L, nh) float32 -> dA_cumsum (N, nchunks, chunk_size) float32."""
    dev = _lib.require_gpu(A)
    a_args, batch, nh, seqlen = _lib.decay_view(A)
    nchunks = math.ceil(seqlen / chunk_size)
    dA_cumsum = torch.empty(batch * nh, nchunks, chunk_size, device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_chunk_cumsum_fwd(
            *a_args, dA_cumsum.data_ptr(), batch, nh, seqlen, chunk_size, _lib.stream_ptr(dev)
        )
    _lib.check(st, "ema_chunk_cumsum_fwd")
    return dA_cumsum
