"""F4, the intra-chunk output: (segsum-decay matrix) x (chunk of x) on MFMA, plus the
carried state.

Mirrors kernels/ema_kernels/ema_scan_fwd.py:161-193 of the reference."""
import torch

from kernels import _lib


def _ema_scan_fwd(x, A_cumsum, states):
    """x: (B, L, T) or (b, L, nh, d); A_cumsum: (N, nchunks, chunk_size);
    states: (N, nchunks, T) states entering each chunk -> out with the shape/dtype of x."""
    dev = _lib.require_gpu(x, A_cumsum, states)
    x, x_args, batch, nh, seqlen, token_dim = _lib.seq_view(x)
    _, nchunks, _ = states.shape
    _, _, chunk_size = A_cumsum.shape
    assert A_cumsum.shape == (batch * nh, nchunks, chunk_size)
    assert states.shape == (batch * nh, nchunks, token_dim)
    assert nchunks == -(-seqlen // chunk_size)
    cs = _lib.f32c(A_cumsum)
    prev = _lib.f32c(states)
    out = torch.empty(x.shape, device=dev, dtype=x.dtype)
    _, y_args, *_ = _lib.seq_view(out)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_scan_fwd(
            *x_args, _lib.dtype_code(x), cs.data_ptr(), prev.data_ptr(), *y_args,
            batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_scan_fwd")
    return out
