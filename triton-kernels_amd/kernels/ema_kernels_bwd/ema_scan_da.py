"""B6, intra-chunk log-decay gradient.  Chunks whose cumsum never rises take the factored form (two
chunk-local scans and one dot per row); the others the dout . x^T contraction over the feature axis
on MFMA, scaled by the segsum decays and reduced by a two-dimensional prefix.

Mirrors kernels/ema_kernels_bwd/ema_scan_da.py:113-137 of the reference."""
import torch

from kernels import _lib


def _ema_chunk_scan_bwd_ddAcs_stable(x, dA_cumsum, dout):
    """x, dout: (B, L, T) or (b, L, nh, d); dA_cumsum: (N, C, Q) -> ddA_cumsum (N, C, Q)."""
    dev = _lib.require_gpu(x, dA_cumsum, dout)
    x, x_args, batch, nh, seqlen, token_dim = _lib.seq_view(x)
    dout, d_args, *_ = _lib.seq_view(dout)
    _, nchunks, chunk_size = dA_cumsum.shape
    assert dout.shape == x.shape
    assert dout.dtype == x.dtype
    assert dA_cumsum.shape[0] == batch * nh and nchunks == -(-seqlen // chunk_size)
    cs = _lib.f32c(dA_cumsum)
    ddA_cumsum = torch.empty(batch * nh, nchunks, chunk_size, device=dev, dtype=torch.float32)
    L = _lib.lib()
    ws_bytes = L.ema_chunk_scan_bwd_ddAcs_workspace_bytes(
        batch, nh, seqlen, token_dim, chunk_size, _lib.dtype_code(x)
    )
    assert ws_bytes > 0, "unsupported shape"
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        st = L.ema_chunk_scan_bwd_ddAcs(
            *x_args, *d_args, _lib.dtype_code(x), cs.data_ptr(), ddA_cumsum.data_ptr(),
            ws.data_ptr(), ws_bytes, batch, nh, seqlen, token_dim, chunk_size, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_chunk_scan_bwd_ddAcs_stable")
    return ddA_cumsum
