"""B2, the reverse inter-chunk recurrence.

Mirrors kernels/ema_kernels_bwd/ema_state_passing_bwd_dstates.py:103-183 of the reference."""
import torch

from kernels import _lib


def _ema_state_passing_bwd(
    states,
    dA_chunk_cumsum,
    dout,
    dfinal_states=None,
    seq_idx=None,
    has_initial_states=False,
    dstates_dtype=None,
    states_dtype=None,
    chunk_size=None,
):
    """states: (N, C, T) states entering each chunk; dA_chunk_cumsum: (N, C) chunk totals of
    the log-decay (any strides); dout: (N, C, T) gradient of `states` from the chunk scan.

    Returns (dstates (N, C, T), ddA_chunk_cumsum (N, C), None[, states_converted]) exactly
    like the reference: dstates[:, c] is the gradient of the chunk-local state of chunk c."""
    batch, nchunks, token_dim = states.shape
    assert dA_chunk_cumsum.shape == (batch, nchunks)
    assert dout.shape == (batch, nchunks, token_dim)
    assert dfinal_states is None
    assert seq_idx is None
    assert not has_initial_states
    dev = _lib.require_gpu(states, dA_chunk_cumsum, dout)
    assert dA_chunk_cumsum.dtype == torch.float32
    prev = _lib.f32c(states)
    ds = _lib.f32c(dout)
    g = torch.empty(batch, nchunks, token_dim, device=dev, dtype=torch.float32)
    ddA = torch.empty(batch, nchunks, device=dev, dtype=torch.float32)
    L = _lib.lib()
    ws_bytes = L.ema_state_passing_bwd_workspace_bytes(batch, nchunks, token_dim)
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        st = L.ema_state_passing_bwd(
            prev.data_ptr(), dA_chunk_cumsum.data_ptr(), dA_chunk_cumsum.stride(0),
            dA_chunk_cumsum.stride(1), ds.data_ptr(), g.data_ptr(), ddA.data_ptr(),
            ws.data_ptr(), ws_bytes, batch, nchunks, token_dim, _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_state_passing_bwd")
    out_dtype = dstates_dtype if dstates_dtype is not None else dout.dtype
    dstates = g if out_dtype == torch.float32 else g.to(out_dtype)
    if states_dtype is None:
        return dstates, ddA, None
    states_converted = states if states_dtype == states.dtype else states.to(out_dtype)
    return dstates, ddA, None, states_converted
