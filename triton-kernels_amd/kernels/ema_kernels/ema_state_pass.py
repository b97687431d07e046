"""F3, the sequential inter-chunk recurrence.

Mirrors kernels/ema_kernels/ema_state_pass.py:125-154 of the reference."""
import torch

from kernels import _lib


def _ema_state_passing_fwd(states, A_cs_last, initial_states=None, chunk_size=None, out_dtype=None):
    """states: (N, nchunks, T); A_cs_last: (N, nchunks) (any strides, e.g. cs[..., -1]).

    Returns (out, final_states): out[:, c] is the state entering chunk c (out[:, 0] = 0),
    final_states (N, T) float32 the state after the last chunk."""
    batch, nchunks, token_dim = states.shape
    assert A_cs_last.shape == (batch, nchunks)
    if initial_states is not None:
        raise NotImplementedError("No support for init_states in EMA kernel.")
    dev = _lib.require_gpu(states, A_cs_last)
    assert A_cs_last.dtype == torch.float32
    out_dtype = states.dtype if out_dtype is None else out_dtype
    st_in = _lib.f32c(states)
    out = torch.empty((batch, nchunks, token_dim), device=dev, dtype=torch.float32)
    final_states = torch.empty((batch, token_dim), device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        st = _lib.lib().ema_state_passing_fwd(
            st_in.data_ptr(), A_cs_last.data_ptr(), A_cs_last.stride(0), A_cs_last.stride(1),
            out.data_ptr(), final_states.data_ptr(), batch, nchunks, token_dim,
            _lib.stream_ptr(dev),
        )
    _lib.check(st, "_ema_state_passing_fwd")
    return (out if out_dtype == torch.float32 else out.to(out_dtype)), final_states
