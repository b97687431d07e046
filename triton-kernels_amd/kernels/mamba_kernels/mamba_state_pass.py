"""SSD stage 3: the inter-chunk recurrence over the flattened (hdim * dstate) states.

Mirrors _state_passing_fwd, kernels/mamba_kernels/mamba_state_pass.py:84-115 of the reference."""
import torch
import torch.nn.functional as F

from kernels import _lib


def _state_passing_fwd(states, dA_chunk_cumsum, initial_states=None, seq_idx=None, chunk_size=None,
                       out_dtype=None):
    batch, nchunks, nheads, dim = states.shape
    assert dA_chunk_cumsum.shape == (batch, nheads, nchunks)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, dim)
    if dim % 4:  # the kernel moves four state elements per thread: pad with zeros, cut off again
        pad = (0, -dim % 4)
        out, final = _state_passing_fwd(F.pad(states, pad), dA_chunk_cumsum,
                                        None if initial_states is None else F.pad(initial_states, pad),
                                        seq_idx=seq_idx, chunk_size=chunk_size, out_dtype=out_dtype)
        return out[..., :dim], final[..., :dim]
    dev = _lib.require_gpu(states, dA_chunk_cumsum)
    seqlen = 0
    if seq_idx is not None:
        assert chunk_size is not None
        seqlen = seq_idx.shape[-1]
        assert nchunks == (seqlen + chunk_size - 1) // chunk_size
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    out_dtype = states.dtype if out_dtype is None else out_dtype
    st = _lib.f32c(states)
    da = dA_chunk_cumsum if dA_chunk_cumsum.dtype == torch.float32 else dA_chunk_cumsum.float()
    init = None if initial_states is None else _lib.f32c(initial_states)
    # float32 and bfloat16 copies of the carried states are written by the kernel itself
    native = out_dtype if out_dtype in (torch.float32, torch.bfloat16) else torch.float32
    out = torch.empty(batch, nchunks, nheads, dim, device=dev, dtype=native)
    final_states = torch.empty(batch, nheads, dim, device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_state_passing_fwd(st.data_ptr(), da.data_ptr(), da.stride(0), da.stride(1), da.stride(2),
                                             None if init is None else init.data_ptr(), out.data_ptr(),
                                             _lib.dtype_code(out), final_states.data_ptr(), batch, nchunks, nheads,
                                             dim, *ids, seqlen, chunk_size or 0, _lib.stream_ptr(dev)),
            "ssd_state_passing_fwd")
    return (out if out_dtype == native else out.to(out_dtype)), final_states
