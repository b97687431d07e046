"""SSD backward: the reverse inter-chunk recurrence.

Mirrors _state_passing_bwd, kernels/mamba_kernels_bwd/mamba_state_passing_bwd_dstates.py:116-172
of the reference (same arguments, same tuple of results)."""
import torch
import torch.nn.functional as F

from kernels import _lib


def _state_passing_bwd(states, dA_chunk_cumsum, dout, dfinal_states=None, seq_idx=None, has_initial_states=None,
                       dstates_dtype=None, states_dtype=None, chunk_size=None):
    """states holds the state entering each chunk (the initial state at index 0); the final state
    is not part of it."""
    batch, nchunks, nheads, dim = states.shape
    assert dA_chunk_cumsum.shape == (batch, nheads, nchunks)
    assert dout.shape == (batch, nchunks, nheads, dim)
    if dim % 4:  # the kernel moves four state elements per thread: pad with zeros, cut off again
        pad = (0, -dim % 4)
        res = _state_passing_bwd(F.pad(states, pad), dA_chunk_cumsum, F.pad(dout, pad),
                                 None if dfinal_states is None else F.pad(dfinal_states, pad), seq_idx=seq_idx,
                                 has_initial_states=has_initial_states, dstates_dtype=dstates_dtype,
                                 states_dtype=states_dtype, chunk_size=chunk_size)
        cut = lambda t: None if t is None else t[..., :dim]
        return (cut(res[0]), res[1], cut(res[2])) + tuple(cut(t) for t in res[3:])
    if dfinal_states is not None:
        assert dfinal_states.shape == (batch, nheads, dim)
    dev = _lib.require_gpu(states, dA_chunk_cumsum, dout)
    lib = _lib.lib()
    seqlen = 0
    if seq_idx is not None:
        assert chunk_size is not None
        seqlen = seq_idx.shape[-1]
        assert nchunks == (seqlen + chunk_size - 1) // chunk_size
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    (st, st_code), (do, do_code) = _lib.state_tensor(states), _lib.state_tensor(dout)
    out_dtype = dstates_dtype if dstates_dtype is not None else dout.dtype
    native = out_dtype if out_dtype in (torch.float32, torch.bfloat16) else torch.float32
    da = dA_chunk_cumsum if dA_chunk_cumsum.dtype == torch.float32 else dA_chunk_cumsum.float()
    dfin = None if dfinal_states is None else _lib.f32c(dfinal_states)
    dstates = torch.empty(batch, nchunks, nheads, dim, device=dev, dtype=native)
    ddA = torch.empty(batch, nheads, nchunks, device=dev, dtype=torch.float32)
    dinit = torch.empty(batch, nheads, dim, device=dev, dtype=torch.float32) if has_initial_states else None
    nbytes = lib.ssd_state_passing_bwd_workspace_bytes(batch, nchunks, nheads, dim)
    ws = torch.empty(max(nbytes, 16), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        _lib.check(
            lib.ssd_state_passing_bwd(st.data_ptr(), st_code, da.data_ptr(), da.stride(0), da.stride(1), da.stride(2),
                                      do.data_ptr(), do_code, None if dfin is None else dfin.data_ptr(),
                                      dstates.data_ptr(), _lib.dtype_code(dstates),
                                      ddA.data_ptr(), None if dinit is None else dinit.data_ptr(), ws.data_ptr(),
                                      nbytes, batch, nchunks, nheads, dim, *ids, seqlen, chunk_size or 0,
                                      _lib.stream_ptr(dev)),
            "ssd_state_passing_bwd")
    if out_dtype != native:
        dstates = dstates.to(out_dtype)
    if out_dtype != torch.float32:
        dinit = None if dinit is None else dinit.to(out_dtype)
    ddA = ddA.to(dA_chunk_cumsum.dtype)
    if states_dtype is None:
        return dstates, ddA, dinit
    states_converted = states if states_dtype == states.dtype else states.to(out_dtype)
    return dstates, ddA, dinit, states_converted
