"""SSD backward: the gradient of the chunk scan with respect to the carried states and the reverse
inter-chunk recurrence, run back to back.

The reference ships the two launchers (_chunk_scan_bwd_dstates,
kernels/mamba_kernels_bwd/mamba_scan_bwd.py:91-116, and _state_passing_bwd,
kernels/mamba_kernels_bwd/mamba_state_passing_bwd_dstates.py:116-172) without a combined backward
that would call them; a caller that does so runs this function in their place."""
import torch

from kernels import _lib
from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates
from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd


def _fused(C, dA_cumsum, dout, states, dfinal_states, has_initial_states, out_dtype):
    """One kernel for both stages (the chunk's gradient stays in the accumulators), or None where
    that kernel does not apply."""
    batch, seqlen, nheads, headdim = dout.shape
    _, _, nchunks, chunk_size = dA_cumsum.shape
    _, _, ngroups, dstate = C.shape
    if (headdim != 64 or dstate != 128 or chunk_size % 64 or chunk_size < 128 or dout.dtype != torch.bfloat16
            or states.dtype != torch.bfloat16 or out_dtype not in (torch.float32, torch.bfloat16)):
        return None
    dev = _lib.require_gpu(C, dA_cumsum, dout, states)
    lib = _lib.lib()
    if C.dtype != dout.dtype:
        C = C.to(dout.dtype)
    dout, ds = _lib.strided4(dout)
    C, cs = _lib.strided4(C)
    if min(ds[1:]) < 0 or min(cs[1:]) < 0:
        return None
    # dense views / copies are bound to names so that they outlive the launch below
    dA_f = _lib.f32c(dA_cumsum)
    st = states.contiguous()
    dfin = None if dfinal_states is None else _lib.f32c(dfinal_states)
    dstates = torch.empty(batch, nchunks, nheads, headdim, dstate, device=dev, dtype=out_dtype)
    ddA = torch.empty(batch, nheads, nchunks, device=dev, dtype=torch.float32)
    dinit = (torch.empty(batch, nheads, headdim, dstate, device=dev, dtype=torch.float32)
             if has_initial_states else None)
    nbytes = lib.ssd_chunk_scan_state_passing_bwd_workspace_bytes(batch, nchunks, nheads)
    ws = torch.empty(max(nbytes, 16), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        _lib.check(
            lib.ssd_chunk_scan_state_passing_bwd(*cs, *ds, _lib.dtype_code(dout), dA_f.data_ptr(), st.data_ptr(),
                                                 _lib.dtype_code(st), None if dfin is None else dfin.data_ptr(),
                                                 dstates.data_ptr(), _lib.dtype_code(dstates), ddA.data_ptr(),
                                                 None if dinit is None else dinit.data_ptr(), ws.data_ptr(), nbytes,
                                                 batch, seqlen, nheads, ngroups, headdim, dstate, chunk_size,
                                                 _lib.stream_ptr(dev)),
            "ssd_chunk_scan_state_passing_bwd")
    return dstates, ddA, dinit


def _chunk_scan_state_passing_bwd(C, dA_cumsum, dout, states, dfinal_states=None, seq_idx=None,
                                  has_initial_states=None, dstates_dtype=None):
    """C (batch, seqlen, ngroups, dstate), dA_cumsum (batch, nheads, nchunks, chunk_size), dout
    (batch, seqlen, nheads, headdim), states (batch, nchunks, nheads, headdim, dstate): the state
    entering each chunk, dfinal_states (batch, nheads, headdim, dstate) or None.  Returns what
    _state_passing_bwd returns, shaped like states: (dstates, the gradient of each chunk's local
    state; ddA_chunk_cumsum (batch, nheads, nchunks); dinitial_states or None).  The gradient with
    respect to the entering states that _chunk_scan_bwd_dstates would return travels between the
    two stages in float32 and is not returned."""
    batch, seqlen, nheads, headdim = dout.shape
    _, _, nchunks, chunk_size = dA_cumsum.shape
    _, _, ngroups, dstate = C.shape
    assert states.shape == (batch, nchunks, nheads, headdim, dstate)
    if dfinal_states is not None:
        assert dfinal_states.shape == (batch, nheads, headdim, dstate)
    out_dtype = dstates_dtype if dstates_dtype is not None else states.dtype
    if seq_idx is None:
        fused = _fused(C, dA_cumsum, dout, states, dfinal_states, has_initial_states, out_dtype)
        if fused is not None:
            return fused
    dim = headdim * dstate
    dprev = _chunk_scan_bwd_dstates(C, dA_cumsum, dout, seq_idx=seq_idx, dtype=torch.float32)
    dfin = None if dfinal_states is None else dfinal_states.reshape(batch, nheads, dim)
    dstates, ddA, dinit = _state_passing_bwd(states.reshape(batch, nchunks, nheads, dim), dA_cumsum[..., -1],
                                             dprev.reshape(batch, nchunks, nheads, dim), dfinal_states=dfin,
                                             seq_idx=seq_idx, has_initial_states=has_initial_states,
                                             dstates_dtype=out_dtype, chunk_size=chunk_size)
    dstates = dstates.reshape(batch, nchunks, nheads, headdim, dstate)
    return dstates, ddA, None if dinit is None else dinit.reshape(batch, nheads, headdim, dstate)
