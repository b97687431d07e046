"""SSD stage 2: chunk states B^T x, weighted by the decay to the end of the chunk and dt.

Mirrors _chunk_state_fwd, kernels/mamba_kernels/mamba_state_fwd.py:138-169 of the reference, and
chunk_state_varlen of its legacy stage file, kernels/ema_chunk_state.py:578-604."""
import torch

from kernels import _lib
from kernels.mamba_kernels._shapes import Plan


def _chunk_state_fwd(B, x, dt, dA_cumsum, seq_idx=None, states=None, states_in_fp32=True):
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    plan = Plan(headdim, dstate)
    if not plan.native:  # bring the shape to one the kernels take, run, cut the result back
        assert states is None, "a preallocated result needs a native shape"
        out = _chunk_state_fwd(plan.bc(B), plan.x(x), plan.per_head(dt), plan.per_head(dA_cumsum), seq_idx=seq_idx,
                               states_in_fp32=states_in_fp32)
        return plan.states_back(out)
    dev = _lib.require_gpu(x, B, dt, dA_cumsum)
    if B.dtype != x.dtype:
        B = B.to(x.dtype)  # the reference rounds the weighted B to x's type before the product
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    x, xs = _lib.strided4(x)
    B, bs = _lib.strided4(B)
    # a preallocated dense float32 result is written in place, as the reference's launcher does
    # (kernels/mamba_kernels/mamba_state_fwd.py:147-151); any other goes through a copy
    in_place = (states is not None and states.dtype == torch.float32 and states.is_contiguous()
                and states.device == dev and states.shape == (batch, nchunks, nheads, headdim, dstate))
    out = states if in_place else torch.empty(batch, nchunks, nheads, headdim, dstate, device=dev,
                                              dtype=torch.float32)
    # float32 views / copies are bound to names so that they outlive the launch below
    dt_f = _lib.f32c(dt)
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_state_fwd(*bs, *xs, _lib.dtype_code(x), dt_f.data_ptr(),
                                           dA_cumsum_f.data_ptr(), out.data_ptr(), batch, seqlen, nheads,
                                           ngroups, headdim, dstate, chunk_size, *ids, _lib.stream_ptr(dev)),
            "ssd_chunk_state_fwd")
    if states is not None:
        assert states.shape == (batch, nchunks, nheads, headdim, dstate)
        if not in_place:
            states.copy_(out)
        return states
    return out if states_in_fp32 else out.to(B.dtype)


def chunk_state_varlen(B, x, dt, dA_cumsum, cu_seqlens, chunk_states):
    """States at the end of each sequence of a packed batch (no batch dimension: x is
    (total_seqlen, nheads, headdim), B (total_seqlen, ngroups, dstate), dt and dA_cumsum
    (nheads, nchunks, chunk_size), chunk_states (nchunks, nheads, headdim, dstate) the state
    entering each chunk, cu_seqlens (num_sequences + 1) the sequence boundaries).  Returns
    (num_sequences, nheads, headdim, dstate) in the dtype of chunk_states."""
    total_seqlen, nheads, headdim = x.shape
    _, nchunks, chunk_size = dt.shape
    _, ngroups, dstate = B.shape
    batch = cu_seqlens.shape[0] - 1
    assert nheads % ngroups == 0
    assert B.shape == (total_seqlen, ngroups, dstate)
    assert dt.shape == (nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    assert chunk_states.shape == (nchunks, nheads, headdim, dstate)
    assert batch >= 1 and nchunks == -(-total_seqlen // chunk_size)
    dev = _lib.require_gpu(x, B, dt, dA_cumsum, chunk_states, cu_seqlens)
    if B.dtype != x.dtype:
        B = B.to(x.dtype)
    if x.stride(-1) != 1:
        x = x.contiguous()
    if B.stride(-1) != 1:
        B = B.contiguous()
    cu = cu_seqlens.to(torch.int32).contiguous()
    st, st_code = _lib.state_tensor(chunk_states, like=x)
    states = torch.empty(batch, nheads, headdim, dstate, device=dev, dtype=torch.float32)
    # float32 views / copies are bound to names so that they outlive the launch below
    dt_f = _lib.f32c(dt)
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_state_varlen(B.data_ptr(), B.stride(0), B.stride(1), x.data_ptr(), x.stride(0),
                                              x.stride(1), _lib.dtype_code(x), dt_f.data_ptr(),
                                              dA_cumsum_f.data_ptr(), st.data_ptr(), st_code,
                                              cu.data_ptr(), states.data_ptr(), batch, total_seqlen, nheads, ngroups,
                                              headdim, dstate, chunk_size, _lib.stream_ptr(dev)),
            "ssd_chunk_state_varlen")
    return states.to(chunk_states.dtype)
