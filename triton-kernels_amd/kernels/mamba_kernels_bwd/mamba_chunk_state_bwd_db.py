"""SSD backward: dB through the chunk states, and the matching gradient of dA.

Mirrors _chunk_state_bwd_db, kernels/mamba_kernels_bwd/mamba_chunk_state_bwd_db.py:131-181 of
the reference.  One workgroup walks all heads of a group, so the reference's split axis and the
torch sum over it are gone; the cumsum of ddA_cumsum is part of the library call."""
import torch

from kernels import _lib
from kernels.mamba_kernels._shapes import Plan


def _chunk_state_bwd_db(x, dt, dA_cumsum, dstates, seq_idx=None, B=None, ngroups=1):
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    dstate = dstates.shape[-1]
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    assert dstates.shape == (batch, nchunks, nheads, headdim, dstate)
    plan = Plan(headdim, dstate)
    if not plan.native:
        res = _chunk_state_bwd_db(plan.x(x), plan.per_head(dt), plan.per_head(dA_cumsum), plan.states(dstates),
                                  seq_idx=seq_idx, B=plan.bc(B), ngroups=ngroups)
        if B is None:
            return plan.bc_back(res)
        return plan.bc_back(res[0]), plan.per_head_sum(res[1])
    dev = _lib.require_gpu(x, dt, dA_cumsum, dstates)
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    x, xs = _lib.strided4(x)
    bs = [None, 0, 0, 0]
    ddA_cumsum = None
    if B is not None:
        assert B.shape == (batch, seqlen, ngroups, dstate)
        B, bs = _lib.strided4(B.to(x.dtype))
        ddA_cumsum = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    dB = torch.empty(batch, seqlen, ngroups, dstate, device=dev, dtype=torch.float32)
    dstates, ds_code = _lib.state_tensor(dstates, like=x)
    # float32 views / copies are bound to names so that they outlive the launch below
    dt_f = _lib.f32c(dt)
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_state_bwd_db(*xs, _lib.dtype_code(x), dt_f.data_ptr(),
                                              dA_cumsum_f.data_ptr(), dstates.data_ptr(), ds_code, *bs,
                                              dB.data_ptr(), None if ddA_cumsum is None else ddA_cumsum.data_ptr(),
                                              batch, seqlen, nheads, ngroups, headdim, dstate, chunk_size, *ids,
                                              _lib.stream_ptr(dev)),
            "ssd_chunk_state_bwd_db")
    return dB if B is None else (dB, ddA_cumsum)
