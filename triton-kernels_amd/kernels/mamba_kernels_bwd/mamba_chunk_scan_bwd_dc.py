"""SSD backward: the part of dC that comes through the carried state, and the matching gradient
of dA_cumsum.

Mirrors _chunk_scan_bwd_dC, kernels/mamba_kernels_bwd/mamba_chunk_scan_bwd_dc.py:118-160 of the
reference (no split axis: one workgroup walks all heads of a group)."""
import torch

from kernels import _lib
from kernels.mamba_kernels._shapes import Plan


def _chunk_scan_bwd_dC(prev_states, dA_cumsum, dout, seq_idx=None, C=None, ngroups=1):
    batch, nchunks, nheads, headdim, dstate = prev_states.shape
    _, seqlen, _, _ = dout.shape
    _, _, _, chunk_size = dA_cumsum.shape
    assert prev_states.shape == (batch, nchunks, nheads, headdim, dstate)
    assert dA_cumsum.shape == (batch, nheads, nchunks, chunk_size)
    assert dout.shape == (batch, seqlen, nheads, headdim)
    plan = Plan(headdim, dstate)
    if not plan.native:
        res = _chunk_scan_bwd_dC(plan.states(prev_states), plan.per_head(dA_cumsum), plan.x(dout), seq_idx=seq_idx,
                                 C=plan.bc(C), ngroups=ngroups)
        if C is None:
            return plan.bc_back(res)
        return plan.bc_back(res[0]), plan.per_head_sum(res[1])
    dev = _lib.require_gpu(prev_states, dA_cumsum, dout)
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    dout, ds = _lib.strided4(dout)
    cs = [None, 0, 0, 0]
    ddA_prev = None
    if C is not None:
        assert C.shape == (batch, seqlen, ngroups, dstate)
        C, cs = _lib.strided4(C.to(dout.dtype))
        ddA_prev = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    dC = torch.empty(batch, seqlen, ngroups, dstate, device=dev, dtype=torch.float32)
    prev_states, st_code = _lib.state_tensor(prev_states, like=dout)
    # float32 views / copies are bound to names so that they outlive the launch below
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_scan_bwd_dc(*ds, _lib.dtype_code(dout), dA_cumsum_f.data_ptr(),
                                             prev_states.data_ptr(), st_code, *cs, dC.data_ptr(),
                                             None if ddA_prev is None else ddA_prev.data_ptr(), batch, seqlen,
                                             nheads, ngroups, headdim, dstate, chunk_size, *ids,
                                             _lib.stream_ptr(dev)),
            "ssd_chunk_scan_bwd_dc")
    return dC if C is None else (dC, ddA_prev)
