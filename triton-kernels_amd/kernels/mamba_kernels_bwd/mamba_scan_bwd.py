"""SSD backward: gradient of the chunk scan with respect to the carried states.

Mirrors _chunk_scan_bwd_dstates, kernels/mamba_kernels_bwd/mamba_scan_bwd.py:91-116 of the
reference."""
import torch

from kernels import _lib
from kernels.mamba_kernels._shapes import Plan


def _chunk_scan_bwd_dstates(C, dA_cumsum, dout, seq_idx=None, dtype=None):
    batch, seqlen, nheads, headdim = dout.shape
    _, _, nchunks, chunk_size = dA_cumsum.shape
    _, _, ngroups, dstate = C.shape
    assert nheads % ngroups == 0
    assert C.shape == (batch, seqlen, ngroups, dstate)
    assert dA_cumsum.shape == (batch, nheads, nchunks, chunk_size)
    plan = Plan(headdim, dstate)
    if not plan.native:
        out = _chunk_scan_bwd_dstates(plan.bc(C), plan.per_head(dA_cumsum), plan.x(dout), seq_idx=seq_idx,
                                      dtype=C.dtype if dtype is None else dtype)
        return plan.states_back(out)
    dev = _lib.require_gpu(C, dA_cumsum, dout)
    dtype = C.dtype if dtype is None else dtype
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    dout, ds = _lib.strided4(dout)
    if C.dtype != dout.dtype:
        C = C.to(dout.dtype)
    C, cs = _lib.strided4(C)
    # the kernel stores float32, or bfloat16 next to bfloat16 inputs; any other type is cast afterwards
    native = dtype if dtype == torch.float32 or (dtype == torch.bfloat16 and dout.dtype == dtype) else torch.float32
    out = torch.empty(batch, nchunks, nheads, headdim, dstate, device=dev, dtype=native)
    # float32 views / copies are bound to names so that they outlive the launch below
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_scan_bwd_dstates(*cs, *ds, _lib.dtype_code(dout), dA_cumsum_f.data_ptr(),
                                                  out.data_ptr(), _lib.dtype_code(out), batch, seqlen, nheads, ngroups, headdim, dstate,
                                                  chunk_size, *ids, _lib.stream_ptr(dev)),
            "ssd_chunk_scan_bwd_dstates")
    return out if dtype == native else out.to(dtype)
