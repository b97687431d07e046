"""SSD backward: dx, the explicit-dt gradient ddt and dD.

Mirrors _chunk_scan_chunk_state_bwd_dx,
kernels/mamba_kernels_bwd/mamba_chunk_scan_chunk_state_bwd_dx.py:189-248 of the reference (same
arguments, returns (dx, ddt, dD)).  For dD = sum dout * x the kernel leaves one partial sum per wave
and feature, which are added up here, as the reference adds its per-block partials (:245-247)."""
import torch

from kernels import _lib
from kernels.mamba_kernels._shapes import Plan


def _chunk_scan_chunk_state_bwd_dx(x, dt, dA_cumsum, B, CB, dout, dstates, D=None, seq_idx=None, dx=None):
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert CB.shape == (batch, nchunks, ngroups, chunk_size, chunk_size)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    assert dout.shape == x.shape
    assert dstates.shape == (batch, nchunks, nheads, headdim, dstate)
    plan = Plan(headdim, dstate)
    if not plan.native:
        assert dx is None, "a preallocated result needs a native shape"
        dxs, ddt, dD = _chunk_scan_chunk_state_bwd_dx(plan.x(x), plan.per_head(dt), plan.per_head(dA_cumsum),
                                                      plan.bc(B), CB, plan.x(dout), plan.states(dstates),
                                                      D=plan.D(D), seq_idx=seq_idx)
        return plan.x_back(dxs), plan.per_head_sum(ddt), plan.dD_back(dD, D)
    if D is not None:
        assert D.shape == (nheads, headdim) or D.shape == (nheads,)
    dev = _lib.require_gpu(x, dt, dA_cumsum, B, CB, dout, dstates)
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    x, xs = _lib.strided4(x)
    dout, ds = _lib.strided4(dout.to(x.dtype))
    B, bs = _lib.strided4(B.to(x.dtype))
    if dx is None:
        dx = torch.empty_like(x)
    else:
        assert dx.shape == x.shape and dx.dtype == x.dtype and dx.stride(-1) == 1
    ddt = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    Df = None if D is None else _lib.f32c(D)
    dstates, ds_code = _lib.state_tensor(dstates, like=x)
    dD_part = None
    if D is not None:  # per-wave partial sums of dout * x, summed below like the reference's per-block ones
        slots = _lib.lib().ssd_chunk_scan_chunk_state_bwd_dx_dD_slots(_lib.dtype_code(x), headdim, dstate, chunk_size)
        assert slots > 0, "unsupported shape"
        dD_part = torch.empty(batch, nchunks, nheads, slots, headdim, device=dev, dtype=torch.float32)
    # float32 views / copies are bound to names so that they outlive the launch below
    CB_f = _lib.f32c(CB)
    dt_f = _lib.f32c(dt)
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_scan_chunk_state_bwd_dx(
                CB_f.data_ptr(), *xs, *ds, _lib.dtype_code(x), dt_f.data_ptr(),
                dA_cumsum_f.data_ptr(), *bs, dstates.data_ptr(), ds_code,
                None if Df is None else Df.data_ptr(), int(D is not None and D.dim() == 2), dx.data_ptr(),
                dx.stride(0), dx.stride(1), dx.stride(2), ddt.data_ptr(), batch, seqlen, nheads, ngroups, headdim,
                dstate, chunk_size, *ids, None if dD_part is None else dD_part.data_ptr(), _lib.stream_ptr(dev)),
            "ssd_chunk_scan_chunk_state_bwd_dx")
    dD = None
    if D is not None:
        dD = dD_part.sum((0, 1, 3))
        dD = (dD if D.dim() == 2 else dD.sum(-1)).to(D.dtype)
    return dx, ddt.to(dtype=dt.dtype), dD
