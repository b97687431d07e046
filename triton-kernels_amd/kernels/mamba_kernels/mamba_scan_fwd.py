"""SSD stage 5: the chunk scan (carried state, causal intra-chunk sum, skip term, gate).

Mirrors _chunk_scan_fwd, kernels/mamba_kernels/mamba_scan_fwd.py:162-210 of the reference;
returns (out, out_x) like it."""
import torch

from kernels import _lib
from kernels.mamba_kernels._shapes import Plan


def _chunk_scan_fwd(cb, x, dt, dA_cumsum, C, states, D=None, z=None, seq_idx=None):
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = C.shape
    assert nheads % ngroups == 0
    assert C.shape == (batch, seqlen, ngroups, dstate)
    assert cb.shape == (batch, nchunks, ngroups, chunk_size, chunk_size)
    if z is not None:
        assert z.shape == x.shape
    if D is not None:
        assert D.shape == (nheads, headdim) or D.shape == (nheads,)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == (batch, nheads, nchunks, chunk_size)
    assert states.shape == (batch, nchunks, nheads, headdim, dstate)
    plan = Plan(headdim, dstate)
    if not plan.native:
        out, out_x = _chunk_scan_fwd(cb, plan.x(x), plan.per_head(dt), plan.per_head(dA_cumsum), plan.bc(C),
                                     plan.states(states), D=plan.D(D), z=plan.x(z), seq_idx=seq_idx)
        return plan.x_back(out), plan.x_back(out_x)
    dev = _lib.require_gpu(x, cb, dt, dA_cumsum, C, states)
    seq_idx, ids = _lib.seq_ids(seq_idx, batch, seqlen, dev)
    x, xs = _lib.strided4(x)
    if C.dtype != x.dtype:
        C = C.to(x.dtype)
    C, cs = _lib.strided4(C)
    zs = [None, 0, 0, 0]
    if z is not None:
        z, zs = _lib.strided4(z.to(x.dtype))
    out = torch.empty(batch, seqlen, nheads, headdim, device=dev, dtype=x.dtype)
    out_x = torch.empty_like(out) if z is not None else None
    Df = None if D is None else _lib.f32c(D)
    states, st_code = _lib.state_tensor(states, like=x)
    # float32 views / copies are bound to names so that they outlive the launch below
    cb_f = _lib.f32c(cb)
    dt_f = _lib.f32c(dt)
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_scan_fwd(
                cb_f.data_ptr(), *xs, *zs, _lib.dtype_code(x), dt_f.data_ptr(),
                dA_cumsum_f.data_ptr(), *cs, states.data_ptr(), st_code,
                None if Df is None else Df.data_ptr(), int(D is not None and D.dim() == 2), out.data_ptr(),
                out.stride(0), out.stride(1), out.stride(2), None if out_x is None else out_x.data_ptr(), batch,
                seqlen, nheads, ngroups, headdim, dstate, chunk_size, *ids, _lib.stream_ptr(dev)),
            "ssd_chunk_scan_fwd")
    return out, out_x
