"""SSD backward: gradient of the causal term of the chunk scan with respect to dA.

Mirrors _chunk_scan_bwd_ddAcs_stable, kernels/mamba_kernels_bwd/mamba_chunk_scan_bwd_da.py:111-140
of the reference; the sum over row blocks that the reference takes in torch is part of the
library call."""
import torch
import torch.nn.functional as F

from kernels import _lib


def _chunk_scan_bwd_ddAcs_stable(x, dt, dA_cumsum, dout, cb):
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dout.shape == x.shape
    assert dA_cumsum.shape == dt.shape
    ngroups = cb.shape[2]
    assert nheads % ngroups == 0
    assert cb.shape == (batch, nchunks, ngroups, chunk_size, chunk_size)
    if headdim % 8:  # rows move in 16-byte pieces: zero features change no dot product
        pad = (0, -headdim % 8)
        return _chunk_scan_bwd_ddAcs_stable(F.pad(x, pad), dt, dA_cumsum, F.pad(dout, pad), cb)
    dev = _lib.require_gpu(x, dt, dA_cumsum, dout, cb)
    lib = _lib.lib()
    x, xs = _lib.strided4(x)
    dout, ds = _lib.strided4(dout.to(x.dtype))
    ddA_cumsum = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    nbytes = lib.ssd_chunk_scan_bwd_ddAcs_workspace_bytes(batch, seqlen, nheads, chunk_size)
    assert nbytes > 0, "unsupported shape"
    ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
    # float32 views / copies are bound to names so that they outlive the launch below
    dt_f = _lib.f32c(dt)
    dA_cumsum_f = _lib.f32c(dA_cumsum)
    cb_f = _lib.f32c(cb)
    with torch.cuda.device(dev):
        _lib.check(
            lib.ssd_chunk_scan_bwd_ddAcs(*xs, *ds, _lib.dtype_code(x), dt_f.data_ptr(),
                                         dA_cumsum_f.data_ptr(), cb_f.data_ptr(),
                                         ddA_cumsum.data_ptr(), ws.data_ptr(), nbytes, batch, seqlen, nheads, ngroups,
                                         headdim, chunk_size, _lib.stream_ptr(dev)),
            "ssd_chunk_scan_bwd_ddAcs")
    return ddA_cumsum
