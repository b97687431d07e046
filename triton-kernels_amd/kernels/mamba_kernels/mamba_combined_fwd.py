"""The five SSD forward stages in sequence.

The reference ships the stage launchers of kernels/mamba_kernels/ without a wrapper that runs
them together (its benchmarks call mamba_ssm's mamba_chunk_scan_combined instead, e.g.
kernels/benchmarks/ema_bench.py:9); this function is that wrapper, with the argument names of
the headed entry point in kernels/ema_combined.py:100-119."""
import torch

from kernels import _lib
from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd
from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd
from kernels.mamba_kernels.mamba_scan_fwd import _chunk_scan_fwd
from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd, chunk_state_varlen
from kernels.mamba_kernels.mamba_state_pass import _state_passing_fwd


def _chunk_state_passing_fwd(B, x, dt, dA_cumsum, initial_states=None, out_dtype=None):
    """_chunk_state_fwd followed by _state_passing_fwd (kernels/mamba_kernels/mamba_state_fwd.py:138-169,
    kernels/mamba_kernels/mamba_state_pass.py:84-115 of the reference) as one kernel that keeps the
    chunk-local states on chip, or None where that kernel does not apply (then the caller runs the two
    launchers).  Returns (states (batch, nchunks, nheads, headdim, dstate) in out_dtype: the state
    entering each chunk; final_states (batch, nheads, headdim, dstate) float32), the same values bit
    for bit as the two launchers give."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    out_dtype = torch.float32 if out_dtype is None else out_dtype
    if (chunk_size % 64 or headdim not in (64, 128) or dstate not in (64, 128)
            or x.dtype not in (torch.float32, torch.bfloat16) or out_dtype not in (torch.float32, torch.bfloat16)):
        return None
    dev = _lib.require_gpu(x, B, dt, dA_cumsum)
    if B.dtype != x.dtype:
        B = B.to(x.dtype)
    x, xs = _lib.strided4(x)
    B, bs = _lib.strided4(B)
    dt_f = _lib.f32c(dt)
    dA_f = _lib.f32c(dA_cumsum)
    init = None if initial_states is None else _lib.f32c(initial_states)
    states = torch.empty(batch, nchunks, nheads, headdim, dstate, device=dev, dtype=out_dtype)
    final_states = torch.empty(batch, nheads, headdim, dstate, device=dev, dtype=torch.float32)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.lib().ssd_chunk_state_passing_fwd(*bs, *xs, _lib.dtype_code(x), dt_f.data_ptr(), dA_f.data_ptr(),
                                                   None if init is None else init.data_ptr(), states.data_ptr(),
                                                   _lib.dtype_code(states), final_states.data_ptr(), batch, seqlen,
                                                   nheads, ngroups, headdim, dstate, chunk_size,
                                                   _lib.stream_ptr(dev)),
            "ssd_chunk_state_passing_fwd")
    return states, final_states


def _mamba_chunk_scan_combined_fwd(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None,
                                   initial_states=None, seq_idx=None, cu_seqlens=None, dt_softplus=False,
                                   dt_limit=(0.0, float("inf"))):
    """Returns (out, out_x, dt_out, dA_cumsum, states, final_states), states (the state entering
    each chunk) in the dtype of C as in kernels/ema_combined.py:48-50, and as a seventh item the state
    at the end of each packed sequence when cu_seqlens is given (batch must be 1 then; the boundaries
    are the ones seq_idx marks), as kernels/ema_combined.py:56-62 of the reference does."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate) and C.shape == B.shape
    assert dt.shape == (batch, seqlen, nheads) and A.shape == (nheads,)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, headdim, dstate)
    dA_cumsum, dt_out = _chunk_cumsum_fwd(dt, A, chunk_size, dt_bias=dt_bias, dt_softplus=dt_softplus,
                                          dt_limit=dt_limit)
    fused = None
    if seq_idx is None and C.dtype in (torch.float32, torch.bfloat16):
        fused = _chunk_state_passing_fwd(B, x, dt_out, dA_cumsum, initial_states=initial_states, out_dtype=C.dtype)
    if fused is not None:
        states, final_states = fused
    else:
        states = _chunk_state_fwd(B, x, dt_out, dA_cumsum, seq_idx=seq_idx, states_in_fp32=True)
        init = None if initial_states is None else initial_states.reshape(batch, nheads, headdim * dstate)
        states, final_states = _state_passing_fwd(states.reshape(batch, -1, nheads, headdim * dstate),
                                                  dA_cumsum[:, :, :, -1], initial_states=init, seq_idx=seq_idx,
                                                  chunk_size=chunk_size, out_dtype=C.dtype)
        states = states.reshape(batch, -1, nheads, headdim, dstate)
        final_states = final_states.reshape(batch, nheads, headdim, dstate)
    CB = _bmm_chunk_fwd(C, B, chunk_size, seq_idx=seq_idx, output_dtype=torch.float32)
    out, out_x = _chunk_scan_fwd(CB, x, dt_out, dA_cumsum, C, states, D=D, z=z, seq_idx=seq_idx)
    if cu_seqlens is None:
        return out, out_x, dt_out, dA_cumsum, states, final_states
    assert batch == 1, "passing cu_seqlens to get the varlen states is only supported if batch dimension is 1"
    varlen_states = chunk_state_varlen(B.squeeze(0), x.squeeze(0), dt_out.squeeze(0), dA_cumsum.squeeze(0),
                                       cu_seqlens, states.squeeze(0))
    return out, out_x, dt_out, dA_cumsum, states, final_states, varlen_states


def mamba_chunk_scan_combined_fwd(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None,
                                  initial_states=None, seq_idx=None, cu_seqlens=None, dt_softplus=False,
                                  dt_limit=(0.0, float("inf")), return_final_states=False,
                                  return_varlen_states=False):
    """out, then the final states and the per-sequence states as asked for, in that order
    (kernels/ema_combined.py:83-87 of the reference)."""
    if return_varlen_states:
        assert cu_seqlens is not None, "cu_seqlens must be provided if return_varlen_states is True"
    else:
        cu_seqlens = None
    out, _, _, _, _, final_states, *rest = _mamba_chunk_scan_combined_fwd(
        x, dt, A, B, C, chunk_size, D=D, z=z, dt_bias=dt_bias, initial_states=initial_states,
        seq_idx=seq_idx, cu_seqlens=cu_seqlens, dt_softplus=dt_softplus, dt_limit=dt_limit)
    res = (out,) + ((final_states,) if return_final_states else ()) + tuple(rest)
    return res if len(res) > 1 else out
