"""Headed, Mamba-encoded entry point of the reference's legacy EMA path.

Mirrors the signature of ema_chunk_scan_combined, kernels/ema_combined.py:100-119 of the
reference.  That path runs the Mamba-2 SSD kernels with a state dimension of 1 and the decay
fixed to dA = -dt (kernels/ema_chunk_state.py:95 ignores A); with that encoding

    state_t = exp(-dt_t) * state_{t-1} + dt_t * B_t * x_t,     out_t = C_t * state_t

per (batch, head, feature), which is the EMA scan with log-decay -dt and input dt * B * x,
scaled by C.  Only that encoding is supported."""
import torch

from kernels.ema_kernels.ema_combined_fwd import _ema_matmul_scan_combined_fwd, ema_matmul_scan_combined


def ema_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None,
                            seq_idx=None, cu_seqlens=None, dt_softplus=False, dt_limit=(0.0, float("inf")),
                            return_final_states=False, return_varlen_states=False):
    """x: (batch, seqlen, nheads, headdim); dt: (batch, seqlen, nheads); A: (nheads,) (unused, as
    in the reference); B, C: (batch, seqlen, ngroups, 1).  Returns out (batch, seqlen, nheads,
    headdim), and the final states (batch, nheads, headdim, 1) if return_final_states."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, seqlen, nheads)
    assert A.shape == (nheads,)
    assert C.shape == B.shape
    if dstate != 1:
        raise NotImplementedError("the EMA encoding has a state dimension of 1")
    if D is not None or z is not None or dt_bias is not None or dt_softplus:
        raise NotImplementedError("D, z, dt_bias and dt_softplus are not part of the EMA encoding")
    if initial_states is not None or seq_idx is not None or cu_seqlens is not None or return_varlen_states:
        raise NotImplementedError("initial_states, seq_idx and varlen states are not supported")
    if tuple(dt_limit) != (0.0, float("inf")):
        raise NotImplementedError("dt_limit is not supported")
    rep = nheads // ngroups
    dtf = dt.float()
    Bh = B[..., 0].float().repeat_interleave(rep, dim=-1)  # (batch, seqlen, nheads)
    Ch = C[..., 0].float().repeat_interleave(rep, dim=-1)
    X = ((dtf * Bh)[..., None] * x.float()).to(x.dtype)
    if return_final_states:
        out, _, _, final = _ema_matmul_scan_combined_fwd(-dtf, X, chunk_size)
        out = (Ch[..., None] * out.float()).to(x.dtype)
        # the state itself is not scaled by C
        return out, final.reshape(batch, nheads, headdim, 1)
    out = ema_matmul_scan_combined(-dtf, X, chunk_size)
    return (Ch[..., None] * out.float()).to(x.dtype)
