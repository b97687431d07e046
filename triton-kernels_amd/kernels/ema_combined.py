"""Headed, Mamba-encoded entry point of the reference's legacy EMA path.

Mirrors the signature of ema_chunk_scan_combined, kernels/ema_combined.py:100-119 of the
reference.  That path runs Mamba-2 SSD kernels with the decay fixed to dA = -dt
(kernels/ema_chunk_state.py:95 ignores A):

    state_t = exp(-dt_t) * state_{t-1} + dt_t * x_t (outer) B_t,     out_t = C_t . state_t + D x_t

The EMA encoding is the case of a state dimension of 1 with no D, z, bias or initial state:
per (batch, head, feature) it is the EMA scan with log-decay -dt and input dt * B * x, scaled by
C, and runs on the EMA kernels.  Every other case runs on the SSD stage kernels with A = -1,
including state dimensions above 1, which the reference's path does not compute (its chunk-state
kernel writes state column 0 only, kernels/ema_chunk_state.py:325-345)."""
import torch

from kernels.ema_kernels.ema_combined_fwd import _ema_matmul_scan_combined_fwd, ema_matmul_scan_combined


def ema_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None,
                            seq_idx=None, cu_seqlens=None, dt_softplus=False, dt_limit=(0.0, float("inf")),
                            return_final_states=False, return_varlen_states=False):
    """x: (batch, seqlen, nheads, headdim); dt: (batch, seqlen, nheads); A: (nheads,) (unused, as
    in the reference); B, C: (batch, seqlen, ngroups, dstate).  Returns out (batch, seqlen, nheads,
    headdim), then the final states (batch, nheads, headdim, dstate) if return_final_states, then
    the state at the end of each packed sequence (num_sequences, nheads, headdim, dstate) if
    return_varlen_states (cu_seqlens (num_sequences + 1), batch of 1)."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, seqlen, nheads)
    assert A.shape == (nheads,)
    assert C.shape == B.shape
    if return_varlen_states:
        assert cu_seqlens is not None, "cu_seqlens must be provided if return_varlen_states is True"
    ema_encoding = (dstate == 1 and D is None and z is None and dt_bias is None and not dt_softplus
                    and initial_states is None and seq_idx is None and not return_varlen_states
                    and tuple(dt_limit) == (0.0, float("inf")))
    if not ema_encoding:
        from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

        minus_one = -torch.ones(nheads, device=x.device, dtype=torch.float32)  # the path ignores A
        return mamba_chunk_scan_combined_fwd(
            x, dt, minus_one, B, C, chunk_size, D=D, z=z, dt_bias=dt_bias, initial_states=initial_states,
            seq_idx=seq_idx, cu_seqlens=cu_seqlens, dt_softplus=dt_softplus, dt_limit=dt_limit,
            return_final_states=return_final_states, return_varlen_states=return_varlen_states)
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
