"""Stage launchers of the reference's legacy headed EMA path under its module path
(kernels/ema_chunk_state.py): the Mamba-2 SSD stages with the decay fixed to dA = -dt."""
import torch

from kernels.mamba_kernels import mamba_cumsum
from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd, chunk_state_varlen


def _chunk_cumsum_fwd(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """Returns (dA_cumsum, dt_out), both (batch, nheads, nchunks, chunk_size) float32.  A only gives
    the number of heads: the cumulative sum runs over -dt (kernels/ema_chunk_state.py:85-96)."""
    assert A.shape == (dt.shape[2],)
    minus_one = -torch.ones(dt.shape[2], device=dt.device, dtype=torch.float32)
    return mamba_cumsum._chunk_cumsum_fwd(dt, minus_one, chunk_size, dt_bias=dt_bias, dt_softplus=dt_softplus,
                                          dt_limit=dt_limit)


def _simplified_chunk_state_fwd(B, x, dt, dA_cumsum, seq_idx=None, states=None, states_in_fp32=True):
    """The reference's variant for a state dimension of 1 (kernels/ema_chunk_state.py:446-494; its
    kernel writes state column 0 only).  Same launcher here; any supported dstate is computed in
    full."""
    return _chunk_state_fwd(B, x, dt, dA_cumsum, seq_idx=seq_idx, states=states, states_in_fp32=states_in_fp32)


__all__ = ["_chunk_cumsum_fwd", "_chunk_state_fwd", "_simplified_chunk_state_fwd", "chunk_state_varlen"]
