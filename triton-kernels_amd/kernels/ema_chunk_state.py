"""Per-sequence end states of a packed batch, under the module path of the reference's legacy
stage file (chunk_state_varlen, kernels/ema_chunk_state.py:578-604)."""
from kernels.mamba_kernels.mamba_state_fwd import chunk_state_varlen

__all__ = ["chunk_state_varlen"]
