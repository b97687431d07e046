"""kernels/ema_state_passing.py of the reference (same kernel as its
kernels/mamba_kernels/mamba_state_pass.py): the recurrence over the chunk states."""
from kernels.mamba_kernels.mamba_state_pass import _state_passing_fwd

__all__ = ["_state_passing_fwd"]
