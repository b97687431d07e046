"""kernels/ema_bmm.py of the reference (same kernel as its kernels/mamba_kernels/mamba_bmm.py):
C B^T per chunk and group."""
from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd

__all__ = ["_bmm_chunk_fwd"]
