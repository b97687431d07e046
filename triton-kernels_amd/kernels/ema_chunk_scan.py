"""kernels/ema_chunk_scan.py of the reference (same kernel as its
kernels/mamba_kernels/mamba_scan_fwd.py): the chunk scan."""
from kernels.mamba_kernels.mamba_scan_fwd import _chunk_scan_fwd

__all__ = ["_chunk_scan_fwd"]
