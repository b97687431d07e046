"""ctypes binding of libema_hip.so (the C ABI declared in include/ema_hip.h).

The library is the only implementation: if it is missing, or no GPU is present, the
operators raise.  There is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# EMA_HIP_LIB names another build of the library (same ABI), e.g. one with a different tile shape
LIB_PATH = os.environ.get("EMA_HIP_LIB") or os.path.join(os.path.dirname(_HERE), "lib", "libema_hip.so")

EMA_F32, EMA_BF16 = 0, 1
EMA_FORM_LOG_DECAY, EMA_FORM_PROBABILITY = 0, 1
EMA_MAX_CHUNK = 1024

_I = c_int64
_P = c_void_p
_SEQ = [_P, _I, _I, _I]  # pointer + (batch, position, head) strides
_IDS = [_P, _I, _I]  # seq_idx pointer (may be null) + (batch, position) strides

_SIGNATURES = {
    "ema_version": (c_char_p, []),
    "ema_status_string": (c_char_p, [c_int]),
    "ema_chunk_cumsum_fwd": (c_int, _SEQ + [_P, _I, _I, _I, _I, _P]),
    "ema_chunk_state_fwd": (c_int, _SEQ + [c_int, _P, _P, _I, _I, _I, _I, _I, _P]),
    "ema_state_passing_fwd": (c_int, [_P, _P, _I, _I, _P, _P, _I, _I, _I, _P]),
    "ema_scan_fwd": (c_int, _SEQ + [c_int, _P, _P] + _SEQ + [_I, _I, _I, _I, _I, _P]),
    "ema_fwd_workspace_bytes": (c_size_t, [_I, _I, _I, _I, _I]),
    "ema_workspace_clear": (c_int, [_P, c_size_t, _P]),
    "ema_stream_copy": (c_int, [_P, _P, _P, c_size_t, _P]),
    "ema_tile_pattern_copy": (c_int, [_P, _P, _P, _I, _I, _I, c_int, _P]),
    "ema_fwd": (c_int, _SEQ + _SEQ + [c_int] + _SEQ + [_P, _P, _P, _P, _P, c_size_t, c_int, _I, _I, _I, _I, _I, _P, _P, _P]),
    "ema_chunk_scan_bwd_dstates": (c_int, _SEQ + [c_int, _P, _P, _I, _I, _I, _I, _I, _P]),
    "ema_state_passing_bwd_workspace_bytes": (c_size_t, [_I, _I, _I]),
    "ema_state_passing_bwd": (c_int, [_P, _P, _I, _I, _P, _P, _P, _P, c_size_t, _I, _I, _I, _P]),
    "ema_chunk_scan_chunk_state_bwd_dx": (c_int, _SEQ + [c_int, _P, _P] + _SEQ + [_I, _I, _I, _I, _I, _P]),
    "ema_chunk_state_bwd_db": (c_int, _SEQ + [c_int, _P, _P, _P, c_int, _I, _I, _I, _I, _I, _P]),
    "ema_chunk_scan_bwd_dc": (c_int, _SEQ + [c_int, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "ema_chunk_scan_bwd_ddAcs_workspace_bytes": (c_size_t, [_I, _I, _I, _I, _I, c_int]),
    "ema_chunk_scan_bwd_ddAcs": (c_int, _SEQ + _SEQ + [c_int, _P, _P, _P, c_size_t, _I, _I, _I, _I, _I, _P]),
    "ema_bwd_dx_dA_fused_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "ema_bwd_dx_dA_fused": (c_int, _SEQ + _SEQ + [c_int, _P, _P, _P] + _SEQ + [_P] + _SEQ + [_P, c_size_t, _I, _I, _I, _I, _P]),
    "ema_bwd_workspace_bytes": (c_size_t, [_I, _I, _I, _I, _I]),
    "ema_bwd": (c_int, _SEQ + _SEQ + _SEQ + [_P, c_int] + _SEQ + [_P] + _SEQ + [_P, c_size_t, c_int, _I, _I, _I, _I, _I, _P, _P, _P]),
    "ema_seq_fwd_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "ema_seq_bwd_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "ema_seq_fwd": (c_int, [c_int] + _SEQ + _SEQ + [c_int] + _SEQ + [_P, _P, _P, _P, c_size_t, c_int, _I, _I, _I, _I, _P, _P, _P]),
    "ema_seq_bwd": (c_int, [c_int] + _SEQ + _SEQ + _SEQ + [_P, _P, c_int] + _SEQ + _SEQ + [_P, _P, c_size_t, c_int, _I, _I, _I, _I, _P, _P, _P]),
    "ema_seq_fwd_static_max_workspace_bytes": (c_size_t, []),
    "ema_seq_fwd_static_init": (c_int, []),
    "ema_seq_fwd_static_error": (c_int, [_P, _P]),
    "ema_seq_fwd_static_reset": (c_int, [_P]),
    "ema_seq_fwd_static": (c_int, [c_int] + _SEQ + _SEQ + [c_int] + _SEQ + [_P, _P, _P, _I, _I, _I, _I, _P]),
    # SSD forward stages (include/ssd_hip.h)
    "ssd_chunk_cumsum_fwd": (c_int, [_P, c_int, _I, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, c_int, c_float, c_float, _P]),
    "ssd_chunk_state_fwd": (c_int, _SEQ + _SEQ + [c_int, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I] + _IDS + [_P]),
    "ssd_state_passing_fwd": (c_int, [_P, _P, _I, _I, _I, _P, _P, c_int, _P, _I, _I, _I, _I] + _IDS + [_I, _I, _P]),
    "ssd_chunk_state_passing_fwd": (c_int, _SEQ + _SEQ + [c_int, _P, _P, _P, _P, c_int, _P, _I, _I, _I, _I, _I, _I, _I, _P]),
    "ssd_bmm_chunk_fwd": (c_int, _SEQ + _SEQ + [c_int, _P, c_int, _I, _I, _I, _I, _I] + _IDS + [_P]),
    "ssd_chunk_scan_fwd": (c_int, [_P] + _SEQ + _SEQ + [c_int, _P, _P] + _SEQ + [_P, c_int, _P, c_int] + _SEQ + [_P, _I, _I, _I, _I, _I, _I, _I] + _IDS + [_P]),
    # SSD backward stages
    "ssd_chunk_scan_bwd_dstates": (c_int, _SEQ + _SEQ + [c_int, _P, _P, c_int, _I, _I, _I, _I, _I, _I, _I] + _IDS + [_P]),
    "ssd_state_passing_bwd_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "ssd_chunk_scan_state_passing_bwd_workspace_bytes": (c_size_t, [_I, _I, _I]),
    "ssd_chunk_scan_state_passing_bwd": (c_int, _SEQ + _SEQ + [c_int, _P, _P, c_int, _P, _P, c_int, _P, _P, _P, c_size_t,
                                                  _I, _I, _I, _I, _I, _I, _I, _P]),
    "ssd_state_passing_bwd": (c_int, [_P, c_int, _P, _I, _I, _I, _P, c_int, _P, _P, c_int, _P, _P, _P, c_size_t, _I, _I, _I, _I] + _IDS + [_I, _I, _P]),
    "ssd_chunk_state_bwd_db": (c_int, _SEQ + [c_int, _P, _P, _P, c_int] + _SEQ + [_P, _P, _I, _I, _I, _I, _I, _I, _I] + _IDS + [_P]),
    "ssd_chunk_scan_bwd_dc": (c_int, _SEQ + [c_int, _P, _P, c_int] + _SEQ + [_P, _P, _I, _I, _I, _I, _I, _I, _I] + _IDS + [_P]),
    "ssd_chunk_scan_chunk_state_bwd_dx": (c_int, [_P] + _SEQ + _SEQ + [c_int, _P, _P] + _SEQ + [_P, c_int, _P, c_int] + _SEQ + [_P, _I, _I, _I, _I, _I, _I, _I] + _IDS + [_P, _P]),
    "ssd_chunk_scan_chunk_state_bwd_dx_dD_slots": (c_int64, [c_int, _I, _I, _I]),
    "ssd_chunk_scan_bwd_ddAcs_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "ssd_chunk_scan_bwd_ddAcs": (c_int, _SEQ + _SEQ + [c_int, _P, _P, _P, _P, _P, c_size_t, _I, _I, _I, _I, _I, _I, _P]),
    "ssd_chunk_state_varlen": (c_int, [_P, _I, _I, _P, _I, _I, c_int, _P, _P, _P, c_int, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]),
}

_lib = None


def exported_symbols():
    """Names every build of the library must export (one per declaration in ema_hip.h)."""
    return sorted(_SIGNATURES)


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python triton-kernels_amd/build.py` "
                "(the EMA operators have no fallback implementation)"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


_ERRORS = {
    -1: (ValueError, "null pointer"),
    -2: (AssertionError, "bad shape"),
    -3: (AssertionError, "dim, stride or pointer not 16-byte aligned"),
    -4: (TypeError, "unsupported dtype"),
    -5: (NotImplementedError, "unsupported"),
    -6: (RuntimeError, "kernel launch failed"),
    -7: (ValueError, "problem exceeds the fixed scratch of the allocation-free entry point"),
}


def check(status: int, what: str) -> None:
    if status != 0:
        exc, msg = _ERRORS.get(status, (RuntimeError, f"status {status}"))
        raise exc(f"{what}: {msg}")


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return EMA_F32
    if t.dtype == torch.bfloat16:
        return EMA_BF16
    raise TypeError(f"EMA kernels take float32 or bfloat16 sequences, got {t.dtype}")


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError("EMA kernels run on the GPU only (tensor is on %s)" % dev)
    for t in tensors:
        if t is not None and t.device != dev:
            raise AssertionError("all tensors must be on the same device")
    return dev


def stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def seq_view(x: torch.Tensor):
    """(tensor with unit feature stride, [ptr, sb, sl, sh], batch, nheads, L, T) of a flat
    (B, L, T) or headed (b, L, nh, d) sequence tensor."""
    assert x.dim() in (3, 4), "expected (B, L, T) or (b, L, nh, d)"
    if x.stride(-1) != 1:
        x = x.contiguous()
    if x.dim() == 3:
        B, L, T = x.shape
        return x, [x.data_ptr(), x.stride(0), x.stride(1), 0], B, 1, L, T
    b, L, nh, d = x.shape
    return x, [x.data_ptr(), x.stride(0), x.stride(1), x.stride(2)], b, nh, L, d


def decay_view(A: torch.Tensor):
    """([ptr, sb, sl, sh], batch, nheads, L) of a flat (B, L) or headed (b, L, nh) log-decay."""
    assert A.dim() in (2, 3), "expected (B, L) or (b, L, nh)"
    assert A.dtype == torch.float32, "log-decay must be float32"
    if A.dim() == 2:
        return [A.data_ptr(), A.stride(0), A.stride(1), 0], A.shape[0], 1, A.shape[1]
    return [A.data_ptr(), A.stride(0), A.stride(1), A.stride(2)], A.shape[0], A.shape[2], A.shape[1]


def event_ptrs(events):
    """(start, stop) raw hipEvent_t handles of a pair of torch.cuda.Event (timing enabled), or
    (None, None).  The events must have been recorded once so that their handles exist."""
    if events is None:
        return None, None
    return events[0].cuda_event, events[1].cuda_event


def strided4(t: torch.Tensor):
    """(tensor with unit last stride, [ptr, s0, s1, s2]) of a 4-d tensor (b, l, h, inner)."""
    assert t.dim() == 4
    if t.stride(-1) != 1:
        t = t.contiguous()
    return t, [t.data_ptr(), t.stride(0), t.stride(1), t.stride(2)]


def f32c(t: torch.Tensor) -> torch.Tensor:
    """Dense float32 view/copy of a chunked intermediate."""
    if t.dtype != torch.float32:
        t = t.float()
    return t.contiguous()


# ---------------------------------------------------------------------------------------------
# Workspace of the single-pass entry points.  The library tags every word it writes to the
# chained part of a workspace with the epoch of the call, so a buffer that was zero-filled once
# serves every later call without being cleared (workspace_ready = 1: the call is the tile kernel
# alone).  Two calls that overlap in time must not share a buffer (they would draw tiles from one
# ticket counter), so the wrappers keep one buffer per (device, stream, problem shape): calls on
# one stream are ordered, calls on different streams get different buffers.  A buffer is created
# at the largest size any entry point needs for its shape with chunk sizes that are multiples of
# 128, and never grows or moves afterwards; a call that needs more (the staged forward with a
# small chunk size, which does not use the chained part) gets a buffer of its own.  Buffers handed
# out while a HIP graph is being captured are pinned: the graph holds their address, so they are
# never dropped.  private_workspaces(True) switches to a fresh, cleared buffer per call.
# ---------------------------------------------------------------------------------------------
HEADER_BYTES = 256
_RECLEAR_AFTER = 1 << 29  # calls; the epoch tag wraps at 2**30
_MAX_SHARED = 16          # unpinned buffers kept (the least recently created goes first)


class _Shared:
    __slots__ = ("buf", "calls", "pinned")

    def __init__(self, buf):
        self.buf, self.calls, self.pinned = buf, 0, False


_shared = {}  # (device index, stream, N, tiles, dim) -> _Shared
_private = False


def private_workspaces(on: bool) -> None:
    global _private
    _private = bool(on)


def _clear(buf: torch.Tensor, dev: torch.device) -> None:
    with torch.cuda.device(dev):
        check(lib().ema_workspace_clear(buf.data_ptr(), buf.numel(), stream_ptr(dev)), "ema_workspace_clear")


def _shared_bytes(batch: int, nh: int, L: int, T: int) -> int:
    """Largest workspace of the four single-pass entry points for this shape (chunk 128)."""
    h = lib()
    return max(h.ema_fwd_workspace_bytes(batch, nh, L, T, 128), h.ema_bwd_workspace_bytes(batch, nh, L, T, 128),
               h.ema_seq_fwd_workspace_bytes(batch, nh, L, T), h.ema_seq_bwd_workspace_bytes(batch, nh, L, T))


def workspace(dev: torch.device, nbytes: int, batch: int, nh: int, L: int, T: int):
    """(uint8 buffer of at least nbytes, workspace_ready flag) for one call on the current
    stream of `dev` of a single-pass entry point on a (batch, L, nh, T) problem."""
    assert nbytes > 0, "unsupported shape"
    capturing = torch.cuda.is_current_stream_capturing()
    key = (dev.index, stream_ptr(dev), batch * nh, -(-L // 128), T)
    entry = _shared.get(key)
    if _private or (entry is None and capturing) or (entry is not None and entry.buf.numel() < nbytes):
        # under capture nothing persistent may be created; an oversized request is served apart
        return torch.empty(nbytes, dtype=torch.uint8, device=dev), 0
    if entry is None:
        size = _shared_bytes(batch, nh, L, T)
        if size < nbytes:
            return torch.empty(nbytes, dtype=torch.uint8, device=dev), 0
        unpinned = [k for k, e in _shared.items() if not e.pinned]
        for k in unpinned[: max(0, len(unpinned) - _MAX_SHARED + 1)]:
            del _shared[k]
        entry = _shared[key] = _Shared(torch.empty(size, dtype=torch.uint8, device=dev))
        _clear(entry.buf, dev)
    elif entry.calls >= _RECLEAR_AFTER and not capturing:
        _clear(entry.buf, dev)
        entry.calls = 0
    if capturing:
        entry.pinned = True
    entry.calls += 1
    return entry.buf, 1


def chain_error(buf: torch.Tensor) -> bool:
    """Whether a tile's bounded wait ran out in some call on this workspace (synchronises)."""
    return bool(buf[:HEADER_BYTES].view(torch.int32)[3].item())


def check_chain_errors(device=None) -> None:
    """Raises if any call since the last check gave up waiting for a predecessor tile (the
    outputs of that call hold NaN).  Reads one word per device back: call it where the program
    synchronises anyway, not between kernels.  The workspace is cleared after a report."""
    for key, entry in list(_shared.items()):
        index = key[0]
        if device is not None and torch.device(device).index not in (None, index):
            continue
        if chain_error(entry.buf):
            # the buffer belongs to another stream, maybe: nothing may be in flight while it is cleared
            torch.cuda.synchronize(entry.buf.device)
            _clear(entry.buf, entry.buf.device)
            torch.cuda.synchronize(entry.buf.device)
            entry.calls = 0
            raise RuntimeError(
                f"EMA chained scan on cuda:{index}: a tile gave up waiting for its predecessor; the "
                "results of that call are NaN (overlapping calls on one workspace, or a workspace "
                "that was not ready)")


def state_tensor(t: torch.Tensor, like: torch.Tensor = None):
    """(dense tensor, dtype code) of a carried-state tensor: kept in bfloat16 when the kernels that
    read it compute in bfloat16 (`like`, None for any), brought to float32 otherwise."""
    if t.dtype == torch.bfloat16 and (like is None or like.dtype == torch.bfloat16):
        return t.contiguous(), EMA_BF16
    return f32c(t), EMA_F32


def seq_ids(seq_idx, batch: int, seqlen: int, dev: torch.device):
    """(int32 tensor kept alive by the caller or None, [ptr, sb, sl]) of the ids of a packed batch."""
    if seq_idx is None:
        return None, [None, 0, 0]
    assert seq_idx.shape == (batch, seqlen)
    if seq_idx.device != dev:
        raise AssertionError("all tensors must be on the same device")
    if seq_idx.dtype != torch.int32:
        seq_idx = seq_idx.to(torch.int32)
    return seq_idx, [seq_idx.data_ptr(), seq_idx.stride(0), seq_idx.stride(1)]
