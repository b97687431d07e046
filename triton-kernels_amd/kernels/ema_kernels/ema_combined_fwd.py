"""Combined forward of the EMA chunked scan and its autograd entry point.

Mirrors kernels/ema_kernels/ema_combined_fwd.py:12-76 of the reference (same names and
positional signatures).  The reference's EMAMatmulCombinedFn.backward returns None; here
it returns the gradients of the log-decay and of the input."""
import math

import torch

from kernels import _lib


def _ema_matmul_scan_combined_fwd(A_ema, X_ema, chunk_size, dtype=torch.float32, return_prev128=False,
                                  kernel_events=None):
    """A_ema: (B, L) or (b, L, nh) float32 log-decay; X_ema: (B, L, T) or (b, L, nh, d).

    Returns (out, dA_cumsum (N, C, Q), states entering each chunk (N, C, T), final (N, T)).
    `dtype` is the dtype of the returned chunk states (computed in float32).  With
    return_prev128 a fifth value follows: the states entering each 128-row chunk, which the
    backward accepts to skip their recomputation (None when chunk_size is not a multiple
    of 128).  kernel_events: optional (start, stop) torch.cuda.Event pair recorded around the
    kernel that reads x."""
    dev = _lib.require_gpu(A_ema, X_ema)
    x, x_args, batch, nh, seqlen, token_dim = _lib.seq_view(X_ema)
    a_args, a_batch, a_nh, a_len = _lib.decay_view(A_ema)
    assert (a_batch, a_nh, a_len) == (batch, nh, seqlen), "A and X disagree on (batch, heads, seqlen)"
    nchunks = math.ceil(seqlen / chunk_size)
    N = batch * nh
    out = torch.empty(x.shape, device=dev, dtype=x.dtype)
    _, y_args, *_ = _lib.seq_view(out)
    cs = torch.empty(N, nchunks, chunk_size, device=dev, dtype=torch.float32)
    prev = torch.empty(N, nchunks, token_dim, device=dev, dtype=torch.float32)
    final = torch.empty(N, token_dim, device=dev, dtype=torch.float32)
    prev128 = None
    if return_prev128 and chunk_size % 128 == 0:
        prev128 = prev if chunk_size == 128 else torch.empty(
            N, math.ceil(seqlen / 128), token_dim, device=dev, dtype=torch.float32)
    L = _lib.lib()
    ws_bytes = L.ema_fwd_workspace_bytes(batch, nh, seqlen, token_dim, chunk_size)
    ws, ready = _lib.workspace(dev, ws_bytes, batch, nh, seqlen, token_dim)
    with torch.cuda.device(dev):
        st = L.ema_fwd(
            *a_args, *x_args, _lib.dtype_code(x), *y_args, cs.data_ptr(), prev.data_ptr(),
            final.data_ptr(), None if prev128 is None or prev128 is prev else prev128.data_ptr(),
            ws.data_ptr(), ws.numel(), ready, batch, nh, seqlen, token_dim, chunk_size,
            _lib.stream_ptr(dev), *_lib.event_ptrs(kernel_events),
        )
    _lib.check(st, "_ema_matmul_scan_combined_fwd")
    if dtype != torch.float32:
        prev = prev.to(dtype)
    return (out, cs, prev, final) + ((prev128,) if return_prev128 else ())


def _unchunk_dA(ddA, A_like, seqlen):
    """(N, C, Q) chunked log-decay gradient -> the layout of A."""
    N = ddA.shape[0]
    flat = ddA.reshape(N, -1)[:, :seqlen]
    if A_like.dim() == 2:
        return flat
    b, _, nh = A_like.shape
    return flat.reshape(b, nh, seqlen).permute(0, 2, 1)


class EMAMatmulCombinedFn(torch.autograd.Function):
    """forward / backward of ema_matmul_scan_combined.  For chunk sizes that are multiples of 128
    both directions are one kernel launch each plus the small reduction of the log-decay
    gradient: the scan does not depend on the chunking, so the sequence-level entry points are
    used and the chunked intermediates of the reference's forward (which its backward, being
    unimplemented, never read) are not formed."""

    @staticmethod
    def forward(ctx, A_ema, X_ema, chunk_size):
        ctx.chunk_size = chunk_size
        if chunk_size % 128 == 0:
            from kernels.ema_seq import ema_seq_fwd

            out, _, prev128 = ema_seq_fwd(A_ema, X_ema, form="log_decay")
            ctx.save_for_backward(A_ema, X_ema, prev128)
            return out
        out, dA_cumsum, states, final_states = _ema_matmul_scan_combined_fwd(A_ema, X_ema, chunk_size=chunk_size)
        ctx.save_for_backward(A_ema, X_ema)
        return out

    @staticmethod
    def backward(ctx, dout, *args):
        if len(ctx.saved_tensors) == 3:
            # the gradient of the log-decay comes back in the layout of A itself: nothing to
            # rearrange afterwards
            from kernels.ema_seq import ema_seq_bwd

            A_ema, X_ema, prev128 = ctx.saved_tensors
            dx, dA, _ = ema_seq_bwd(dout, X_ema, A_ema, prev128, form="log_decay")
            return dA, dx, None
        from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_chunk_scan_combined_bwd

        A_ema, X_ema = ctx.saved_tensors
        dx, ddA = _ema_chunk_scan_combined_bwd(dout, X_ema, A_ema, ctx.chunk_size)
        dA = _unchunk_dA(ddA, A_ema, X_ema.shape[1])
        return dA, dx, None


def ema_matmul_scan_combined(A_ema, X_ema, chunk_size):
    return EMAMatmulCombinedFn.apply(A_ema, X_ema, chunk_size)
