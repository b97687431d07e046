"""Combined forward of the EMA chunked scan and its autograd entry point.

Mirrors kernels/ema_kernels/ema_combined_fwd.py:12-76 of the reference (same names and
positional signatures).  The reference's EMAMatmulCombinedFn.backward returns None; here
it returns the gradients of the log-decay and of the input."""
import math

import torch

from kernels import _lib


def _ema_matmul_scan_combined_fwd(A_ema, X_ema, chunk_size, dtype=torch.float32, return_prev128=False,
                                  kernel_events=None, prepare_backward=False):
    """A_ema: (B, L) or (b, L, nh) float32 log-decay; X_ema: (B, L, T) or (b, L, nh, d).

    Returns (out, dA_cumsum (N, C, Q), states entering each chunk (N, C, T), final (N, T)).
    `dtype` is the dtype of the returned chunk states (computed in float32).  With
    return_prev128 a fifth value follows: the states entering each 128-row chunk, which the
    backward accepts to skip their recomputation (None when chunk_size is not a multiple
    of 128).  kernel_events: optional (start, stop) torch.cuda.Event pair recorded around the
    kernel that reads x.  prepare_backward (chunk_size a multiple of 128): a sixth value
    follows, the workspace of the backward pass, prepared by this pass's set-up launch
    (_lib.BackwardWorkspace; kernels.ema_seq.ema_seq_bwd takes it)."""
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
    assert ws_bytes > 0, "unsupported shape"
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    bwd_ws = None
    if prepare_backward and chunk_size % 128 == 0:
        bwd_ws = _lib.BackwardWorkspace(batch, nh, seqlen, token_dim, dev)
    with torch.cuda.device(dev):
        st = L.ema_fwd(
            *a_args, *x_args, _lib.dtype_code(x), *y_args, cs.data_ptr(), prev.data_ptr(),
            final.data_ptr(), None if prev128 is None or prev128 is prev else prev128.data_ptr(),
            ws.data_ptr(), ws_bytes, None if bwd_ws is None else bwd_ws.buf.data_ptr(),
            0 if bwd_ws is None else bwd_ws.nbytes, batch, nh, seqlen, token_dim, chunk_size,
            _lib.stream_ptr(dev), *_lib.event_ptrs(kernel_events),
        )
    _lib.check(st, "_ema_matmul_scan_combined_fwd")
    if dtype != torch.float32:
        prev = prev.to(dtype)
    res = (out, cs, prev, final) + ((prev128,) if return_prev128 else ())
    return res + ((bwd_ws,) if prepare_backward else ())


def _unchunk_dA(ddA, A_like, seqlen):
    """(N, C, Q) chunked log-decay gradient -> the layout of A."""
    N = ddA.shape[0]
    flat = ddA.reshape(N, -1)[:, :seqlen]
    if A_like.dim() == 2:
        return flat
    b, _, nh = A_like.shape
    return flat.reshape(b, nh, seqlen).permute(0, 2, 1)


class EMAMatmulCombinedFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, A_ema, X_ema, chunk_size):
        wants_grad = any(ctx.needs_input_grad)
        out, dA_cumsum, states, final_states, prev128, bwd_ws = _ema_matmul_scan_combined_fwd(
            A_ema, X_ema, chunk_size=chunk_size, return_prev128=True, prepare_backward=True
        ) if wants_grad else _ema_matmul_scan_combined_fwd(
            A_ema, X_ema, chunk_size=chunk_size, return_prev128=True) + (None,)
        ctx.save_for_backward(out, dA_cumsum, states, final_states, A_ema, X_ema)
        ctx.prev128 = prev128  # a small float32 tensor the backward reuses; not an input or output
        ctx.bwd_ws = bwd_ws    # the backward's workspace, set up by the forward's set-up launch
        ctx.chunk_size = chunk_size
        return out

    @staticmethod
    def backward(ctx, dout, *args):
        from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_chunk_scan_combined_bwd

        out, dA_cumsum, states, final_states, A_ema, X_ema = ctx.saved_tensors
        if ctx.prev128 is not None:
            # the same single-pass kernel through the entry point that returns the gradient of the
            # log-decay in the layout of A itself: nothing to rearrange afterwards
            from kernels.ema_seq import ema_seq_bwd

            dx, dA, _ = ema_seq_bwd(dout, X_ema, A_ema, ctx.prev128, form="log_decay", workspace=ctx.bwd_ws)
            return dA, dx, None
        dx, ddA = _ema_chunk_scan_combined_bwd(dout, X_ema, A_ema, ctx.chunk_size)
        dA = _unchunk_dA(ddA, A_ema, X_ema.shape[1])
        return dA, dx, None


def ema_matmul_scan_combined(A_ema, X_ema, chunk_size):
    return EMAMatmulCombinedFn.apply(A_ema, X_ema, chunk_size)
