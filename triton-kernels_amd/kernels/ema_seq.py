"""Sequence-level EMA scan on the caller's raw tensors: one pass forward, one pass backward.

What the reference leaves to torch around its kernels is folded into the loads and stores of
the single-pass kernels here:

  * the probability form  y[t] = (1 - p[t]) * y[t-1] + p[t] * x[t]  without forming
    A = log(1 - p) and X = p * x first (kernels/benchmarks/ema_bench.py:135-136) and with the
    gradient returned for p itself (the reference's dP = -dA * exp(A) is commented out,
    kernels/tests/ema_bwd/_ema_full_bwd.py:128-130);
  * the gradient of the coefficient in the coefficient's own (b, L, nh) layout instead of the
    chunked (B, C, Q) one (rearranged in torch at _ema_full_bwd.py:71);
  * an initial state, the final state and the gradients through both, which the reference's
    launchers reject (kernels/ema_kernels/ema_state_pass.py:129-130,
    kernels/ema_kernels_bwd/ema_state_passing_bwd_dstates.py:120-122).

x is (B, L, T) or (b, L, nh, d), float32 or bfloat16; the coefficient (B, L) or (b, L, nh)
float32; states (B, T) or (b, nh, d) float32.
"""
import torch

from kernels import _lib

FORMS = {"log_decay": _lib.EMA_FORM_LOG_DECAY, "probability": _lib.EMA_FORM_PROBABILITY}


def _state_2d(s, batch, nh, T, name):
    """(N, T) float32 contiguous view of a boundary state, N = batch * nh."""
    expect = (batch, T) if nh == 1 and s.dim() == 2 else (batch, nh, T)
    assert tuple(s.shape) == expect, f"{name} must have shape {expect}, got {tuple(s.shape)}"
    return _lib.f32c(s).reshape(batch * nh, T)


def ema_seq_fwd(coef, x, form="log_decay", initial_states=None, kernel_events=None, workspace=None):
    """Forward pass.  Returns (y, final_states, prev128); prev128 (N, ceil(L/128), T) float32 is
    what ema_seq_bwd needs from the forward.  workspace: optional (uint8 buffer, ready flag) to
    use instead of the device's shared one."""
    dev = _lib.require_gpu(x, coef)
    x, xs, batch, nh, L, T = _lib.seq_view(x)
    cs_, cb, cnh, cL = _lib.decay_view(coef)
    assert (cb, cnh, cL) == (batch, nh, L), "coefficient and x disagree in (batch, heads, length)"
    lib = _lib.lib()
    N = batch * nh
    y = torch.empty_like(x)
    _, ys, *_ = _lib.seq_view(y)
    final = torch.empty(N, T, dtype=torch.float32, device=dev)
    prev128 = torch.empty(N, -(-L // 128), T, dtype=torch.float32, device=dev)
    init = None if initial_states is None else _state_2d(initial_states, batch, nh, T, "initial_states")
    nbytes = lib.ema_seq_fwd_workspace_bytes(batch, nh, L, T)
    ws, ready = _lib.workspace(dev, nbytes, batch, nh, L, T) if workspace is None else workspace
    assert ws.numel() >= nbytes
    ev0, ev1 = _lib.event_ptrs(kernel_events)
    with torch.cuda.device(dev):
        _lib.check(
            lib.ema_seq_fwd(FORMS[form], *cs_, *xs, _lib.dtype_code(x), *ys,
                            None if init is None else init.data_ptr(), final.data_ptr(),
                            prev128.data_ptr(), ws.data_ptr(), ws.numel(), ready, batch, nh, L, T,
                            _lib.stream_ptr(dev), ev0, ev1),
            "ema_seq_fwd")
    final = final.reshape(batch, T) if x.dim() == 3 else final.reshape(batch, nh, T)
    return y, final, prev128


def ema_seq_bwd(dy, x, coef, prev128, form="log_decay", dfinal_states=None, want_dinit=False,
                kernel_events=None, workspace=None):
    """Backward pass.  Returns (dx, dcoef, dinitial_states or None).  workspace: optional
    (uint8 buffer, ready flag) to use instead of the device's shared one."""
    dev = _lib.require_gpu(dy, x, coef, prev128)
    x, xs, batch, nh, L, T = _lib.seq_view(x)
    if dy.dtype != x.dtype:
        dy = dy.to(x.dtype)
    dy, ds, *_ = _lib.seq_view(dy)
    assert dy.shape == x.shape
    cs_, cb, cnh, cL = _lib.decay_view(coef)
    assert (cb, cnh, cL) == (batch, nh, L)
    lib = _lib.lib()
    N = batch * nh
    assert prev128.shape == (N, -(-L // 128), T) and prev128.dtype == torch.float32 and prev128.is_contiguous()
    dx = torch.empty_like(x)
    _, dxs, *_ = _lib.seq_view(dx)
    dcoef = torch.empty_like(coef)
    dcs, *_ = _lib.decay_view(dcoef)
    dfin = None if dfinal_states is None else _state_2d(dfinal_states, batch, nh, T, "dfinal_states")
    dinit = torch.empty(N, T, dtype=torch.float32, device=dev) if want_dinit else None
    nbytes = lib.ema_seq_bwd_workspace_bytes(batch, nh, L, T)
    ws, ready = _lib.workspace(dev, nbytes, batch, nh, L, T) if workspace is None else workspace
    assert ws.numel() >= nbytes
    ev0, ev1 = _lib.event_ptrs(kernel_events)
    with torch.cuda.device(dev):
        _lib.check(
            lib.ema_seq_bwd(FORMS[form], *ds, *xs, *cs_, prev128.data_ptr(),
                            None if dfin is None else dfin.data_ptr(), _lib.dtype_code(x), *dxs, *dcs,
                            None if dinit is None else dinit.data_ptr(), ws.data_ptr(), ws.numel(),
                            ready, batch, nh, L, T, _lib.stream_ptr(dev), ev0, ev1),
            "ema_seq_bwd")
    if dinit is not None:
        dinit = dinit.reshape(batch, T) if x.dim() == 3 else dinit.reshape(batch, nh, T)
    return dx, dcoef, dinit


class EMASeqFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, coef, x, initial_states, form):
        y, final, prev128 = ema_seq_fwd(coef, x, form, initial_states)
        ctx.save_for_backward(coef, x, prev128)
        ctx.form = form
        ctx.has_init = initial_states is not None
        ctx.init_dtype = None if initial_states is None else initial_states.dtype
        ctx.set_materialize_grads(False)  # an unused final state brings None, not a tensor of zeros
        return y, final

    @staticmethod
    def backward(ctx, dy, dfinal):
        coef, x, prev128 = ctx.saved_tensors
        if dy is None:
            dy = torch.zeros_like(x)
        dx, dcoef, dinit = ema_seq_bwd(dy.contiguous(), x, coef, prev128, ctx.form,
                                       dfinal_states=dfinal, want_dinit=ctx.has_init)
        if dinit is not None:
            dinit = dinit.to(ctx.init_dtype)
        return dcoef, dx, dinit, None


def pack_log_decay(A, seq_idx):
    """Log-decay of several sequences packed along the length axis: wherever seq_idx (batch, L)
    changes, the state must not carry over, which is a decay of exp(-inf) = 0 at the first
    position of the new sequence (what the reference's seq_idx arguments ask of its kernels, e.g.
    kernels/ema_chunk_state.py:500-604: scale = where(seq_idx_k == seq_idx_last, exp(...), 0)).
    A is (B, L) or (b, L, nh); returns a tensor of A's shape.  The gradient that reaches the
    masked positions is zero."""
    assert seq_idx.shape == A.shape[:2], "seq_idx must be (batch, seqlen)"
    start = torch.zeros_like(seq_idx, dtype=torch.bool)
    start[:, 1:] = seq_idx[:, 1:] != seq_idx[:, :-1]
    if A.dim() == 3:
        start = start[..., None]
    return torch.where(start, torch.full_like(A, float("-inf")), A)


def pack_probability(p, seq_idx):
    """Probabilities of several sequences packed along the length axis: the kernels drop the
    state at a position whose probability carries a set sign bit, so p is negated (0 becomes
    -0.0) at the first position of each new sequence.  Autograd through the negation returns the
    gradient with respect to p itself."""
    assert seq_idx.shape == p.shape[:2], "seq_idx must be (batch, seqlen)"
    start = torch.zeros_like(seq_idx, dtype=torch.bool)
    start[:, 1:] = seq_idx[:, 1:] != seq_idx[:, :-1]
    if p.dim() == 3:
        start = start[..., None]
    return torch.where(start, -p, p)


def ema_seq_scan(coef, x, form="log_decay", initial_states=None, return_final_states=False, seq_idx=None):
    """Differentiable in coef, x and initial_states (and through the final states).  seq_idx
    (batch, L) marks packed sequences: the state is reset where it changes."""
    if seq_idx is not None:
        coef = pack_log_decay(coef, seq_idx) if form == "log_decay" else pack_probability(coef, seq_idx)
    y, final = EMASeqFn.apply(coef, x, initial_states, form)
    return (y, final) if return_final_states else y
