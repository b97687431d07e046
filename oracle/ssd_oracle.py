"""CPU oracle for the Mamba-2 SSD chunked scan (forward).

TEST INFRASTRUCTURE ONLY.  Nothing in the product path may import this module: only tests/,
__graft_entry__.smoke() and the cpu_baseline leg of bench.py use it, and only as the checker.

It restates, in plain PyTorch on the CPU, the arithmetic of the reference repository
kartiksrinivas007/triton-kernels (paths relative to its root):

* the sequential definition (the state-space recurrence)
      h_t = exp(dt_t * A) * h_{t-1} + dt_t * x_t (outer) B_t,   y_t = C_t . h_t + D * x_t,
  optionally gated y_t * z_t * sigmoid(z_t): ssd_step_ref,
  kernels/mamba_3_kernels/mamba_ssd_fwd.py:795-860, without its trapezoid / rotary / bias
  options and with the natural exponential that kernels/mamba_kernels/ uses (that file's
  own kernels use exp2);
* the five stages of the chunked forward in kernels/mamba_kernels/:
      chunk_cumsum   mamba_cumsum.py:32-128      (dt bias / softplus / clamp, dA = dt * A, cumsum)
      chunk_state    mamba_state_fwd.py:54-169   (B^T x weighted by exp(dA_last - dA_k) * dt_k)
      state_passing  mamba_state_pass.py:20-115  (inter-chunk recurrence, optional initial state)
      bmm_chunk      mamba_bmm.py                (C B^T per chunk and group)
      chunk_scan     mamba_scan_fwd.py:30-210    (C.prev * exp(dA_m) + causal (CB o decay o dt) x
                                                  + D x, z gate)

Layouts as in the reference: x (b, L, nh, hdim); dt (b, L, nh); A (nh,); B, C (b, L, g, dstate);
chunked dt / dA_cumsum (b, nh, C, Q); states (b, C, nh, hdim, dstate); CB (b, C, g, Q, Q).

Pinning status (tests/test_ssd_oracle.py): the reference holds no golden vectors for this path
and its comparison provider (mamba_ssm) is not installed, so the functions here are pinned by
what the mathematics fixes: a pure-Python brute force of the closed form on tiny inputs, the
composition of the five stages against the sequential recurrence for several chunk sizes
(chunk-size invariance), the reduction to the EMA scan for dstate = 1, B = C = 1, dt = 1 (whose
oracle is pinned separately), the segsum form of ssd_fwd_ref, and linearity in x.  Packed
batches (seq_idx, the HAS_SEQ_IDX branches of the same kernels) are pinned by running every
sequence of the pack on its own through the recurrence, and the backward stages with seq_idx
by autograd through the forward stages with seq_idx.  No function is left "parity unpinned".
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def _up(t):
    """float32 arithmetic as in the kernels; float64 inputs (used to pin the oracle) stay float64."""
    return t if t.dtype == torch.float64 else t.float()


def process_dt(dt, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """dt (b, L, nh) -> float32 after bias, softplus (identity above 20) and clamp;
    mamba_cumsum.py:72-80."""
    dt = _up(dt)
    if dt_bias is not None:
        dt = dt + _up(dt_bias)
    if dt_softplus:
        dt = torch.where(dt <= 20.0, F.softplus(dt), dt)
    return torch.clamp(dt, dt_limit[0], dt_limit[1])


def ssd_loop(x, dt, A, B, C, D=None, z=None, initial_states=None, seq_idx=None):
    """Sequential recurrence; dt is already processed (float32).  x (b,L,nh,p), dt (b,L,nh),
    A (nh,), B/C (b,L,g,n), D (nh,) or (nh,p), z like x, initial_states (b,nh,p,n).
    seq_idx (b, L) marks a packed batch: the state is cleared where the id changes, and the
    state a row starts with carries id 0 (mamba_state_pass.py:62).
    Returns (y (b,L,nh,p), final_states (b,nh,p,n)) in x's dtype / float32 arithmetic of x."""
    b, L, nh, p = x.shape
    g, n = B.shape[2], B.shape[3]
    rep = nh // g
    Bh = B.repeat_interleave(rep, dim=2)
    Ch = C.repeat_interleave(rep, dim=2)
    h = x.new_zeros(b, nh, p, n) if initial_states is None else initial_states.to(x.dtype).clone()
    y = torch.empty_like(x)
    cur = None if seq_idx is None else torch.zeros_like(seq_idx[:, 0])
    for t in range(L):
        if seq_idx is not None:
            h = h * (seq_idx[:, t] == cur).to(h.dtype)[:, None, None, None]
            cur = seq_idx[:, t]
        a = torch.exp(dt[:, t] * A)  # (b, nh)
        h = a[..., None, None] * h + (dt[:, t, :, None] * x[:, t])[..., None] * Bh[:, t, :, None, :]
        out = (h * Ch[:, t, :, None, :]).sum(-1)
        if D is not None:
            out = out + (D[None, :, None] if D.dim() == 1 else D[None]) * x[:, t]
        if z is not None:
            out = out * z[:, t] * torch.sigmoid(z[:, t])
        y[:, t] = out
    return y, h


# ------------------------------------------------------------------ the five stages


def _pad_seq(t, Q):
    pad = (-t.shape[1]) % Q
    if pad == 0:
        return t
    return torch.cat([t, t.new_zeros(t.shape[0], pad, *t.shape[2:])], 1)


def _seq_chunks(seq_idx, Q):
    """seq_idx (b, L) -> (ids (b, nc, Q) padded with -1, last (b, nc) = id of each chunk's last
    position inside the sequence, prev (b, nc) = last of the chunk before, 0 for the first)."""
    b, L = seq_idx.shape
    pad = (-L) % Q
    ids = torch.cat([seq_idx, seq_idx.new_full((b, pad), -1)], 1).reshape(b, -1, Q)
    nc = ids.shape[1]
    ends = torch.tensor([min((c + 1) * Q, L) - 1 for c in range(nc)])
    last = seq_idx[:, ends]
    prev = torch.cat([torch.zeros_like(last[:, :1]), last[:, :-1]], 1)
    return ids, last, prev


def chunk_cumsum(dt, A, Q, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """-> (dA_cumsum, dt_out), both (b, nh, C, Q) float32; positions past L hold dt = 0."""
    b, L, nh = dt.shape
    d = _pad_seq(process_dt(dt, dt_bias, dt_softplus, dt_limit), Q)
    valid = _pad_seq(torch.ones(b, L, nh, dtype=d.dtype), Q)
    d = d * valid
    C = d.shape[1] // Q
    d = d.reshape(b, C, Q, nh).permute(0, 3, 1, 2).contiguous()
    dA = d * _up(A)[None, :, None, None]
    return torch.cumsum(dA, -1), d


def _round(t, dtype):
    """The reference rounds some operands to the input type before its tl.dot; `dtype` None
    keeps full precision."""
    return t if dtype is None else t.to(dtype).to(t.dtype)


def chunk_state(B, x, dt, dA_cumsum, round_to=None, seq_idx=None):
    """states[b,c,h,p,n] = sum_k x[k,p] * B[k,n] * exp(min(dA_last - dA_k, 0)) * dt_k.
    With round_to the weighted B is rounded to that type first (mamba_state_fwd.py:118-119).
    With seq_idx, k only counts if its id equals the (non-negative) id of the chunk's last
    position (mamba_state_fwd.py:113)."""
    b, L, nh, p = x.shape
    _, _, C, Q = dt.shape
    g, n = B.shape[2], B.shape[3]
    xc = _pad_seq(_up(x), Q).reshape(b, C, Q, nh, p)
    Bc = _pad_seq(_up(B), Q).reshape(b, C, Q, g, n).repeat_interleave(nh // g, dim=3)
    w = torch.exp(torch.clamp(dA_cumsum[..., -1:] - dA_cumsum, max=0.0)) * dt  # (b, nh, C, Q)
    w = w.permute(0, 2, 3, 1)  # (b, C, Q, nh)
    if seq_idx is not None:
        ids, last, _ = _seq_chunks(seq_idx, Q)
        w = w * ((last[..., None] >= 0) & (ids == last[..., None])).to(w.dtype)[..., None]
    return torch.einsum("bcqhp,bcqhn->bchpn", xc, _round(Bc * w[..., None], round_to))


def _chunk_keep(seq_idx, chunk_size, dtype):
    """(b, nc) factor 1 / 0: the state survives a chunk whose last position has the id of the
    previous chunk's last position (id 0 before the first); mamba_state_pass.py:68-71."""
    _, last, prev = _seq_chunks(seq_idx, chunk_size)
    return (last == prev).to(dtype)


def state_passing(states, dA_chunk_cumsum, initial_states=None, seq_idx=None, chunk_size=None):
    """states (b, C, nh, dim), dA_chunk_cumsum (b, nh, C) -> (out (b, C, nh, dim) = state
    entering each chunk, final (b, nh, dim))."""
    b, C, nh, dim = states.shape
    outs = []
    s = states.new_zeros(b, nh, dim) if initial_states is None else _up(initial_states).clone()
    keep = None if seq_idx is None else _chunk_keep(seq_idx, chunk_size, states.dtype)
    for c in range(C):
        outs.append(s)
        scale = torch.exp(dA_chunk_cumsum[:, :, c])
        if keep is not None:
            scale = scale * keep[:, c, None]
        s = scale[..., None] * s + states[:, c]
    return torch.stack(outs, 1), s


def bmm_chunk(a, bm, Q, seq_idx=None):
    """out[b,c,g,m,k] = sum_n a[b,cQ+m,g,n] * bm[b,cQ+k,g,n]  (a = C, bm = B); with seq_idx, 0
    where the ids of m and k differ (mamba_bmm.py:70-73)."""
    b, L, g, n = a.shape
    ac = _pad_seq(_up(a), Q).reshape(b, -1, Q, g, n)
    bc = _pad_seq(_up(bm), Q).reshape(b, -1, Q, g, n)
    out = torch.einsum("bcmgn,bckgn->bcgmk", ac, bc)
    if seq_idx is not None:
        ids, _, _ = _seq_chunks(seq_idx, Q)
        out = out * (ids[..., :, None] == ids[..., None, :]).to(out.dtype)[:, :, None]
    return out


def chunk_scan(cb, x, dt, dA_cumsum, C, states, D=None, z=None, round_to=None, seq_idx=None):
    """out[m,p] = exp(dA_m) * sum_n C[m,n] prev[p,n]
                 + sum_{k<=m} cb[m,k] exp(min(dA_m - dA_k, 0)) dt_k x[k,p]  + D x,  then the z gate.
    Returns (out, out_x) with out_x the value before gating (None without z).  With round_to the
    weighted cb and prev are rounded to that type first (mamba_scan_fwd.py:97,137).  With seq_idx
    the first term only reaches the rows whose id equals that of the previous chunk's last
    position (mamba_scan_fwd.py:77-92); cb is expected to be masked already."""
    b, L, nh, p = x.shape
    _, _, nc, Q = dt.shape
    g, n = C.shape[2], C.shape[3]
    rep = nh // g
    xc = _pad_seq(_up(x), Q).reshape(b, nc, Q, nh, p)
    Cc = _pad_seq(_up(C), Q).reshape(b, nc, Q, g, n).repeat_interleave(rep, dim=3)
    cbh = _up(cb).repeat_interleave(rep, dim=2)  # (b, nc, nh, Q, Q)
    dA = dA_cumsum.permute(0, 2, 1, 3)  # (b, nc, nh, Q)
    dtc = dt.permute(0, 2, 1, 3)
    decay = torch.exp(torch.clamp(dA[..., :, None] - dA[..., None, :], max=0.0))
    mask = torch.tril(torch.ones(Q, Q, dtype=torch.bool))
    w = cbh * decay * dtc[..., None, :]
    w = _round(torch.where(mask, w, w.new_zeros(())), round_to)
    out = torch.einsum("bchmk,bckhp->bcmhp", w, xc)
    scale_m = torch.exp(dA)
    if seq_idx is not None:
        ids, _, prev = _seq_chunks(seq_idx, Q)
        scale_m = scale_m * (ids == prev[..., None]).to(scale_m.dtype)[:, :, None]
    out = out + torch.einsum("bcmhn,bchpn,bchm->bcmhp", Cc, _round(_up(states), round_to), scale_m)
    out = out.reshape(b, nc * Q, nh, p)[:, :L]
    if D is not None:
        out = out + (_up(D)[None, None, :, None] if D.dim() == 1 else _up(D)[None, None]) * _up(x)
    out_x = None
    if z is not None:
        out_x = out
        out = out * _up(z) * torch.sigmoid(_up(z))
    return out, out_x


def chunk_state_varlen(B, x, dt, dA_cumsum, cu_seqlens, chunk_states, round_to=None):
    """State at the end of each sequence of a packed batch without batch dimension
    (kernels/ema_chunk_state.py:500-604 of the reference).  B (L, g, n), x (L, nh, p), dt and
    dA_cumsum (nh, C, Q), chunk_states (C, nh, p, n) = state entering each chunk, cu_seqlens
    (nseq + 1).  For a sequence [start, end) with c the chunk of end - 1: the positions of the
    sequence inside chunk c, weighted by exp(min(dA[end-1] - dA[k], 0)) * dt[k] (:551-555), plus
    exp(dA[end-1]) * chunk_states[c] if the sequence began before chunk c (:563-568)."""
    L, nh, p = x.shape
    _, C, Q = dt.shape
    g, n = B.shape[1], B.shape[2]
    Bh = _up(B).repeat_interleave(nh // g, dim=1)  # (L, nh, n)
    xs = _up(x)
    out = []
    for s in range(len(cu_seqlens) - 1):
        start, end = int(cu_seqlens[s]), int(cu_seqlens[s + 1])
        c = (end - 1) // Q
        lo = max(start, c * Q)
        k = torch.arange(lo, end)
        dA_last = dA_cumsum[:, c, end - 1 - c * Q]  # (nh,)
        w = torch.exp(torch.clamp(dA_last[:, None] - dA_cumsum[:, c, k - c * Q], max=0.0)) * dt[:, c, k - c * Q]
        st = torch.einsum("khp,khn->hpn", xs[k], _round(Bh[k] * w.T[..., None], round_to))
        if start < c * Q:
            st = st + torch.exp(dA_last)[:, None, None] * chunk_states[c]
        out.append(st)
    return torch.stack(out)


def combined_fwd(x, dt, A, B, C, Q, D=None, z=None, dt_bias=None, initial_states=None,
                 dt_softplus=False, dt_limit=(0.0, float("inf")), round_to=None, seq_idx=None, cu_seqlens=None):
    """The five stages in the order of mamba_ssm's combined forward, which the reference's
    kernels/mamba_kernels/ files were taken from.  Returns (out, final_states), and the states at
    the sequence ends as a third item when cu_seqlens is given (batch of 1,
    kernels/ema_combined.py:56-62)."""
    b, L, nh, p = x.shape
    n = B.shape[-1]
    dA_cs, dt_out = chunk_cumsum(dt, A, Q, dt_bias, dt_softplus, dt_limit)
    states = chunk_state(B, x, dt_out, dA_cs, round_to, seq_idx)
    init = None if initial_states is None else initial_states.reshape(b, nh, p * n)
    prev, final = state_passing(states.reshape(b, -1, nh, p * n), dA_cs[..., -1], init, seq_idx, Q)
    prev = prev.reshape(b, -1, nh, p, n)
    cb = bmm_chunk(C, B, Q, seq_idx)
    out, _ = chunk_scan(cb, x, dt_out, dA_cs, C, prev, D, z, round_to, seq_idx)
    if cu_seqlens is None:
        return out, final.reshape(b, nh, p, n)
    assert b == 1
    varlen = chunk_state_varlen(B[0], x[0], dt_out[0], dA_cs[0], cu_seqlens, prev[0], round_to)
    return out, final.reshape(b, nh, p, n), varlen


# ------------------------------------------------------------------ inputs and brute force


def make_inputs(b, L, nh, p, g, n, seed, dtype=torch.float32, with_z=False):
    """benchmark configuration 5's distributions: x, B, C ~ N(0,1); dt = softplus(N(-2, 0.5));
    A = -exp(U(log 1, log 16)) per head; D = 0 is the configuration's choice (a non-zero D is
    returned for the tests that want one); z ~ N(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(b, L, nh, p, generator=gen).to(dtype)
    Bm = torch.randn(b, L, g, n, generator=gen).to(dtype)
    Cm = torch.randn(b, L, g, n, generator=gen).to(dtype)
    dt = F.softplus(torch.randn(b, L, nh, generator=gen) * 0.5 - 2.0)
    A = -torch.exp(torch.rand(nh, generator=gen) * math.log(16.0))
    D = torch.randn(nh, generator=gen)
    z = torch.randn(b, L, nh, p, generator=gen).to(dtype) if with_z else None
    return x, dt, A, Bm, Cm, D, z


def brute_force(x, dt, A, B, C):
    """Pure-Python O(L^2) evaluation of y_t = sum_{s<=t} (C_t . B_s) exp(A sum_{j=s+1..t} dt_j) dt_s x_s
    (one group), tiny inputs only; shares no code with anything above."""
    b, L, nh, p = x.shape
    n = B.shape[-1]
    out = torch.zeros(b, L, nh, p, dtype=torch.float64)
    for bi in range(b):
        for h in range(nh):
            for t in range(L):
                for s in range(t + 1):
                    cbv = sum(float(C[bi, t, 0, k]) * float(B[bi, s, 0, k]) for k in range(n))
                    dec = math.exp(float(A[h]) * sum(float(dt[bi, j, h]) for j in range(s + 1, t + 1)))
                    wgt = cbv * dec * float(dt[bi, s, h])
                    for f in range(p):
                        out[bi, t, h, f] += wgt * float(x[bi, s, h, f])
    return out


# ------------------------------------------------------------------ backward stages
# Restatements of the six launchers in kernels/mamba_kernels_bwd/ (the reference ships no
# combined backward and no gradient of CB, dt's cumsum or the gate).  Each is pinned in
# tests/test_ssd_oracle.py by torch.autograd (float64) through the forward stage it differentiates.


def bwd_dstates(C, dA_cumsum, dout, round_to=None, seq_idx=None):
    """dprev[b,c,h,p,n] = sum_m round(dout[m,p] * exp(dA_m)) * C[m,n]: the gradient of chunk_scan
    with respect to the carried states; mamba_scan_bwd.py:62-76 (seq_idx: only the rows with the
    id of the previous chunk's last position, :63-71)."""
    b, L, nh, p = dout.shape
    _, _, nc, Q = dA_cumsum.shape
    g, n = C.shape[2], C.shape[3]
    dc = _pad_seq(_up(dout), Q).reshape(b, nc, Q, nh, p)
    Cc = _pad_seq(_up(C), Q).reshape(b, nc, Q, g, n).repeat_interleave(nh // g, dim=3)
    valid = _pad_seq(torch.ones(b, L, 1, dtype=dc.dtype), Q).reshape(b, nc, Q, 1)
    w = torch.exp(dA_cumsum).permute(0, 2, 3, 1) * valid  # (b, nc, Q, nh)
    if seq_idx is not None:
        ids, _, prev = _seq_chunks(seq_idx, Q)
        w = w * (ids == prev[..., None]).to(w.dtype)[..., None]
    return torch.einsum("bcqhp,bcqhn->bchpn", _round(dc * w[..., None], round_to), Cc)


def state_passing_bwd(states, dA_chunk_cumsum, dout, dfinal_states=None, has_initial_states=False,
                      seq_idx=None, chunk_size=None):
    """states (b, C, nh, dim) = the states entering each chunk (index 0 the initial one), dout the
    gradient with respect to them.  Returns (dstates, ddA_chunk_cumsum, dinitstates):
    dstates[c] = gradient of the chunk-local state of chunk c, ddA[c] = <states[c], dstates[c]> *
    exp(dA[c]) (0 for c = 0 without initial states); mamba_state_passing_bwd_dstates.py:66-112.
    With seq_idx exp(dA[c]) is replaced by 0 for the chunks across which the forward drops the
    state (:72-80, :105)."""
    b, nc, nh, dim = states.shape
    dstates = torch.empty_like(dout)
    ddA = dA_chunk_cumsum.new_zeros(b, nh, nc)
    G = dout.new_zeros(b, nh, dim) if dfinal_states is None else _up(dfinal_states).clone()
    keep = None if seq_idx is None else _chunk_keep(seq_idx, chunk_size, dout.dtype)
    for c in range(nc - 1, -1, -1):
        dstates[:, c] = G
        scale = torch.exp(dA_chunk_cumsum[:, :, c])
        if keep is not None:
            scale = scale * keep[:, c, None]
        if c > 0 or has_initial_states:
            ddA[:, :, c] = (states[:, c] * G).sum(-1) * scale
        G = scale[..., None] * G + dout[:, c]
    return dstates, ddA, (G if has_initial_states else None)


def chunk_state_bwd_db(x, dt, dA_cumsum, dstates, B=None, ngroups=1, round_to=None, seq_idx=None):
    """dB[b,l,g,n] = sum over the heads of group g of (sum_p x[m,p] * round(dstates[p,n])) *
    exp(min(dA_last - dA_m, 0)) * dt_m.  With B also ddA_cumsum (b, nh, C, Q): the inclusive cumsum
    along the chunk of r shifted by one slot, r[m] = sum_n db_h[m,n] * B[m,n]: the gradient of the
    chunk states with respect to the per-position dA; mamba_chunk_state_bwd_db.py:91-125,172-180
    (seq_idx: the weight is 0 unless m has the id of the chunk's last position, :88-104)."""
    b, L, nh, p = x.shape
    _, _, nc, Q = dt.shape
    n = dstates.shape[-1]
    xc = _pad_seq(_up(x), Q).reshape(b, nc, Q, nh, p)
    w = (torch.exp(torch.clamp(dA_cumsum[..., -1:] - dA_cumsum, max=0.0)) * dt).permute(0, 2, 3, 1)
    if seq_idx is not None:
        ids, last, _ = _seq_chunks(seq_idx, Q)
        w = w * (ids == last[..., None]).to(w.dtype)[..., None]
    dbh = torch.einsum("bcqhp,bchpn->bcqhn", xc, _round(_up(dstates), round_to)) * w[..., None]
    dB = dbh.reshape(b, nc, Q, ngroups, nh // ngroups, n).sum(4).reshape(b, nc * Q, ngroups, n)[:, :L]
    if B is None:
        return dB
    Bc = _pad_seq(_up(B), Q).reshape(b, nc, Q, ngroups, n).repeat_interleave(nh // ngroups, dim=3)
    r = (dbh * Bc).sum(-1).permute(0, 3, 1, 2)  # (b, nh, nc, Q)
    raw = torch.zeros_like(r)
    raw[..., 1:] = r[..., :-1]
    return dB, torch.cumsum(raw, -1)


def chunk_scan_bwd_dC(prev_states, dA_cumsum, dout, C=None, ngroups=1, round_to=None, seq_idx=None):
    """dC[b,l,g,n] = sum over the heads of group g of (sum_p dout[m,p] * round(prev[p,n])) * exp(dA_m):
    the part of dC that comes through the carried state.  With C also ddA_cumsum_prev[m] =
    sum_n dc_h[m,n] * C[m,n], the gradient with respect to dA_cumsum[m] of that term;
    mamba_chunk_scan_bwd_dc.py:84-101 (seq_idx: weight 0 unless m has the id of the previous
    chunk's last position, :84-96)."""
    b, L, nh, p = dout.shape
    _, _, nc, Q = dA_cumsum.shape
    n = prev_states.shape[-1]
    dc_ = _pad_seq(_up(dout), Q).reshape(b, nc, Q, nh, p)
    w = torch.exp(dA_cumsum).permute(0, 2, 3, 1)
    if seq_idx is not None:
        ids, _, prev = _seq_chunks(seq_idx, Q)
        w = w * (ids == prev[..., None]).to(w.dtype)[..., None]
    dch = torch.einsum("bcqhp,bchpn->bcqhn", dc_, _round(_up(prev_states), round_to)) * w[..., None]
    dC = dch.reshape(b, nc, Q, ngroups, nh // ngroups, n).sum(4).reshape(b, nc * Q, ngroups, n)[:, :L]
    if C is None:
        return dC
    Cc = _pad_seq(_up(C), Q).reshape(b, nc, Q, ngroups, n).repeat_interleave(nh // ngroups, dim=3)
    return dC, (dch * Cc).sum(-1).permute(0, 3, 1, 2)


def chunk_scan_chunk_state_bwd_dx(x, dt, dA_cumsum, B, CB, dout, dstates, D=None, round_to=None,
                                  seq_idx=None):
    """acc[m,p] = exp(min(dA_last - dA_m, 0)) * sum_n B[m,n] * round(dstates[p,n])
                + sum_{k>=m} round(CB[k,m] * exp(min(dA_k - dA_m, 0))) * dout[k,p]
    dx = acc * dt_m + D * dout,  ddt[m] = sum_p acc[m,p] * x[m,p],  dD = sum dout * x;
    mamba_chunk_scan_chunk_state_bwd_dx.py:86-187 (seq_idx: the first term only for the rows with
    the id of the chunk's last position, :93-96).  Returns (dx, ddt (b,nh,C,Q), dD)."""
    b, L, nh, p = x.shape
    _, _, nc, Q = dt.shape
    g, n = B.shape[2], B.shape[3]
    rep = nh // g
    xc = _pad_seq(_up(x), Q).reshape(b, nc, Q, nh, p)
    dc_ = _pad_seq(_up(dout), Q).reshape(b, nc, Q, nh, p)
    Bc = _pad_seq(_up(B), Q).reshape(b, nc, Q, g, n).repeat_interleave(rep, dim=3)
    dA = dA_cumsum.permute(0, 2, 1, 3)  # (b, nc, nh, Q)
    scale = torch.exp(torch.clamp(dA[..., -1:] - dA, max=0.0))  # (b, nc, nh, Q)
    if seq_idx is not None:
        ids, last, _ = _seq_chunks(seq_idx, Q)
        scale = scale * (ids == last[..., None]).to(scale.dtype)[:, :, None]
    acc = torch.einsum("bcmhn,bchpn,bchm->bcmhp", Bc, _round(_up(dstates), round_to), scale)
    cbh = _up(CB).repeat_interleave(rep, dim=2)  # (b, nc, nh, k, m)
    decay = torch.exp(torch.clamp(dA[..., :, None] - dA[..., None, :], max=0.0))  # [k, m]
    valid = _pad_seq(torch.ones(b, L, 1, dtype=xc.dtype), Q).reshape(b, nc, 1, Q, 1)  # k < limit
    mask = torch.tril(torch.ones(Q, Q, dtype=torch.bool))  # k >= m
    w = cbh * decay * valid
    w = _round(torch.where(mask, w, w.new_zeros(())), round_to)
    acc = acc + torch.einsum("bchkm,bckhp->bcmhp", w, dc_)
    dtc = dt.permute(0, 2, 3, 1)  # (b, nc, Q, nh)
    dx = acc * dtc[..., None]
    ddt = (acc * xc).sum(-1).permute(0, 3, 1, 2)
    dD = None
    if D is not None:
        Dv = _up(D)[None, None, None, :, None] if D.dim() == 1 else _up(D)[None, None, None]
        dx = dx + dc_ * Dv
        dD = (dc_ * xc).sum((0, 1, 2)) if D.dim() == 2 else (dc_ * xc).sum((0, 1, 2, 4))
    return dx.reshape(b, nc * Q, nh, p)[:, :L], ddt, dD


def chunk_scan_bwd_ddAcs_stable(x, dt, dA_cumsum, dout, cb):
    """With G[m,n] = <dout[m], x[n]> * dt_n * cb[m,n] * exp(min(dA_m - dA_n, 0)) for n < m:
    ddA_cumsum[j] = sum_{m>=j} sum_{n<j} G[m,n] (0 for j = 0): the gradient of the causal term of
    chunk_scan with respect to the per-position dA; mamba_chunk_scan_bwd_da.py:62-103."""
    b, L, nh, p = x.shape
    _, _, nc, Q = dt.shape
    rep = nh // cb.shape[2]
    xc = _pad_seq(_up(x), Q).reshape(b, nc, Q, nh, p)
    dc_ = _pad_seq(_up(dout), Q).reshape(b, nc, Q, nh, p)
    dA = dA_cumsum.permute(0, 2, 1, 3)
    dtc = dt.permute(0, 2, 1, 3)
    G = torch.einsum("bcmhp,bcnhp->bchmn", dc_, xc) * dtc[..., None, :] * _up(cb).repeat_interleave(rep, dim=2)
    G = G * torch.exp(torch.clamp(dA[..., :, None] - dA[..., None, :], max=0.0))
    strict = torch.tril(torch.ones(Q, Q, dtype=torch.bool), diagonal=-1)
    G = torch.where(strict, G, G.new_zeros(()))
    cum = torch.cumsum(G, -1)                         # over n
    cum = torch.where(strict, cum, cum.new_zeros(()))
    out = torch.zeros_like(dA)
    out[..., 1:] = cum.sum(-2)[..., :-1]              # over m, shifted by one slot
    return out.permute(0, 2, 1, 3)
