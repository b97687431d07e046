"""CPU oracle for the EMA chunked scan (forward and backward).

TEST INFRASTRUCTURE ONLY.  Nothing in the product path may import this module:
only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py use
it, and only as the checker.

It restates, in plain PyTorch on the CPU, the arithmetic of the reference
repository kartiksrinivas007/triton-kernels (paths relative to its root):

* the sequential definition  y_t = exp(A_t) * y_{t-1} + X_t
  (kernels/tests/ema/test_ema_scan_fwd.py:25-37 and
  kernels/tests/ema_bwd/_ema_full_bwd.py:24-34, where P = 1 - exp(A));
* every stage of the chunked forward
  (kernels/ema_kernels/ema_combined_fwd.py:12-45);
* every stage of the chunked backward
  (kernels/ema_kernels_bwd/ema_combined_bwd.py:13-83).

"Flat" layout, as in the reference kernels: A is (N, L) log-decay (A <= 0),
X is (N, L, T); chunk size Q, C = ceil(L / Q) chunks.  The "headed" layout
x:(b, L, nh, d), A:(b, L, nh) is the flat algorithm applied to each (b, h)
pair; `to_flat` / `from_flat` convert.

Pinning status (see tests/test_oracle.py): the reference holds no golden
vectors for this path, so every function here is pinned by what the
mathematics fixes: closed forms (constant decay -> geometric sum, A == 0 ->
cumulative sum), a brute-force pure-Python evaluation on tiny inputs,
chunk-size invariance, equality of the chunked composition with the sequential
recurrence, torch.autograd through the sequential loop, and float64 central
finite differences.  The sequence-level forms (probability coefficient, boundary states)
are pinned the same way: equivalence with the log-decay form under A = log(1 - p),
X = p * x, closed forms, and float64 autograd / finite differences.  No function is left
"parity unpinned".
"""
from __future__ import annotations

import math

import torch

# --------------------------------------------------------------------------------------
# layout helpers
# --------------------------------------------------------------------------------------


def to_flat(x: torch.Tensor, A: torch.Tensor):
    """(b, L, nh, d), (b, L, nh) -> (b*nh, L, d), (b*nh, L)."""
    b, L, nh, d = x.shape
    assert A.shape == (b, L, nh)
    xf = x.permute(0, 2, 1, 3).reshape(b * nh, L, d)
    Af = A.permute(0, 2, 1).reshape(b * nh, L)
    return xf, Af


def from_flat(y: torch.Tensor, b: int, nh: int) -> torch.Tensor:
    """(b*nh, L, d) -> (b, L, nh, d)."""
    N, L, d = y.shape
    assert N == b * nh
    return y.reshape(b, nh, L, d).permute(0, 2, 1, 3).contiguous()


def _pad_chunks(t: torch.Tensor, Q: int, dim: int = 1) -> torch.Tensor:
    """Zero-pad the sequence axis up to a multiple of Q.

    The reference masks loads past L with other=0.0
    (kernels/ema_kernels/ema_cumsum.py:57-60, ema_state_fwd.py:107)."""
    L = t.shape[dim]
    pad = (-L) % Q
    if pad == 0:
        return t
    shape = list(t.shape)
    shape[dim] = pad
    return torch.cat([t, t.new_zeros(shape)], dim=dim)


# --------------------------------------------------------------------------------------
# sequential definition (the textbook recurrence) and its closed-form gradient
# --------------------------------------------------------------------------------------


def ema_loop(X: torch.Tensor, A: torch.Tensor) -> torch.Tensor:
    """y_t = exp(A_t) * y_{t-1} + X_t, y_{-1} = 0; X:(N,L,T), A:(N,L).

    Follows kernels/tests/ema_bwd/_ema_full_bwd.py:24-34 (with 1 - p = exp(A)),
    vectorised over the sequence index n and the feature index."""
    N, L, T = X.shape
    a = torch.exp(A)
    y = torch.empty_like(X)
    z = X.new_zeros(N, T)
    for t in range(L):
        z = a[:, t, None] * z + X[:, t]
        y[:, t] = z
    return y


def ema_loop_bwd(dy: torch.Tensor, X: torch.Tensor, A: torch.Tensor):
    """Gradients of sum(y * dy) for y = ema_loop(X, A), by the reverse recurrence

        g_t = dy_t + exp(A_{t+1}) * g_{t+1},   dX_t = g_t,
        dA_t = exp(A_t) * <g_t, y_{t-1}>       (dA_0 = 0).

    This is what torch.autograd gives through the loop of
    kernels/tests/ema_bwd/_ema_full_bwd.py:56-79; tests check it against autograd.
    Returns (dX:(N,L,T), dA:(N,L))."""
    N, L, T = X.shape
    a = torch.exp(A)
    y = ema_loop(X, A)
    dX = torch.empty_like(X)
    dA = A.new_zeros(N, L)
    g = X.new_zeros(N, T)
    for t in range(L - 1, -1, -1):
        if t + 1 < L:
            g = dy[:, t] + a[:, t + 1, None] * g
        else:
            g = dy[:, t].clone()
        dX[:, t] = g
        if t > 0:
            dA[:, t] = a[:, t] * (g * y[:, t - 1]).sum(-1)
    return dX, dA


# --------------------------------------------------------------------------------------
# sequence-level forms: probability coefficient, boundary states
# --------------------------------------------------------------------------------------


def ema_seq_loop(X: torch.Tensor, coef: torch.Tensor, form: str = "log_decay", init=None):
    """Sequential recurrence from an optional initial state, in either form:

        log_decay:    z_t = exp(min(A_t, 0)) * z_{t-1} + X_t
                      (clamp as in kernels/ema_kernels/ema_scan_fwd.py:141)
        probability:  z_t = (1 - p_t) * z_{t-1} + p_t * X_t
                      (main.py:120-131, kernels/benchmarks/ema_bench.py:53-64)

    X:(N,L,T), coef:(N,L), init:(N,T) or None.  Returns (y:(N,L,T), final:(N,T))."""
    N, L, T = X.shape
    if form == "probability":
        keep, gain = 1.0 - coef, coef
    else:
        keep, gain = torch.exp(torch.clamp(coef, max=0.0)), None
    y = torch.empty_like(X)
    z = X.new_zeros(N, T) if init is None else init.to(X.dtype).clone()
    for t in range(L):
        xin = X[:, t] if gain is None else gain[:, t, None] * X[:, t]
        z = keep[:, t, None] * z + xin
        y[:, t] = z
    return y, z


def ema_seq_loop_bwd(dy, X, coef, form="log_decay", init=None, dfinal=None):
    """Gradients of sum(y * dy) + sum(final * dfinal) for (y, final) = ema_seq_loop(...), by the
    reverse recurrence r_t = dy_t + keep_{t+1} * r_{t+1} (r_{L-1} = dy_{L-1} + dfinal):

        log_decay:    dX_t = r_t,        dA_t = keep_t * <r_t, y_{t-1}>   (0 where A_t > 0)
        probability:  dX_t = p_t * r_t,  dp_t = <r_t, X_t - y_{t-1}>
        dinit = keep_0 * r_0,            y_{-1} = init.

    Returns (dX, dcoef, dinit); tests check it against torch.autograd through ema_seq_loop."""
    N, L, T = X.shape
    prob = form == "probability"
    keep = 1.0 - coef if prob else torch.exp(torch.clamp(coef, max=0.0))
    y, _ = ema_seq_loop(X, coef, form, init)
    y_before = X.new_zeros(N, T) if init is None else init.to(X.dtype)
    dX = torch.empty_like(X)
    dcoef = coef.new_zeros(N, L)
    r = X.new_zeros(N, T) if dfinal is None else dfinal.to(X.dtype).clone()
    for t in range(L - 1, -1, -1):
        r = dy[:, t] + r  # r now holds keep_{t+1} * r_{t+1} (or dfinal) from the step before
        yp = y[:, t - 1] if t > 0 else y_before
        if prob:
            dX[:, t] = coef[:, t, None] * r
            dcoef[:, t] = (r * (X[:, t] - yp)).sum(-1)
        else:
            dX[:, t] = r
            dcoef[:, t] = torch.where(coef[:, t] > 0, torch.zeros_like(coef[:, t]),
                                      keep[:, t] * (r * yp).sum(-1))
        r = keep[:, t, None] * r
    return dX, dcoef, r


# --------------------------------------------------------------------------------------
# chunked forward, stage by stage
# --------------------------------------------------------------------------------------


def chunk_cumsum(A: torch.Tensor, Q: int) -> torch.Tensor:
    """F1.  cs[n,c,q] = sum_{j<=q} A[n, cQ+j], restarting every chunk; positions past L
    add 0 (kernels/ema_kernels/ema_cumsum.py:57-63).  Returns (N, C, Q)."""
    N, L = A.shape
    Ap = _pad_chunks(A, Q)
    return torch.cumsum(Ap.reshape(N, -1, Q), dim=-1)


def chunk_state(X: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """F2.  states[n,c,t] = sum_q exp(min(cs[n,c,Q-1] - cs[n,c,q], 0)) * X[n,cQ+q,t]
    (kernels/ema_kernels/ema_state_fwd.py:99-118; torch form in
    kernels/tests/ema/test_ema_state_fwd.py:46-52).  Returns (N, C, T)."""
    N, C, Q = cs.shape
    Xc = _pad_chunks(X, Q).reshape(N, C, Q, -1)
    scale = torch.exp(torch.clamp(cs[..., -1:] - cs, max=0.0))
    return torch.einsum("ncq,ncqt->nct", scale, Xc)


def state_passing(states: torch.Tensor, cs_last: torch.Tensor):
    """F3.  S_0 = 0; prev[c] = S_c; S_{c+1} = exp(cs_last[c]) * S_c + states[c]
    (kernels/ema_kernels/ema_state_pass.py:100-120).
    Returns (prev:(N,C,T), final:(N,T))."""
    N, C, T = states.shape
    prev = torch.empty_like(states)
    S = states.new_zeros(N, T)
    for c in range(C):
        prev[:, c] = S
        S = torch.exp(cs_last[:, c, None]) * S + states[:, c]
    return prev, S


def chunk_scan(X: torch.Tensor, cs: torch.Tensor, prev: torch.Tensor) -> torch.Tensor:
    """F4.  y[n,cQ+m] = exp(min(cs[m],0)) * prev[n,c]
                       + sum_{k<=m} exp(min(cs[m]-cs[k],0)) * X[n,cQ+k]
    (kernels/ema_kernels/ema_scan_fwd.py:105-159).  Returns (N, L, T)."""
    N, L, T = X.shape
    _, C, Q = cs.shape
    Xc = _pad_chunks(X, Q).reshape(N, C, Q, T)
    seg = torch.exp(torch.clamp(cs[..., :, None] - cs[..., None, :], max=0.0))
    seg = torch.tril(seg)
    y = torch.einsum("ncmk,nckt->ncmt", seg, Xc)
    y = y + torch.exp(torch.clamp(cs, max=0.0))[..., None] * prev[:, :, None, :]
    return y.reshape(N, C * Q, T)[:, :L]


def combined_fwd(A: torch.Tensor, X: torch.Tensor, Q: int):
    """The four stages in the order of kernels/ema_kernels/ema_combined_fwd.py:12-45.
    Returns (y, cs, prev, final)."""
    cs = chunk_cumsum(A, Q)
    states = chunk_state(X, cs)
    prev, final = state_passing(states, cs[..., -1])
    y = chunk_scan(X, cs, prev)
    return y, cs, prev, final


# --------------------------------------------------------------------------------------
# chunked backward, stage by stage
# --------------------------------------------------------------------------------------


def bwd_dstates(cs: torch.Tensor, dy: torch.Tensor) -> torch.Tensor:
    """B1.  ds[n,c,t] = sum_m exp(cs[n,c,m]) * dy[n,cQ+m,t]
    (kernels/ema_kernels_bwd/ema_scan_bwd.py:87-127; torch form in
    kernels/tests/ema_bwd/test_ema_scan_bwd_dstates.py:113-119)."""
    N, C, Q = cs.shape
    dyc = _pad_chunks(dy, Q).reshape(N, C, Q, -1)
    return torch.einsum("ncq,ncqt->nct", torch.exp(cs), dyc)


def state_passing_bwd(prev: torch.Tensor, cs_last: torch.Tensor, ds: torch.Tensor):
    """B2.  g_{C-1} = 0; g_{c-1} = exp(cs_last[c]) * g_c + ds[c];
    ddA_chunk[c] = exp(cs_last[c]) * <prev[c], g_c>, ddA_chunk[0] = 0
    (kernels/ema_kernels_bwd/ema_state_passing_bwd_dstates.py:59-98).
    Returns (g:(N,C,T), ddA_chunk:(N,C))."""
    N, C, T = prev.shape
    g = torch.empty_like(ds)
    ddA = cs_last.new_zeros(N, C)
    cur = ds.new_zeros(N, T)
    for c in range(C - 1, -1, -1):
        g[:, c] = cur
        scale = torch.exp(cs_last[:, c])
        if c > 0:
            ddA[:, c] = scale * (prev[:, c] * cur).sum(-1)
        cur = scale[:, None] * cur + ds[:, c]
    return g, ddA


def bwd_dx(cs: torch.Tensor, dy: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """B3.  dx[n,cQ+m] = exp(min(cs[Q-1]-cs[m],0)) * g[n,c]
                        + sum_{k>=m} exp(min(cs[k]-cs[m],0)) * dy[n,cQ+k]
    (kernels/ema_kernels_bwd/ema_chunk_scan_chunk_state_bwd_dx.py:128-205)."""
    N, L, T = dy.shape
    _, C, Q = cs.shape
    dyc = _pad_chunks(dy, Q).reshape(N, C, Q, T)
    W = torch.exp(torch.clamp(cs[..., None, :] - cs[..., :, None], max=0.0))  # [m, k]
    W = torch.triu(W)
    dx = torch.einsum("ncmk,nckt->ncmt", W, dyc)
    dx = dx + torch.exp(torch.clamp(cs[..., -1:] - cs, max=0.0))[..., None] * g[:, :, None, :]
    return dx.reshape(N, C * Q, T)[:, :L]


def _valid_mask(L: int, C: int, Q: int, like: torch.Tensor) -> torch.Tensor:
    pos = torch.arange(C * Q).reshape(C, Q)
    return (pos < L).to(like.dtype)


def bwd_db(X: torch.Tensor, cs: torch.Tensor, g: torch.Tensor, raw: bool = False) -> torch.Tensor:
    """B4.  r[m] = exp(min(cs[Q-1]-cs[m],0)) * <g[n,c], X[n,cQ+m]> stored in slot m+1
    (slot 0 = 0, the last row is dropped), then an inclusive cumsum along the chunk
    unless `raw` (kernels/ema_kernels_bwd/ema_chunk_state_bwd_db.py:75-117,146-151).
    Returns (N, C, Q)."""
    N, L, T = X.shape
    _, C, Q = cs.shape
    Xc = _pad_chunks(X, Q).reshape(N, C, Q, T)
    r = torch.exp(torch.clamp(cs[..., -1:] - cs, max=0.0)) * torch.einsum("nct,ncqt->ncq", g, Xc)
    r = r * _valid_mask(L, C, Q, r)
    out = torch.zeros_like(r)
    out[..., 1:] = r[..., :-1]
    return out if raw else torch.cumsum(out, dim=-1)


def bwd_dc(prev: torch.Tensor, cs: torch.Tensor, dy: torch.Tensor) -> torch.Tensor:
    """B5 (before the reverse cumsum).  s[m] = exp(cs[m]) * <dy[n,cQ+m], prev[n,c]>
    (kernels/ema_kernels_bwd/ema_chunk_scan_bwd_dc.py:82-111).  Returns (N, C, Q)."""
    N, L, T = dy.shape
    _, C, Q = cs.shape
    dyc = _pad_chunks(dy, Q).reshape(N, C, Q, T)
    s = torch.exp(cs) * torch.einsum("ncqt,nct->ncq", dyc, prev)
    return s * _valid_mask(L, C, Q, s)


def bwd_da_intra(X: torch.Tensor, cs: torch.Tensor, dy: torch.Tensor) -> torch.Tensor:
    """B6.  G[m,k] = exp(min(cs[m]-cs[k],0)) * <dy[m], X[k]> for k < m;
    ddA[j] = sum_{m>=j} sum_{k<j} G[m,k], ddA[0] = 0
    (kernels/ema_kernels_bwd/ema_scan_da.py:59-102; hand-derived torch form in
    kernels/tests/ema_bwd/test_ema_scan_da.py:19-38).  Returns (N, C, Q)."""
    N, L, T = X.shape
    _, C, Q = cs.shape
    Xc = _pad_chunks(X, Q).reshape(N, C, Q, T)
    dyc = _pad_chunks(dy, Q).reshape(N, C, Q, T)
    G = torch.einsum("ncmt,nckt->ncmk", dyc, Xc)
    G = G * torch.exp(torch.clamp(cs[..., :, None] - cs[..., None, :], max=0.0))
    G = torch.tril(G, diagonal=-1)
    # P[m, j] = sum_{k<=j} G[m,k], kept strictly below the diagonal, summed over rows
    # m > j, lands in slot j+1: ddA[j+1] = sum_{m>j} sum_{k<=j} G[m,k].
    P = torch.tril(torch.cumsum(G, dim=-1), diagonal=-1)
    col = P.sum(dim=-2)
    out = torch.zeros_like(col)
    out[..., 1:] = col[..., :-1]
    return out


def combined_bwd(dy: torch.Tensor, X: torch.Tensor, A: torch.Tensor, Q: int):
    """Backward in the order of kernels/ema_kernels_bwd/ema_combined_bwd.py:13-83.
    Returns (dX:(N,L,T), ddA:(N,C,Q)); ddA.reshape(N, C*Q)[:, :L] is dL/dA."""
    cs = chunk_cumsum(A, Q)
    states = chunk_state(X, cs)
    prev, _ = state_passing(states, cs[..., -1])
    ds = bwd_dstates(cs, dy)
    g, ddA_chunk = state_passing_bwd(prev, cs[..., -1], ds)
    dx = bwd_dx(cs, dy, g)
    ddA_next = bwd_db(X, cs, g)
    ddA_prev = bwd_dc(prev, cs, dy)
    ddA_prev[..., -1] += ddA_chunk
    ddA_prev = ddA_prev.flip([-1]).cumsum(dim=-1).flip([-1])
    ddA = bwd_da_intra(X, cs, dy) + ddA_next + ddA_prev
    return dx, ddA


# --------------------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations (CPU generator so that the oracle
# and the GPU see identical bits)
# --------------------------------------------------------------------------------------


def make_inputs(b, nh, L, d, seed, dtype=torch.float32, u_mean=2.0, scale_x=False, with_dy=True):
    """x ~ N(0,1) (b,L,nh,d); A = log(sigmoid(u)), u ~ N(u_mean, 1) (b,L,nh) fp32;
    dy ~ N(0,1).  With scale_x the kernel input is (1 - alpha) * x, as in
    kernels/tests/ema/test_ema_scan_fwd.py:104-105."""
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(b, L, nh, d, generator=gen, dtype=torch.float32)
    u = torch.randn(b, L, nh, generator=gen, dtype=torch.float32) + u_mean
    A = torch.nn.functional.logsigmoid(u)
    if scale_x:
        x = (1.0 - torch.sigmoid(u))[..., None] * x
    x = x.to(dtype)
    dy = torch.randn(b, L, nh, d, generator=gen, dtype=torch.float32).to(dtype) if with_dy else None
    return x, A, dy


def brute_force(X, A):
    """Pure-Python O(L^2) evaluation of y_t = sum_{k<=t} exp(sum_{j=k+1..t} A_j) X_k,
    for tiny inputs only; shares no code with anything above."""
    N, L, T = X.shape
    out = [[[0.0] * T for _ in range(L)] for _ in range(N)]
    for n in range(N):
        for t in range(L):
            for k in range(t + 1):
                w = math.exp(sum(float(A[n, j]) for j in range(k + 1, t + 1)))
                for f in range(T):
                    out[n][t][f] += w * float(X[n, k, f])
    return torch.tensor(out, dtype=torch.float64)
