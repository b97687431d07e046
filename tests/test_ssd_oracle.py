"""Pins the SSD oracle (oracle/ssd_oracle.py) by what the mathematics fixes.  CPU only.

The reference holds no golden vectors for the Mamba-2 path and its comparison provider
(mamba_ssm) is not installed, so nothing here compares with reference outputs."""
import math

import pytest
import torch

from oracle import ema_oracle as E
from oracle import ssd_oracle as S

D64 = torch.float64


def _f64(*ts):
    return [None if t is None else t.to(D64) for t in ts]


def test_loop_matches_brute_force():
    x, dt, A, B, C, _, _ = _f64(*S.make_inputs(1, 7, 2, 3, 1, 4, seed=0))
    y, _ = S.ssd_loop(x, dt, A, B, C)
    assert torch.allclose(y, S.brute_force(x, dt, A, B, C), rtol=1e-12, atol=1e-12)


def test_loop_reduces_to_ema_scan():
    # dstate = 1, B = C = 1, dt = 1: h_t = exp(A) h_{t-1} + x_t per head, the EMA recurrence
    b, L, nh, p = 2, 33, 3, 5
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(b, L, nh, p, generator=gen, dtype=D64)
    A = -torch.rand(nh, generator=gen, dtype=D64)
    ones = torch.ones(b, L, 1, 1, dtype=D64)
    y, fin = S.ssd_loop(x, torch.ones(b, L, nh, dtype=D64), A, ones, ones)
    xf, Af = E.to_flat(x, A.expand(b, L, nh).contiguous())
    y_ema = E.from_flat(E.ema_loop(xf, Af), b, nh)
    assert torch.allclose(y, y_ema, rtol=1e-12, atol=1e-12)
    assert torch.allclose(fin[..., 0], y[:, -1], rtol=1e-12, atol=1e-12)


def test_loop_matches_segsum_matrix_form():
    # the quadratic form of ssd_fwd_ref (mamba_ssd_fwd.py:772-777) with natural exp
    x, dt, A, B, C, D, z = _f64(*S.make_inputs(2, 19, 4, 3, 2, 5, seed=2, with_z=True))
    y, _ = S.ssd_loop(x, dt, A, B, C, D, z)
    dA = (dt * A).permute(0, 2, 1)  # (b, h, s)
    cs = torch.cumsum(dA, -1)
    seg = cs[..., :, None] - cs[..., None, :]
    L = x.shape[1]
    mask = torch.tril(torch.ones(L, L, dtype=torch.bool))
    Bh = B.repeat_interleave(2, dim=2) * dt[..., None]
    Ch = C.repeat_interleave(2, dim=2)
    cb = torch.einsum("bthd,bshd->bhts", Ch, Bh)
    w = torch.where(mask, cb * torch.exp(torch.where(mask, seg, torch.zeros((), dtype=D64))), torch.zeros((), dtype=D64))
    out = torch.einsum("bhts,bshd->bthd", w, x) + D[None, None, :, None] * x
    out = out * z * torch.sigmoid(z)
    assert torch.allclose(y, out, rtol=1e-11, atol=1e-11)


@pytest.mark.parametrize("L,Q", [(64, 16), (50, 16), (37, 64), (96, 32), (5, 8)])
@pytest.mark.parametrize("g", [1, 2])
def test_chunked_stages_equal_loop(L, Q, g):
    x, dt, A, B, C, D, z = _f64(*S.make_inputs(2, L, 4, 6, g, 5, seed=L + Q, with_z=True))
    gen = torch.Generator().manual_seed(9)
    init = torch.randn(2, 4, 6, 5, generator=gen, dtype=D64)
    y_ref, fin_ref = S.ssd_loop(x, dt, A, B, C, D, z, init)
    y, fin = S.combined_fwd(x, dt, A, B, C, Q, D=D, z=z, initial_states=init)
    assert torch.allclose(y, y_ref, rtol=1e-10, atol=1e-10)
    assert torch.allclose(fin, fin_ref, rtol=1e-10, atol=1e-10)


def test_chunk_size_invariance_f32():
    x, dt, A, B, C, D, _ = S.make_inputs(1, 200, 2, 8, 1, 16, seed=4)
    outs = [S.combined_fwd(x, dt, A, B, C, Q, D=D)[0] for Q in (16, 64, 256)]
    for o in outs[1:]:
        assert torch.allclose(o, outs[0], rtol=1e-4, atol=1e-4)


def test_process_dt_bias_softplus_clamp():
    dt = torch.tensor([[[-3.0, 0.5, 25.0]]])
    bias = torch.tensor([0.5, -0.5, 0.0])
    out = S.process_dt(dt, bias, True, (0.1, 10.0))
    want = [max(0.1, math.log1p(math.exp(-2.5))), math.log1p(math.exp(0.0)), 10.0]
    assert torch.allclose(out.flatten(), torch.tensor(want), rtol=1e-6)


def test_chunk_cumsum_restarts_and_pads():
    dt = torch.rand(1, 10, 2)
    A = torch.tensor([-1.0, -2.0])
    dA_cs, dt_out = S.chunk_cumsum(dt, A, 4)
    assert dA_cs.shape == (1, 2, 3, 4) and dt_out.shape == (1, 2, 3, 4)
    assert torch.allclose(dA_cs[0, 1, 1], torch.cumsum(dt[0, 4:8, 1] * -2.0, 0))
    assert torch.equal(dt_out[0, :, 2, 2:], torch.zeros(2, 2))  # past L
    assert torch.allclose(dA_cs[0, 0, 2, 3], dA_cs[0, 0, 2, 1])


def test_chunk_state_is_final_state_of_local_scan():
    x, dt, A, B, C, _, _ = _f64(*S.make_inputs(1, 24, 2, 3, 1, 4, seed=6))
    dA_cs, dt_out = S.chunk_cumsum(dt, A, 8)
    st = S.chunk_state(B, x, dt_out.to(D64), dA_cs.to(D64))
    for c in range(3):
        sl = slice(8 * c, 8 * c + 8)
        _, fin = S.ssd_loop(x[:, sl], dt[:, sl], A, B[:, sl], C[:, sl])
        assert torch.allclose(st[:, c], fin, rtol=1e-6, atol=1e-7)  # dA_cs went through float32


def test_linearity_in_x():
    x, dt, A, B, C, D, _ = _f64(*S.make_inputs(1, 40, 2, 4, 1, 4, seed=7))
    x2 = torch.randn_like(x)
    f = lambda v: S.combined_fwd(v, dt, A, B, C, 16, D=D)[0]
    assert torch.allclose(f(2.0 * x - 3.0 * x2), 2.0 * f(x) - 3.0 * f(x2), rtol=1e-10, atol=1e-10)


def test_bmm_chunk_matches_einsum_per_chunk():
    gen = torch.Generator().manual_seed(8)
    Cm = torch.randn(2, 21, 2, 6, generator=gen)
    Bm = torch.randn(2, 21, 2, 6, generator=gen)
    cb = S.bmm_chunk(Cm, Bm, 8)
    assert cb.shape == (2, 3, 2, 8, 8)
    assert torch.allclose(cb[1, 1, 0], Cm[1, 8:16, 0] @ Bm[1, 8:16, 0].T, rtol=1e-5, atol=1e-5)
    assert torch.equal(cb[0, 2, 1, 5:], torch.zeros(3, 8))  # rows past L


# ---------------------------------------------------------------- packed batches (seq_idx)


def _ids(lengths_per_row, first=0):
    """(b, L) int32 ids from per-row sequence lengths; ids count up from `first`."""
    rows = []
    for lengths in lengths_per_row:
        rows.append(torch.cat([torch.full((n,), first + i, dtype=torch.int32) for i, n in enumerate(lengths)]))
    return torch.stack(rows)


PACKS = [
    [[13, 8, 16], [37]],          # boundaries inside chunks, a row that is one sequence
    [[16, 16, 5], [1, 35, 1]],    # boundaries on chunk edges (Q = 16), sequences of one position
    [[3, 2, 4, 28], [20, 17]],    # several boundaries inside one chunk
]


@pytest.mark.parametrize("pack", PACKS)
def test_packed_loop_equals_each_sequence_alone(pack):
    L = sum(pack[0])
    x, dt, A, B, C, D, z = _f64(*S.make_inputs(2, L, 4, 3, 2, 5, seed=21, with_z=True))
    gen = torch.Generator().manual_seed(5)
    init = torch.randn(2, 4, 3, 5, generator=gen, dtype=D64)
    seq = _ids(pack)
    y, fin = S.ssd_loop(x, dt, A, B, C, D, z, init, seq_idx=seq)
    for r, lengths in enumerate(pack):
        t0 = 0
        for i, n in enumerate(lengths):
            sl = slice(t0, t0 + n)
            one = lambda t: t[r:r + 1, sl]
            yi, fi = S.ssd_loop(one(x), one(dt), A, one(B), one(C), D, one(z),
                                init[r:r + 1] if i == 0 else None)  # only id 0 continues the initial state
            assert torch.allclose(y[r:r + 1, sl], yi, rtol=1e-12, atol=1e-12)
            t0 += n
        assert torch.allclose(fin[r:r + 1], fi, rtol=1e-12, atol=1e-12)


def test_packed_loop_drops_initial_state_when_first_id_is_not_zero():
    x, dt, A, B, C, _, _ = _f64(*S.make_inputs(1, 9, 2, 3, 1, 4, seed=22))
    init = torch.randn(1, 2, 3, 4, dtype=D64)
    y, _ = S.ssd_loop(x, dt, A, B, C, initial_states=init, seq_idx=_ids([[9]], first=1))
    y0, _ = S.ssd_loop(x, dt, A, B, C)
    assert torch.allclose(y, y0, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("pack", PACKS)
@pytest.mark.parametrize("Q", [8, 16, 64])
def test_chunked_stages_equal_loop_packed(pack, Q):
    L = sum(pack[0])
    x, dt, A, B, C, D, z = _f64(*S.make_inputs(2, L, 4, 6, 2, 5, seed=Q, with_z=True))
    gen = torch.Generator().manual_seed(9)
    init = torch.randn(2, 4, 6, 5, generator=gen, dtype=D64)
    seq = _ids(pack)
    y_ref, fin_ref = S.ssd_loop(x, dt, A, B, C, D, z, init, seq_idx=seq)
    y, fin = S.combined_fwd(x, dt, A, B, C, Q, D=D, z=z, initial_states=init, seq_idx=seq)
    assert torch.allclose(y, y_ref, rtol=1e-10, atol=1e-10)
    assert torch.allclose(fin, fin_ref, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("lengths", [[13, 8, 16], [16, 16, 5], [1, 35, 1], [3, 2, 4, 28], [37]])
@pytest.mark.parametrize("Q", [8, 16, 64])
def test_varlen_states_equal_each_sequence_alone(lengths, Q):
    """The state at the end of every packed sequence is the final state of that sequence run
    through the recurrence on its own.  The first one continues the initial state only if it reaches
    past the first chunk: the reference adds the state entering the last chunk of a sequence only
    for sequences that began before that chunk (kernels/ema_chunk_state.py:563), which leaves the
    initial state out for a first sequence that ends inside chunk 0."""
    L = sum(lengths)
    x, dt, A, B, C, _, _ = _f64(*S.make_inputs(1, L, 4, 6, 2, 5, seed=Q + L))
    init = torch.randn(1, 4, 6, 5, generator=torch.Generator().manual_seed(2), dtype=D64)
    cu = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)
    _, fin, varlen = S.combined_fwd(x, dt, A, B, C, Q, initial_states=init, seq_idx=_ids([lengths]), cu_seqlens=cu)
    assert varlen.shape == (len(lengths), 4, 6, 5)
    for i in range(len(lengths)):
        sl = slice(int(cu[i]), int(cu[i + 1]))
        continues = i == 0 and int(cu[1]) > Q
        _, fi = S.ssd_loop(x[:, sl], dt[:, sl], A, B[:, sl], C[:, sl], initial_states=init if continues else None)
        assert torch.allclose(varlen[i], fi[0], rtol=1e-10, atol=1e-10)
    if len(lengths) > 1 or L > Q:
        assert torch.allclose(varlen[-1], fin[0], rtol=1e-10, atol=1e-10)


def test_bmm_chunk_masks_pairs_of_different_sequences():
    gen = torch.Generator().manual_seed(8)
    Cm = torch.randn(1, 21, 1, 6, generator=gen)
    Bm = torch.randn(1, 21, 1, 6, generator=gen)
    seq = _ids([[5, 6, 10]])
    cb = S.bmm_chunk(Cm, Bm, 8, seq_idx=seq)
    full = S.bmm_chunk(Cm, Bm, 8)
    for c in range(3):
        for m in range(8):
            for k in range(8):
                tm, tk = 8 * c + m, 8 * c + k
                same = tm < 21 and tk < 21 and seq[0, tm] == seq[0, tk]
                assert cb[0, c, 0, m, k] == (full[0, c, 0, m, k] if same else 0.0)


# ---------------------------------------------------------------- backward stages vs autograd

# every backward pin also runs on a packed batch: L = 21, Q = 8, boundaries inside the first and
# the last chunk in row 0 and on a chunk edge in row 1
BWD_SEQ = [None, "packed"]


def _bwd_seq(kind):
    return None if kind is None else _ids([[3, 15, 3], [8, 13]])


def _bwd_case(b=2, L=21, nh=4, p=3, g=2, n=5, Q=8, seed=11):
    x, dt_raw, A, B, C, D, _ = _f64(*S.make_inputs(b, L, nh, p, g, n, seed=seed))
    dA_cs, dt = S.chunk_cumsum(dt_raw, A, Q)
    gen = torch.Generator().manual_seed(seed + 1)
    dout = torch.randn(b, L, nh, p, generator=gen, dtype=D64)
    nc = dt.shape[2]
    prev = torch.randn(b, nc, nh, p, n, generator=gen, dtype=D64)
    dstates = torch.randn(b, nc, nh, p, n, generator=gen, dtype=D64)
    return x, dt, dA_cs, B, C, D, dout, prev, dstates, Q


def _cumsum_of(dA):
    return torch.cumsum(dA, -1)


def _per_position(dA_cs):
    d = dA_cs.clone()
    d[..., 1:] = dA_cs[..., 1:] - dA_cs[..., :-1]
    return d


@pytest.mark.parametrize("kind", BWD_SEQ)
def test_bwd_dstates_is_grad_of_chunk_scan_wrt_prev(kind):
    x, dt, dA_cs, B, C, D, dout, prev, _, Q = _bwd_case()
    seq = _bwd_seq(kind)
    pr = prev.clone().requires_grad_()
    out, _ = S.chunk_scan(S.bmm_chunk(C, B, Q, seq), x, dt, dA_cs, C, pr, D, seq_idx=seq)
    (out * dout).sum().backward()
    assert torch.allclose(S.bwd_dstates(C, dA_cs, dout, seq_idx=seq), pr.grad, rtol=1e-10, atol=1e-10)
    if seq is not None:
        assert not torch.allclose(S.bwd_dstates(C, dA_cs, dout), pr.grad, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("kind", BWD_SEQ)
def test_state_passing_bwd_is_autograd_of_state_passing(kind):
    gen = torch.Generator().manual_seed(3)
    b, nc, nh, dim = 2, 5, 3, 7
    # chunk size 4, L = 18 (a short last chunk): row 0 changes id inside chunks 1 and 3, row 1 on
    # the edge between chunks 1 and 2, and row 1 starts with id 1 (its initial state is dropped)
    seq = None if kind is None else torch.stack([_ids([[6, 8, 4]])[0], _ids([[8, 10]], first=1)[0]])
    kw = {} if seq is None else dict(seq_idx=seq, chunk_size=4)
    st = torch.randn(b, nc, nh, dim, generator=gen, dtype=D64).requires_grad_()
    dA = (-torch.rand(b, nh, nc, generator=gen, dtype=D64)).requires_grad_()
    init = torch.randn(b, nh, dim, generator=gen, dtype=D64).requires_grad_()
    dprev = torch.randn(b, nc, nh, dim, generator=gen, dtype=D64)
    dfin = torch.randn(b, nh, dim, generator=gen, dtype=D64)
    for use_init in (True, False):
        for t in (st, dA, init):
            t.grad = None
        prev, fin = S.state_passing(st, dA, init if use_init else None, **kw)
        ((prev * dprev).sum() + (fin * dfin).sum()).backward()
        dst, ddA, dinit = S.state_passing_bwd(prev.detach(), dA.detach(), dprev, dfin, has_initial_states=use_init,
                                              **kw)
        assert torch.allclose(dst, st.grad, rtol=1e-10, atol=1e-10)
        assert torch.allclose(ddA, dA.grad, rtol=1e-10, atol=1e-10)
        if use_init:
            assert torch.allclose(dinit, init.grad, rtol=1e-10, atol=1e-10)
        else:
            assert dinit is None and torch.equal(ddA[:, :, 0], torch.zeros(b, nh, dtype=D64))
        if seq is not None:
            assert torch.equal(ddA[1, :, 0], torch.zeros(nh, dtype=D64))  # row 1 starts with id 1


@pytest.mark.parametrize("kind", BWD_SEQ)
def test_chunk_state_bwd_db_is_grad_of_chunk_state(kind):
    x, dt, dA_cs, B, C, D, dout, prev, dstates, Q = _bwd_case()
    seq = _bwd_seq(kind)
    Br = B.clone().requires_grad_()
    dA = _per_position(dA_cs).requires_grad_()
    st = S.chunk_state(Br, x, dt, _cumsum_of(dA), seq_idx=seq)
    (st * dstates).sum().backward()
    dB, ddA = S.chunk_state_bwd_db(x, dt, dA_cs, dstates, B=B, ngroups=B.shape[2], seq_idx=seq)
    assert torch.allclose(dB, Br.grad, rtol=1e-10, atol=1e-10)
    assert torch.allclose(ddA, dA.grad, rtol=1e-10, atol=1e-10)
    assert torch.allclose(S.chunk_state_bwd_db(x, dt, dA_cs, dstates, ngroups=B.shape[2], seq_idx=seq), dB)


@pytest.mark.parametrize("kind", BWD_SEQ)
def test_chunk_scan_bwd_dC_is_grad_of_the_carried_state_term(kind):
    x, dt, dA_cs, B, C, D, dout, prev, _, Q = _bwd_case()
    seq = _bwd_seq(kind)
    Cr = C.clone().requires_grad_()
    dAr = dA_cs.clone().requires_grad_()
    zero_cb = torch.zeros(x.shape[0], dt.shape[2], C.shape[2], Q, Q, dtype=D64)  # leaves only C . prev
    out, _ = S.chunk_scan(zero_cb, x, dt, dAr, Cr, prev, seq_idx=seq)
    (out * dout).sum().backward()
    dC, ddA_prev = S.chunk_scan_bwd_dC(prev, dA_cs, dout, C=C, ngroups=C.shape[2], seq_idx=seq)
    assert torch.allclose(dC, Cr.grad, rtol=1e-10, atol=1e-10)
    assert torch.allclose(ddA_prev, dAr.grad, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("kind", BWD_SEQ)
def test_bwd_dx_is_grad_wrt_x_and_explicit_dt(kind):
    x, dt, dA_cs, B, C, D, dout, prev, dstates, Q = _bwd_case()
    seq = _bwd_seq(kind)
    cb = S.bmm_chunk(C, B, Q, seq)
    xr, dtr, Dr = x.clone().requires_grad_(), dt.clone().requires_grad_(), D.clone().requires_grad_()
    zero_prev = torch.zeros_like(prev)
    out, _ = S.chunk_scan(cb, xr, dtr, dA_cs, C, zero_prev, Dr, seq_idx=seq)   # dA_cs held fixed: only the explicit dt
    st = S.chunk_state(B, xr, dtr, dA_cs, seq_idx=seq)
    ((out * dout).sum() + (st * dstates).sum()).backward()
    dx, ddt, dD = S.chunk_scan_chunk_state_bwd_dx(x, dt, dA_cs, B, cb, dout, dstates, D=D, seq_idx=seq)
    assert torch.allclose(dx, xr.grad, rtol=1e-10, atol=1e-10)
    assert torch.allclose(ddt, dtr.grad, rtol=1e-10, atol=1e-10)
    assert torch.allclose(dD, Dr.grad, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("kind", BWD_SEQ)
def test_ddAcs_stable_is_grad_of_the_causal_term_wrt_dA(kind):
    x, dt, dA_cs, B, C, D, dout, prev, _, Q = _bwd_case()
    cb = S.bmm_chunk(C, B, Q, _bwd_seq(kind))  # the masked cb is all a packed batch needs here
    dA = _per_position(dA_cs).requires_grad_()
    out, _ = S.chunk_scan(cb, x, dt, _cumsum_of(dA), C, torch.zeros_like(prev))
    (out * dout).sum().backward()
    got = S.chunk_scan_bwd_ddAcs_stable(x, dt, dA_cs, dout, cb)
    assert torch.allclose(got, dA.grad, rtol=1e-10, atol=1e-10)
