"""Pins the CPU oracle (oracle/ema_oracle.py) by checks the mathematics fixes.

The reference repository holds no golden vectors for the EMA path (every one of its tests
draws fresh random inputs), so the oracle is pinned by: a brute-force pure-Python
evaluation, closed forms, invariances, torch.autograd through the sequential loop and
float64 central finite differences.  Each check is chosen so that a plausible slip (a
dropped term, a shifted index, a wrong sign, a transposed decay matrix) fails it.
"""
import math

import pytest
import torch

from oracle import ema_oracle as O

torch.manual_seed(0)
F64 = torch.float64


def rand_case(N, L, T, seed, dtype=F64, lo=0.05, hi=0.999):
    g = torch.Generator().manual_seed(seed)
    alpha = torch.rand(N, L, generator=g, dtype=dtype) * (hi - lo) + lo
    A = torch.log(alpha)
    X = torch.randn(N, L, T, generator=g, dtype=dtype)
    dy = torch.randn(N, L, T, generator=g, dtype=dtype)
    return A, X, dy


# ---------------------------------------------------------------- sequential definition


def test_loop_matches_brute_force():
    A, X, _ = rand_case(2, 9, 3, seed=1)
    assert torch.allclose(O.ema_loop(X, A), O.brute_force(X, A), rtol=1e-12, atol=1e-12)


def test_loop_constant_decay_closed_form():
    N, L, T = 1, 40, 2
    alpha = 0.9
    A = torch.full((N, L), math.log(alpha), dtype=F64)
    X = torch.randn(N, L, T, dtype=F64)
    y = O.ema_loop(X, A)
    t = torch.arange(L, dtype=F64)
    W = torch.tril(alpha ** (t[:, None] - t[None, :]).clamp(min=0))
    assert torch.allclose(y[0], W @ X[0], rtol=1e-12, atol=1e-12)


def test_loop_zero_log_decay_is_cumsum():
    X = torch.randn(2, 33, 4, dtype=F64)
    A = torch.zeros(2, 33, dtype=F64)
    assert torch.allclose(O.ema_loop(X, A), torch.cumsum(X, dim=1), rtol=1e-12, atol=1e-12)


def test_loop_first_step_ignores_first_decay():
    A, X, _ = rand_case(1, 5, 2, seed=2)
    A2 = A.clone()
    A2[:, 0] = -7.0  # y_{-1} = 0, so A_0 never matters
    assert torch.equal(O.ema_loop(X, A), O.ema_loop(X, A2))


def test_probability_form_config1():
    # benchmark configuration 1: y_t = alpha_t y_{t-1} + (1 - alpha_t) x_t with X = (1-alpha) x
    x, A, _ = O.make_inputs(1, 2, 512, 64, seed=11, scale_x=False)
    xs, _, _ = O.make_inputs(1, 2, 512, 64, seed=11, scale_x=True)
    alpha = torch.exp(A)
    z = torch.zeros(1, 2, 64)
    ref = torch.empty_like(x)
    for t in range(512):
        z = alpha[:, t, :, None] * z + (1 - alpha[:, t, :, None]) * x[:, t]
        ref[:, t] = z
    xf, Af = O.to_flat(xs, A)
    y = O.from_flat(O.ema_loop(xf, Af), 1, 2)
    assert torch.allclose(y, ref, rtol=1e-4, atol=1e-6)


# ---------------------------------------------------------------- sequential gradient


def test_loop_bwd_matches_autograd():
    A, X, dy = rand_case(2, 37, 5, seed=3)
    A.requires_grad_()
    X.requires_grad_()
    (O.ema_loop(X, A) * dy).sum().backward()
    dX, dA = O.ema_loop_bwd(dy, X.detach(), A.detach())
    assert torch.allclose(dX, X.grad, rtol=1e-10, atol=1e-12)
    assert torch.allclose(dA, A.grad, rtol=1e-10, atol=1e-12)


def test_loop_bwd_finite_differences():
    A, X, dy = rand_case(1, 12, 3, seed=4)
    dX, dA = O.ema_loop_bwd(dy, X, A)
    loss = lambda X_, A_: (O.ema_loop(X_, A_) * dy).sum()
    eps = 1e-6
    for t in range(12):
        Ap, Am = A.clone(), A.clone()
        Ap[0, t] += eps
        Am[0, t] -= eps
        fd = (loss(X, Ap) - loss(X, Am)) / (2 * eps)
        assert abs(fd - dA[0, t]) < 1e-6 * max(1.0, abs(fd)), (t, fd, dA[0, t])
    for (t, f) in [(0, 0), (5, 2), (11, 1)]:
        Xp, Xm = X.clone(), X.clone()
        Xp[0, t, f] += eps
        Xm[0, t, f] -= eps
        fd = (loss(Xp, A) - loss(Xm, A)) / (2 * eps)
        assert abs(fd - dX[0, t, f]) < 1e-6 * max(1.0, abs(fd))


def test_impulse_gradient():
    # dy = delta at (t0, f0): dX_k = exp(sum_{j=k+1..t0} A_j) for k <= t0, else 0
    A, X, _ = rand_case(1, 20, 2, seed=5)
    dy = torch.zeros(1, 20, 2, dtype=F64)
    t0 = 13
    dy[0, t0, 1] = 1.0
    dX, _ = O.ema_loop_bwd(dy, X, A)
    for k in range(20):
        want = math.exp(float(A[0, k + 1 : t0 + 1].sum())) if k <= t0 else 0.0
        assert abs(float(dX[0, k, 1]) - want) < 1e-12
        assert float(dX[0, k, 0]) == 0.0


# ---------------------------------------------------------------- chunked forward stages


@pytest.mark.parametrize("L,Q", [(64, 16), (70, 16), (5, 8), (128, 128), (129, 64), (1, 4)])
def test_chunked_forward_equals_loop(L, Q):
    A, X, _ = rand_case(3, L, 4, seed=10 + L)
    y, cs, prev, final = O.combined_fwd(A, X, Q)
    ref = O.ema_loop(X, A)
    assert torch.allclose(y, ref, rtol=1e-10, atol=1e-12)
    assert torch.allclose(final, ref[:, -1], rtol=1e-10, atol=1e-12)
    # prev[c] is the sequential state just before chunk c
    C = cs.shape[1]
    for c in range(1, C):
        assert torch.allclose(prev[:, c], ref[:, c * Q - 1], rtol=1e-10, atol=1e-12)
    assert torch.equal(prev[:, 0], torch.zeros_like(prev[:, 0]))


def test_cumsum_restarts_and_pads():
    A = -torch.arange(1, 11, dtype=F64).reshape(1, 10)
    cs = O.chunk_cumsum(A, 4)
    assert cs.shape == (1, 3, 4)
    assert cs[0, 0].tolist() == [-1, -3, -6, -10]
    assert cs[0, 1].tolist() == [-5, -11, -18, -26]
    assert cs[0, 2].tolist() == [-9, -19, -19, -19]  # the tail repeats the last valid sum


def test_chunk_state_is_local_scan_end():
    A, X, _ = rand_case(2, 48, 3, seed=20)
    Q = 16
    cs = O.chunk_cumsum(A, Q)
    st = O.chunk_state(X, cs)
    for c in range(3):
        sl = slice(c * Q, (c + 1) * Q)
        local = O.ema_loop(X[:, sl], A[:, sl])
        assert torch.allclose(st[:, c], local[:, -1], rtol=1e-10, atol=1e-12)


def test_chunk_size_invariance():
    A, X, dy = rand_case(2, 96, 3, seed=21)
    outs = [O.combined_fwd(A, X, Q)[0] for Q in (8, 32, 96, 128)]
    for o in outs[1:]:
        assert torch.allclose(o, outs[0], rtol=1e-10, atol=1e-12)
    grads = []
    for Q in (8, 32, 96, 128):
        dx, ddA = O.combined_bwd(dy, X, A, Q)
        grads.append((dx, ddA.reshape(2, -1)[:, :96]))
    for dx, dA in grads[1:]:
        assert torch.allclose(dx, grads[0][0], rtol=1e-10, atol=1e-12)
        assert torch.allclose(dA, grads[0][1], rtol=1e-9, atol=1e-11)


def test_forward_linearity_in_x():
    A, X, X2 = rand_case(1, 40, 3, seed=22)
    f = lambda X_: O.combined_fwd(A, X_, 16)[0]
    assert torch.allclose(f(2.5 * X - X2), 2.5 * f(X) - f(X2), rtol=1e-10, atol=1e-12)


# ---------------------------------------------------------------- chunked backward stages


@pytest.mark.parametrize("L,Q", [(64, 16), (70, 16), (128, 128), (33, 64), (2, 2)])
def test_chunked_backward_equals_autograd(L, Q):
    A, X, dy = rand_case(2, L, 4, seed=30 + L)
    A.requires_grad_()
    X.requires_grad_()
    (O.ema_loop(X, A) * dy).sum().backward()
    dx, ddA = O.combined_bwd(dy, X.detach(), A.detach(), Q)
    assert torch.allclose(dx, X.grad, rtol=1e-9, atol=1e-11)
    assert torch.allclose(ddA.reshape(2, -1)[:, :L], A.grad, rtol=1e-8, atol=1e-10)


def _stage_inputs(seed, N=2, L=48, T=3, Q=16):
    A, X, dy = rand_case(N, L, T, seed=seed)
    cs = O.chunk_cumsum(A, Q)
    states = O.chunk_state(X, cs)
    prev, _ = O.state_passing(states, cs[..., -1])
    return A, X, dy, cs, states, prev


def test_dstates_is_grad_of_scan_wrt_prev():
    A, X, dy, cs, states, prev = _stage_inputs(40)
    p = prev.clone().requires_grad_()
    (O.chunk_scan(X, cs, p) * dy).sum().backward()
    assert torch.allclose(O.bwd_dstates(cs, dy), p.grad, rtol=1e-10, atol=1e-12)


def test_state_passing_bwd_is_autograd_of_state_passing():
    A, X, dy, cs, states, prev = _stage_inputs(41)
    ds = torch.randn_like(prev)
    st = states.clone().requires_grad_()
    cl = cs[..., -1].clone().requires_grad_()
    p, _ = O.state_passing(st, cl)
    (p * ds).sum().backward()
    g, ddA_chunk = O.state_passing_bwd(prev, cs[..., -1], ds)
    assert torch.allclose(g, st.grad, rtol=1e-10, atol=1e-12)
    # d/d cs_last[c] reaches prev[c+1..]; index 0 has no incoming state
    want = cl.grad.clone()
    assert torch.allclose(ddA_chunk[:, 1:], want[:, 1:], rtol=1e-10, atol=1e-12)
    assert torch.equal(ddA_chunk[:, 0], torch.zeros_like(ddA_chunk[:, 0]))
    assert torch.allclose(want[:, 0], torch.zeros_like(want[:, 0]), atol=1e-14)


def test_dx_is_grad_wrt_x_given_g():
    # dL/dX = direct path through the scan + path through states with upstream g
    A, X, dy, cs, states, prev = _stage_inputs(42)
    g = torch.randn_like(prev)
    x = X.clone().requires_grad_()
    loss = (O.chunk_scan(x, cs, prev) * dy).sum() + (O.chunk_state(x, cs) * g).sum()
    loss.backward()
    assert torch.allclose(O.bwd_dx(cs, dy, g), x.grad, rtol=1e-10, atol=1e-12)


def test_db_is_grad_of_chunk_state_wrt_A():
    # restates kernels/tests/ema_bwd/test_ema_chunk_state_bwd_db.py:22-33,94-96
    A, X, dy, cs, states, prev = _stage_inputs(43)
    g = torch.randn_like(prev)
    N, L, T = X.shape
    Q = cs.shape[-1]
    a = A.reshape(N, -1, Q).clone().requires_grad_()
    csa = torch.cumsum(a, -1)
    scale = torch.exp(torch.clamp(csa[..., -1:] - csa, max=0.0))
    st = torch.einsum("ncq,ncqt->nct", scale, X.reshape(N, -1, Q, T))
    (st * g).sum().backward()
    assert torch.allclose(O.bwd_db(X, cs, g), a.grad, rtol=1e-10, atol=1e-12)
    raw = O.bwd_db(X, cs, g, raw=True)
    assert torch.equal(raw[..., 0], torch.zeros_like(raw[..., 0]))
    assert torch.allclose(torch.cumsum(raw, -1), a.grad, rtol=1e-10, atol=1e-12)


def test_dc_is_grad_of_prev_term_wrt_cs_and_A():
    # restates kernels/tests/ema_bwd/test_ema_chunk_scan_bwd_dc.py:7-20,83
    A, X, dy, cs, states, prev = _stage_inputs(44)
    N, L, T = X.shape
    Q = cs.shape[-1]
    c = cs.clone().requires_grad_()
    out = torch.exp(torch.clamp(c, max=0.0))[..., None] * prev[:, :, None, :]
    (out * dy.reshape(N, -1, Q, T)).sum().backward()
    s = O.bwd_dc(prev, cs, dy)
    assert torch.allclose(s, c.grad, rtol=1e-10, atol=1e-12)
    a = A.reshape(N, -1, Q).clone().requires_grad_()
    out = torch.exp(torch.cumsum(a, -1))[..., None] * prev[:, :, None, :]
    (out * dy.reshape(N, -1, Q, T)).sum().backward()
    assert torch.allclose(s.flip([-1]).cumsum(-1).flip([-1]), a.grad, rtol=1e-10, atol=1e-12)


def test_da_intra_is_grad_of_masked_segsum_matmul():
    # restates kernels/tests/ema_bwd/test_ema_scan_da.py:8-15
    A, X, dy, cs, states, prev = _stage_inputs(45)
    N, L, T = X.shape
    Q = cs.shape[-1]
    a = A.reshape(N, -1, Q).clone().requires_grad_()
    csa = torch.cumsum(a, -1)
    seg = torch.tril(torch.exp(torch.clamp(csa[..., :, None] - csa[..., None, :], max=0.0)))
    out = seg @ X.reshape(N, -1, Q, T)
    (out * dy.reshape(N, -1, Q, T)).sum().backward()
    got = O.bwd_da_intra(X, cs, dy)
    assert torch.allclose(got, a.grad, rtol=1e-10, atol=1e-12)
    assert torch.equal(got[..., 0], torch.zeros_like(got[..., 0]))


def test_da_intra_brute_force_tiny():
    A, X, dy = rand_case(1, 6, 2, seed=46)
    cs = O.chunk_cumsum(A, 6)
    got = O.bwd_da_intra(X, cs, dy)[0, 0]
    for j in range(6):
        want = 0.0
        for m in range(j, 6):
            for k in range(j):
                w = math.exp(float(cs[0, 0, m] - cs[0, 0, k]))
                want += w * float((dy[0, m] * X[0, k]).sum())
        assert abs(float(got[j]) - want) < 1e-12


# ---------------------------------------------------------------- layouts and fp32


def test_headed_layout_round_trip():
    x = torch.randn(2, 7, 3, 4)
    A = -torch.rand(2, 7, 3)
    xf, Af = O.to_flat(x, A)
    assert xf.shape == (6, 7, 4) and Af.shape == (6, 7)
    assert torch.equal(xf[1 * 3 + 2], x[1, :, 2])
    assert torch.equal(Af[1 * 3 + 2], A[1, :, 2])
    assert torch.equal(O.from_flat(xf, 2, 3), x)


def test_fp32_oracle_close_to_fp64():
    x, A, dy = O.make_inputs(1, 2, 512, 64, seed=7, scale_x=True)
    xf, Af = O.to_flat(x, A)
    dyf, _ = O.to_flat(dy, A)
    y32 = O.ema_loop(xf, Af)
    y64 = O.ema_loop(xf.double(), Af.double())
    assert torch.allclose(y32.double(), y64, rtol=1e-5, atol=1e-6)
    dx32, dA32 = O.combined_bwd(dyf, xf, Af, 128)
    dx64, dA64 = O.ema_loop_bwd(dyf.double(), xf.double(), Af.double())
    assert torch.allclose(dx32.double(), dx64, rtol=1e-4, atol=1e-5)
    assert torch.allclose(dA32.reshape(2, -1).double(), dA64, rtol=1e-4, atol=1e-4)


# ---------------------------------------------------------------- sequence-level forms


def _seq_inputs(N=3, L=37, T=5, seed=0, dtype=torch.float64):
    gen = torch.Generator().manual_seed(seed)
    X = torch.randn(N, L, T, generator=gen, dtype=dtype)
    p = torch.sigmoid(torch.randn(N, L, generator=gen, dtype=dtype) - 1.0)
    init = torch.randn(N, T, generator=gen, dtype=dtype)
    dy = torch.randn(N, L, T, generator=gen, dtype=dtype)
    dfinal = torch.randn(N, T, generator=gen, dtype=dtype)
    return X, p, init, dy, dfinal


def test_seq_probability_form_is_log_decay_form_of_scaled_input():
    # the change of variables the reference's bench applies (ema_bench.py:135-136)
    X, p, *_ = _seq_inputs()
    y_p, fin_p = O.ema_seq_loop(X, p, "probability")
    y_a = O.ema_loop(p[..., None] * X, torch.log1p(-p))
    assert torch.allclose(y_p, y_a, rtol=1e-12, atol=1e-12)
    assert torch.allclose(fin_p, y_a[:, -1], rtol=1e-12, atol=1e-12)


def test_seq_constant_probability_closed_form():
    # z_t = sum_k p (1-p)^(t-k) x_k + (1-p)^(t+1) init
    N, L, T, p0 = 2, 20, 3, 0.3
    gen = torch.Generator().manual_seed(3)
    X = torch.randn(N, L, T, generator=gen, dtype=torch.float64)
    init = torch.randn(N, T, generator=gen, dtype=torch.float64)
    y, fin = O.ema_seq_loop(X, torch.full((N, L), p0, dtype=torch.float64), "probability", init)
    for t in (0, 7, L - 1):
        want = sum(p0 * (1 - p0) ** (t - k) * X[:, k] for k in range(t + 1)) + (1 - p0) ** (t + 1) * init
        assert torch.allclose(y[:, t], want, rtol=1e-12, atol=1e-12)
    assert torch.equal(fin, y[:, -1])


def test_seq_initial_state_is_an_extra_first_row():
    # a scan from state s equals the scan of [s, x_0, x_1, ...] from zero, first output dropped
    X, p, init, *_ = _seq_inputs()
    A = torch.log1p(-p)
    y, _ = O.ema_seq_loop(X, A, "log_decay", init)
    Xe = torch.cat([init[:, None], X], 1)
    Ae = torch.cat([torch.zeros_like(A[:, :1]), A], 1)
    assert torch.allclose(y, O.ema_loop(Xe, Ae)[:, 1:], rtol=1e-12, atol=1e-12)


def test_seq_log_decay_clamps_positive_values():
    X, p, *_ = _seq_inputs()
    A = torch.log1p(-p)
    A[:, 5] = 0.7
    y, _ = O.ema_seq_loop(X, A, "log_decay")
    A0 = A.clone()
    A0[:, 5] = 0.0
    assert torch.equal(y, O.ema_seq_loop(X, A0, "log_decay")[0])


@pytest.mark.parametrize("form", ["log_decay", "probability"])
@pytest.mark.parametrize("with_states", [False, True])
def test_seq_bwd_matches_autograd(form, with_states):
    X, p, init, dy, dfinal = _seq_inputs()
    coef = p if form == "probability" else torch.log1p(-p)
    Xr, cr = X.clone().requires_grad_(), coef.clone().requires_grad_()
    ir = init.clone().requires_grad_() if with_states else None
    y, fin = O.ema_seq_loop(Xr, cr, form, ir)
    loss = (y * dy).sum() + ((fin * dfinal).sum() if with_states else 0.0)
    loss.backward()
    dX, dc, dinit = O.ema_seq_loop_bwd(dy, X, coef, form, init if with_states else None,
                                       dfinal if with_states else None)
    assert torch.allclose(dX, Xr.grad, rtol=1e-10, atol=1e-10)
    assert torch.allclose(dc, cr.grad, rtol=1e-10, atol=1e-10)
    if with_states:
        assert torch.allclose(dinit, ir.grad, rtol=1e-10, atol=1e-10)


def test_seq_bwd_finite_differences_probability():
    X, p, init, dy, dfinal = _seq_inputs(N=1, L=9, T=2)
    _, dp, dinit = O.ema_seq_loop_bwd(dy, X, p, "probability", init, dfinal)

    def loss(pp, ii):
        y, fin = O.ema_seq_loop(X, pp, "probability", ii)
        return float((y * dy).sum() + (fin * dfinal).sum())

    eps = 1e-6
    for t in (0, 4, 8):
        d = torch.zeros_like(p)
        d[0, t] = eps
        assert math.isclose((loss(p + d, init) - loss(p - d, init)) / (2 * eps), float(dp[0, t]), rel_tol=1e-6, abs_tol=1e-8)
    d = torch.zeros_like(init)
    d[0, 1] = eps
    assert math.isclose((loss(p, init + d) - loss(p, init - d)) / (2 * eps), float(dinit[0, 1]), rel_tol=1e-6, abs_tol=1e-8)


def test_seq_probability_gradient_is_chain_rule_of_log_decay_gradient():
    # dp = <dX_scaled, x> - dA / (1 - p): the relation the reference leaves commented out
    # (kernels/tests/ema_bwd/_ema_full_bwd.py:128-130) plus the input-scaling term
    X, p, _, dy, _ = _seq_inputs()
    dXs, dA = O.ema_loop_bwd(dy, p[..., None] * X, torch.log1p(-p))
    _, dp, _ = O.ema_seq_loop_bwd(dy, X, p, "probability")
    want = (dXs * X).sum(-1) - dA / (1 - p)
    assert torch.allclose(dp, want, rtol=1e-10, atol=1e-10)
