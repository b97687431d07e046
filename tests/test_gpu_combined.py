"""GPU parity of the combined forward / backward and of the autograd entry point against
the sequential CPU oracle, including benchmark configurations 1-4 at their full sizes."""
import pytest
import torch

from oracle import ema_oracle as O
from parity_util import announce, check_close, flat_case

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16


def _run_flat(A, X, dy, Q, device, recompute_output=False):
    from kernels.ema_kernels.ema_combined_fwd import _ema_matmul_scan_combined_fwd
    from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_chunk_scan_combined_bwd

    Ad, Xd, dyd = A.to(device), X.to(device), dy.to(device)
    y, cs, prev, final = _ema_matmul_scan_combined_fwd(Ad, Xd, Q)
    res = _ema_chunk_scan_combined_bwd(dyd, Xd, Ad, Q, recompute_output=recompute_output)
    torch.cuda.synchronize()
    return y, cs, prev, final, res


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize(
    "N,L,T,Q,kind",
    [
        (4, 2048, 512, 128, "neg_rand"),  # tests/ema_bwd/_ema_full_bwd.py:56-79, L shortened
        (2, 1000, 64, 128, "sigmoid"),    # ragged
        (2, 640, 136, 64, "sigmoid"),
        (1, 2048, 128, 512, "sigmoid"),
        (3, 200, 8, 256, "sigmoid"),      # one ragged chunk
        (2, 1, 8, 128, "sigmoid"),        # L = 1
    ],
)
def test_combined_vs_sequential(N, L, T, Q, kind, dtype, device):
    announce(f"combined N{N} L{L} T{T} Q{Q} {kind} {dtype}")
    A, X, dy = flat_case(N, L, T, seed=77 + L + T, dtype=dtype, kind=kind)
    y, cs, prev, final, (dx, ddA, y2) = _run_flat(A, X, dy, Q, device, recompute_output=True)
    y_ref = O.ema_loop(X.float(), A)
    dx_ref, dA_ref = O.ema_loop_bwd(dy.float(), X.float(), A)
    check_close("y", y, y_ref, dtype)
    check_close("y (recomputed in bwd)", y2, y_ref, dtype)
    check_close("final", final, y_ref[:, -1], F32 if dtype == F32 else BF16)
    check_close("dx", dx, dx_ref, dtype)
    assert ddA.shape == (N, -(-L // Q), Q) and ddA.dtype == F32
    check_close("dA", ddA.reshape(N, -1)[:, :L], dA_ref, dtype)
    C = cs.shape[1]
    ref_prev = torch.stack([y_ref[:, c * Q - 1] if c else torch.zeros(N, T) for c in range(C)], 1)
    check_close("prev", prev, ref_prev, F32 if dtype == F32 else BF16)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("N,L,T,Q", [(2, 1024, 256, 128), (2, 900, 64, 256), (1, 512, 128, 64)])
def test_staged_backward_composition(N, L, T, Q, dtype, device):
    """The stage launchers, glued as in kernels/ema_kernels_bwd/ema_combined_bwd.py:32-83 of
    the reference, give the same gradients as the single-call backward and the oracle."""
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd
    from kernels.ema_kernels.ema_state_fwd import _ema_chunk_state_fwd
    from kernels.ema_kernels.ema_state_pass import _ema_state_passing_fwd
    from kernels.ema_kernels_bwd.ema_chunk_scan_bwd_dc import _ema_chunk_scan_bwd_dC
    from kernels.ema_kernels_bwd.ema_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx
    from kernels.ema_kernels_bwd.ema_chunk_state_bwd_db import _ema_chunk_state_bwd_db
    from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_chunk_scan_combined_bwd
    from kernels.ema_kernels_bwd.ema_scan_bwd import _ema_chunk_scan_bwd_dstates
    from kernels.ema_kernels_bwd.ema_scan_da import _ema_chunk_scan_bwd_ddAcs_stable
    from kernels.ema_kernels_bwd.ema_state_passing_bwd_dstates import _ema_state_passing_bwd

    announce(f"staged backward N{N} L{L} T{T} Q{Q} {dtype}")
    A, X, dy = flat_case(N, L, T, seed=300 + L, dtype=dtype)
    Ad, Xd, dyd = A.to(device), X.to(device), dy.to(device)
    cs = ema_chunk_cumsum_fwd(Ad, Q)
    states = _ema_chunk_state_fwd(Xd, cs)
    prev, _ = _ema_state_passing_fwd(states, cs[..., -1], out_dtype=torch.float32)
    ds = _ema_chunk_scan_bwd_dstates(cs, dyd)
    g, ddA_chunk, _ = _ema_state_passing_bwd(prev, cs[..., -1], ds, chunk_size=Q)
    dx = _chunk_scan_chunk_state_bwd_dx(Xd, cs, dyd, g)
    ddA_next = _ema_chunk_state_bwd_db(Xd, cs, g)
    ddA_prev = _ema_chunk_scan_bwd_dC(prev, cs, dyd)
    ddA_prev[..., -1] += ddA_chunk
    ddA_prev = ddA_prev.flip([-1]).cumsum(dim=-1).flip([-1])
    ddA = _ema_chunk_scan_bwd_ddAcs_stable(Xd, cs, dyd) + ddA_next + ddA_prev
    dx_ref, dA_ref = O.ema_loop_bwd(dy.float(), X.float(), A)
    check_close("dx staged", dx, dx_ref, dtype)
    check_close("dA staged", ddA.reshape(N, -1)[:, :L], dA_ref, dtype)
    dx1, ddA1 = _ema_chunk_scan_combined_bwd(dyd, Xd, Ad, Q)
    check_close("dx single call", dx1, dx_ref, dtype)
    check_close("dA single call", ddA1.reshape(N, -1)[:, :L], dA_ref, dtype)
    # slots past the end of the sequence are defined as zero by the single-call backward
    assert float(ddA1.reshape(N, -1)[:, L:].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("N,L,T", [(2, 1024, 256), (2, 300, 64), (1, 128, 1024)])
def test_fused_dx_dA_stage(N, L, T, dtype, device):
    """The fused backward launcher on the oracle's chunk-128 intermediates."""
    from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_bwd_dx_dA_fused
    from parity_util import oracle_intermediates

    announce(f"fused dx/dA stage N{N} L{L} T{T} {dtype}")
    A, X, dy = flat_case(N, L, T, seed=500 + L, dtype=dtype)
    it = oracle_intermediates(A, X, dy, 128)
    dx, ddA, y = _ema_bwd_dx_dA_fused(
        X.to(device), it["cs"].to(device), dy.to(device), it["prev"].to(device), it["g"].to(device),
        recompute_output=True,
    )
    dx_ref, dA_ref = O.ema_loop_bwd(dy.float(), X.float(), A)
    check_close("dx", dx, dx_ref, dtype)
    check_close("dA", ddA.reshape(N, -1)[:, :L], dA_ref, dtype)
    check_close("y", y, O.ema_loop(X.float(), A), dtype)


def _headed_reference(x, A, dy):
    b, L, nh, d = x.shape
    xf, Af = O.to_flat(x.float(), A)
    dyf, _ = O.to_flat(dy.float(), A)
    y = O.from_flat(O.ema_loop(xf, Af), b, nh)
    dx, dA = O.ema_loop_bwd(dyf, xf, Af)
    return y, O.from_flat(dx, b, nh), dA.reshape(b, nh, L).permute(0, 2, 1)


def _autograd_headed(x, A, dy, Q, device):
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    xg = x.to(device).requires_grad_()
    Ag = A.to(device).requires_grad_()
    y = ema_matmul_scan_combined(Ag, xg, Q)
    y.backward(dy.to(device))
    torch.cuda.synchronize()
    return y, xg.grad, Ag.grad


def test_config1_fp32_forward(device):
    """benchmark configuration 1: b1 nh2 L512 d64 Q128 fp32, input scaled by (1 - alpha), compared
    with y_t = alpha_t y_{t-1} + (1 - alpha_t) x_t."""
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    announce("config 1")
    x, A, _ = O.make_inputs(1, 2, 512, 64, seed=11, scale_x=False)
    xs, _, _ = O.make_inputs(1, 2, 512, 64, seed=11, scale_x=True)
    alpha = torch.exp(A)
    z = torch.zeros(1, 2, 64)
    ref = torch.empty_like(x)
    for t in range(512):
        z = alpha[:, t, :, None] * z + (1 - alpha[:, t, :, None]) * x[:, t]
        ref[:, t] = z
    y = ema_matmul_scan_combined(A.to(device), xs.to(device), 128)
    check_close("y", y, ref, F32)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
def test_autograd_headed_small(dtype, device):
    announce(f"autograd headed b2 L300 nh2 d64 {dtype}")
    x, A, dy = O.make_inputs(2, 2, 300, 64, seed=5, dtype=dtype)
    y, dx, dA = _autograd_headed(x, A, dy, 128, device)
    y_ref, dx_ref, dA_ref = _headed_reference(x, A, dy)
    assert dA.shape == A.shape and dx.shape == x.shape
    check_close("y", y, y_ref, dtype)
    check_close("dx", dx, dx_ref, dtype)
    check_close("dA", dA, dA_ref, dtype)


@pytest.mark.parametrize("Q", [128, 256, 512])
def test_config3_bf16_fwd_bwd_full_size(Q, device):
    """benchmark configurations 2 and 3: b16 nh2 d1024 L4096, bf16, chunk size swept, seed fixed per
    chunk size; forward, dx and dA against the sequential oracle at full size."""
    announce(f"config 2/3 full size Q{Q}")
    x, A, dy = O.make_inputs(16, 2, 4096, 1024, seed=1000 + Q, dtype=BF16)
    y, dx, dA = _autograd_headed(x, A, dy, Q, device)
    y_ref, dx_ref, dA_ref = _headed_reference(x, A, dy)
    check_close("y", y, y_ref, BF16)
    check_close("dx", dx, dx_ref, BF16)
    check_close("dA", dA, dA_ref, BF16)


def test_config4_long_sequence(device):
    """benchmark configuration 4: b4 nh2 d1024 L32768 Q256, bf16, u ~ N(4,1) (long memory)."""
    announce("config 4 full size")
    x, A, dy = O.make_inputs(4, 2, 32768, 1024, seed=4, dtype=BF16, u_mean=4.0)
    y, dx, dA = _autograd_headed(x, A, dy, 256, device)
    y_ref, dx_ref, dA_ref = _headed_reference(x, A, dy)
    check_close("y", y, y_ref, BF16)
    check_close("dx", dx, dx_ref, BF16)
    check_close("dA", dA, dA_ref, BF16)


def test_chunk_size_invariance_and_linearity_full_size(device):
    """Size-independent properties at the bench shape: the output does not depend on the
    chunk size, and the scan is linear in x."""
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    announce("invariance / linearity at b16 nh2 d1024 L4096")
    x, A, _ = O.make_inputs(16, 2, 4096, 1024, seed=21, dtype=F32, with_dy=False)
    xd, Ad = x.to(device), A.to(device)
    y128 = ema_matmul_scan_combined(Ad, xd, 128)
    y512 = ema_matmul_scan_combined(Ad, xd, 512)
    check_close("Q128 vs Q512", y128, y512, F32)
    x2 = torch.roll(xd, 1, dims=0)
    lhs = ema_matmul_scan_combined(Ad, 2.0 * xd - x2, 128)
    rhs = 2.0 * y128 - ema_matmul_scan_combined(Ad, x2, 128)
    check_close("linearity", lhs, rhs, F32)


def test_zero_log_decay_is_cumsum(device):
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    announce("A == 0")
    X = torch.randn(2, 500, 64)
    A = torch.zeros(2, 500)
    y = ema_matmul_scan_combined(A.to(device), X.to(device), 128)
    check_close("y", y, torch.cumsum(X, 1), F32)


def test_strong_decay_no_nan(device):
    """Very negative log-decays underflow to 0 instead of producing inf * 0."""
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    announce("A = -60")
    X = torch.randn(1, 256, 64)
    A = torch.full((1, 256), -60.0)
    y = ema_matmul_scan_combined(A.to(device), X.to(device), 128)
    check_close("y", y, O.ema_loop(X, A), F32)


def test_error_behaviour(device):
    """Same refusals as the reference launchers."""
    from kernels.ema_kernels.ema_state_pass import _ema_state_passing_fwd
    from kernels.ema_kernels.ema_state_fwd import _ema_chunk_state_fwd
    from kernels.ema_kernels_bwd.ema_state_passing_bwd_dstates import _ema_state_passing_bwd

    st = torch.zeros(2, 3, 8, device=device)
    cl = torch.zeros(2, 3, device=device)
    with pytest.raises(NotImplementedError):  # kernels/ema_kernels/ema_state_pass.py:129-130
        _ema_state_passing_fwd(st, cl, initial_states=torch.zeros(2, 8, device=device))
    with pytest.raises(AssertionError):
        _ema_state_passing_fwd(st, torch.zeros(2, 4, device=device))
    with pytest.raises(AssertionError):  # ...state_passing_bwd_dstates.py:120-122
        _ema_state_passing_bwd(st, cl, st, dfinal_states=torch.zeros(2, 8, device=device))
    with pytest.raises(AssertionError):  # kernels/ema_kernels/ema_state_fwd.py:135-140
        _ema_chunk_state_fwd(torch.zeros(2, 24, 8, device=device), torch.zeros(2, 2, 8, device=device))
    with pytest.raises(AssertionError):  # feature size must allow 16-byte rows
        _ema_chunk_state_fwd(torch.zeros(2, 16, 6, device=device), torch.zeros(2, 2, 8, device=device))


def test_legacy_probability_entry_point(device):
    """ema_scan_combined(x, p) against z_t = (1-p) z_{t-1} + p x_t (main.py:120-131 of the reference)."""
    from kernels.ema import ema_scan_combined

    announce("ema_scan_combined(x, p)")
    g = torch.Generator().manual_seed(3)
    X = torch.randn(2, 300, 64, generator=g)
    P = torch.rand(2, 300, 1, generator=g) * 0.98 + 0.01
    ref = torch.empty_like(X)
    zprev = torch.zeros(2, 64)
    for t in range(300):
        zprev = (1 - P[:, t]) * zprev + P[:, t] * X[:, t]
        ref[:, t] = zprev
    got = ema_scan_combined(X.to(device), P.to(device))
    check_close("z", got, ref, F32)


def test_legacy_mamba_encoded_entry_point(device):
    """ema_chunk_scan_combined with the encoding of main.py:92-98 of the reference
    (dt = -log(1-p), B = p, C = 1, x / dt) reproduces the EMA loop."""
    from kernels.ema_combined import ema_chunk_scan_combined

    announce("ema_chunk_scan_combined(x, dt, A, B, C)")
    g = torch.Generator().manual_seed(4)
    b, L, nh, hd = 2, 260, 2, 32
    X = torch.randn(b, L, nh * hd, generator=g)
    P = torch.rand(b, L, 1, generator=g) * 0.9 + 0.05
    ref = torch.empty_like(X)
    zprev = torch.zeros(b, nh * hd)
    for t in range(L):
        zprev = (1 - P[:, t]) * zprev + P[:, t] * X[:, t]
        ref[:, t] = zprev
    dt = -torch.log(1 - P).squeeze(-1)
    X_m = (X / dt[..., None]).reshape(b, L, nh, hd)
    dt_h = dt[..., None].expand(b, L, nh).contiguous()
    A = -torch.ones(nh)
    B_m = P.reshape(b, L, 1, 1)
    C_m = torch.ones_like(B_m)
    out, final = ema_chunk_scan_combined(
        X_m.to(device), dt_h.to(device), A.to(device), B_m.to(device), C_m.to(device), 64,
        return_final_states=True,
    )
    check_close("out", out.reshape(b, L, nh * hd), ref, F32)
    check_close("final", final.reshape(b, nh * hd), ref[:, -1], F32)
    # anything but the EMA encoding (here a state of 4, D, z and an initial state) is the general
    # recurrence with dA = -dt, whatever A holds (kernels/ema_chunk_state.py:95 of the reference)
    from oracle import ssd_oracle as S

    g2 = torch.Generator().manual_seed(5)
    Bg, Cg = torch.randn(b, L, 1, 4, generator=g2), torch.randn(b, L, 1, 4, generator=g2)
    D, z = torch.randn(nh, generator=g2), torch.randn(b, L, nh, hd, generator=g2)
    init = torch.randn(b, nh, hd, 4, generator=g2)
    y_ref, fin_ref = S.ssd_loop(X_m, dt_h, -torch.ones(nh), Bg, Cg, D, z, init)
    out, final = ema_chunk_scan_combined(
        X_m.to(device), dt_h.to(device), torch.full((nh,), -3.0, device=device), Bg.to(device), Cg.to(device), 64,
        D=D.to(device), z=z.to(device), initial_states=init.to(device), return_final_states=True)
    check_close("general case: out", out, y_ref, F32)
    check_close("general case: final", final, fin_ref, F32)
    # the state at the end of each packed sequence (a batch of 1): every sequence on its own
    cu = torch.tensor([0, 70, 200, L], dtype=torch.int32)
    seq = torch.repeat_interleave(torch.arange(3, dtype=torch.int32), cu.diff())[None]
    one = lambda t: t[:1].to(device)
    out, varlen = ema_chunk_scan_combined(one(X_m), one(dt_h), A.to(device), one(Bg), one(Cg), 64, seq_idx=seq.to(device),
                                          cu_seqlens=cu.to(device), return_varlen_states=True)
    assert varlen.shape == (3, nh, hd, 4)
    for i in range(3):
        sl = slice(int(cu[i]), int(cu[i + 1]))
        y_i, fin_i = S.ssd_loop(X_m[:1, sl], dt_h[:1, sl], -torch.ones(nh), Bg[:1, sl], Cg[:1, sl])
        check_close(f"packed sequence {i}: out", out[:, sl], y_i, F32)
        check_close(f"packed sequence {i}: end state", varlen[i], fin_i[0], F32)
    with pytest.raises(AssertionError):
        ema_chunk_scan_combined(one(X_m), one(dt_h), A.to(device), one(Bg), one(Cg), 64, return_varlen_states=True)
