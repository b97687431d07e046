"""Shared helpers of the GPU parity tests."""
import sys

import torch

from oracle import ema_oracle as O

# Tolerances of the parity bar.
#   float32 inputs: rtol 1e-4; the absolute term is 1e-5 of the largest reference
#     magnitude of the compared tensor (an allclose with rtol alone would reject every
#     element that is near zero by cancellation).
#   bfloat16 inputs, float32 accumulation: atol 2e-2, rtol 1e-2 on y, dx and dA.
F32_RTOL = 1e-4
F32_ATOL_REL = 1e-5
BF16_ATOL = 2e-2
BF16_RTOL = 1e-2


def announce(msg):
    print("\n[case] " + msg, flush=True)
    sys.stdout.flush()


def check_close(name, got, ref, dtype, loose=False, regrouped=False):
    """Asserts got ~= ref under the bar for `dtype` and prints the measured error.  With
    loose the absolute term of the bfloat16 bar becomes 1 % of the largest reference magnitude:
    for comparisons with a reference that skips roundings the checked arithmetic is required
    to make (the tight comparison is then the one with a reference that makes them too).
    With regrouped it becomes 0.4 % of the largest reference magnitude (2^-8: one bfloat16
    rounding on each of the two operands of a product): for two computations that round the
    same operands to bfloat16 at different points of the same sum, so that their rounding
    errors, which scale with the terms of the sum and not with its value, do not cancel."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    scale = max(1.0, float(ref.abs().max()))
    if dtype == torch.float32:
        atol, rtol = F32_ATOL_REL * scale, F32_RTOL
    else:
        atol, rtol = BF16_ATOL, BF16_RTOL
        if loose:
            atol = max(atol, 1e-2 * scale)
        elif regrouped:
            atol = max(atol, 2.0 ** -8 * scale)
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs()
    worst = float((err / bound).max())
    print(
        f"  {name}: max|err|={float(err.max()):.3e} max|ref|={float(ref.abs().max()):.3e} "
        f"err/bound={worst:.3f} (atol={atol:.2e}, rtol={rtol:.0e})",
        flush=True,
    )
    assert worst <= 1.0, f"{name}: error exceeds the bar by x{worst:.2f}"


def flat_case(N, L, T, seed, dtype=torch.float32, kind="sigmoid", u_mean=2.0):
    """Flat-layout inputs (A:(N,L) f32, X:(N,L,T) dtype, dy like X), generated on the CPU."""
    g = torch.Generator().manual_seed(seed)
    if kind == "sigmoid":
        A = torch.nn.functional.logsigmoid(torch.randn(N, L, generator=g) + u_mean)
    elif kind == "neg_rand":  # A = -rand, as kernels/tests/ema_bwd/_ema_full_bwd.py:50-51
        A = -torch.rand(N, L, generator=g)
    else:
        raise ValueError(kind)
    X = torch.randn(N, L, T, generator=g).to(dtype)
    dy = torch.randn(N, L, T, generator=g).to(dtype)
    return A, X, dy


def oracle_intermediates(A, X, dy, Q):
    """All chunked intermediates of the oracle in float32 on the CPU."""
    Xf, dyf = X.float(), dy.float()
    cs = O.chunk_cumsum(A, Q)
    states = O.chunk_state(Xf, cs)
    prev, final = O.state_passing(states, cs[..., -1])
    ds = O.bwd_dstates(cs, dyf)
    g, ddA_chunk = O.state_passing_bwd(prev, cs[..., -1], ds)
    return dict(cs=cs, states=states, prev=prev, final=final, ds=ds, g=g, ddA_chunk=ddA_chunk)
