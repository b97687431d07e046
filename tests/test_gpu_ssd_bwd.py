"""GPU parity of the Mamba-2 SSD backward stages (through the C ABI) against the CPU oracle's
restatements, which tests/test_ssd_oracle.py pins by autograd.  bfloat16 cases compare with the
oracle making the roundings the reference makes before its dots."""
import pytest
import torch

from oracle import ssd_oracle as S
from parity_util import announce, check_close

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16

CASES = [
    # b, L, nh, P, g, N, Q
    (2, 300, 4, 64, 1, 64, 64),
    (1, 256, 4, 64, 2, 128, 128),
    (2, 200, 4, 64, 1, 128, 256),   # one ragged chunk
    (1, 520, 2, 128, 1, 64, 128),
    (1, 130, 2, 128, 2, 128, 64),
    (1, 900, 2, 64, 1, 64, 512),
    (1, 150, 2, 64, 1, 64, 48),     # chunk sizes that are no multiple of the 64-row tiles
    (1, 333, 2, 64, 2, 64, 200),
    (1, 1100, 2, 64, 1, 128, 1024),  # the largest chunk size, second chunk ragged
    (1, 320, 7, 64, 1, 128, 64),    # seven heads in a group: the three head slots of the dB / dC kernel wrap twice
    (1, 192, 2, 64, 2, 128, 64),    # one head per group
    # head and state sizes the kernels do not take natively (split into sub-heads / zero-padded
    # around them); the reference's EMA tests and benchmarks call its Mamba launchers with
    # dstate = 1 and head sizes 8, 32 and 512
    (1, 200, 2, 32, 1, 1, 64),
    (1, 300, 2, 512, 1, 1, 128),
    (2, 150, 4, 8, 2, 16, 64),
    (1, 260, 2, 200, 1, 100, 256),
    (1, 100, 2, 6, 1, 1, 32),
]


def _inputs(b, L, nh, P, g, N, Q, dtype):
    x, dt_raw, A, B, C, D, _ = S.make_inputs(b, L, nh, P, g, N, seed=2 * L + N + Q, dtype=dtype)
    dA_cs, dt = S.chunk_cumsum(dt_raw, A, Q)
    gen = torch.Generator().manual_seed(L + Q)
    dout = torch.randn(b, L, nh, P, generator=gen).to(dtype)
    nc = dt.shape[2]
    prev = torch.randn(b, nc, nh, P, N, generator=gen)
    dstates = torch.randn(b, nc, nh, P, N, generator=gen)
    return x, dt, dA_cs, B, C, D, dout, prev, dstates


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_dstates_db_dc_vs_oracle(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_dc import _chunk_scan_bwd_dC
    from kernels.mamba_kernels_bwd.mamba_chunk_state_bwd_db import _chunk_state_bwd_db
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates

    announce(f"ssd bwd dstates/db/dc b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, dA_cs, B, C, D, dout, prev, dstates = _inputs(b, L, nh, P, g, N, Q, dtype)
    rt = None if dtype == F32 else dtype
    d = lambda t: t.to(device)

    got = _chunk_scan_bwd_dstates(d(C), d(dA_cs), d(dout), dtype=torch.float32)
    check_close("dprev_states", got, S.bwd_dstates(C, dA_cs, dout, round_to=rt), dtype)
    if dtype == BF16:  # stored in the inputs' type by the kernel: the rounded float32 result
        got16 = _chunk_scan_bwd_dstates(d(C), d(dA_cs), d(dout))
        assert got16.dtype == BF16 and torch.equal(got16, got.to(BF16))

    dB_ref, ddA_ref = S.chunk_state_bwd_db(x, dt, dA_cs, dstates, B=B, ngroups=g, round_to=rt)
    dB, ddA = _chunk_state_bwd_db(d(x), d(dt), d(dA_cs), d(dstates), B=d(B), ngroups=g)
    check_close("dB", dB, dB_ref, dtype)
    check_close("ddA_cumsum (chunk state)", ddA, ddA_ref, dtype)
    check_close("dB without B", _chunk_state_bwd_db(d(x), d(dt), d(dA_cs), d(dstates), ngroups=g), dB_ref, dtype)
    if dtype == BF16:  # gradient states already in bfloat16: the product rounds them there either way
        dB16, ddA16 = _chunk_state_bwd_db(d(x), d(dt), d(dA_cs), d(dstates).to(BF16), B=d(B), ngroups=g)
        assert torch.equal(dB16, dB) and torch.equal(ddA16, ddA)
        dB16n = _chunk_state_bwd_db(d(x), d(dt), d(dA_cs), d(dstates).to(BF16), ngroups=g)  # no B: no row sums asked for
        assert torch.equal(dB16n if not isinstance(dB16n, tuple) else dB16n[0], dB)

    dC_ref, ddAp_ref = S.chunk_scan_bwd_dC(prev, dA_cs, dout, C=C, ngroups=g, round_to=rt)
    dC, ddAp = _chunk_scan_bwd_dC(d(prev), d(dA_cs), d(dout), C=d(C), ngroups=g)
    check_close("dC", dC, dC_ref, dtype)
    check_close("ddA_cumsum_prev", ddAp, ddAp_ref, dtype)
    if dtype == BF16:  # carried states already in bfloat16: the product rounds them there either way
        dC16, ddAp16 = _chunk_scan_bwd_dC(d(prev).to(BF16), d(dA_cs), d(dout), C=d(C), ngroups=g)
        assert torch.equal(dC16, dC) and torch.equal(ddAp16, ddAp)
        dC16n = _chunk_scan_bwd_dC(d(prev).to(BF16), d(dA_cs), d(dout), ngroups=g)  # no C: no row sums asked for
        assert torch.equal(dC16n if not isinstance(dC16n, tuple) else dC16n[0], dC)


@pytest.mark.parametrize("has_init", [False, True])
@pytest.mark.parametrize("b,nc,nh,dim", [(2, 5, 3, 64 * 64), (1, 33, 2, 64 * 128), (1, 1, 1, 128 * 128), (2, 7, 2, 100)])
def test_state_passing_bwd_vs_oracle(b, nc, nh, dim, has_init, device):
    from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd

    announce(f"ssd state passing bwd b{b} C{nc} nh{nh} dim{dim} init={has_init}")
    gen = torch.Generator().manual_seed(dim + nc)
    states = torch.randn(b, nc, nh, dim, generator=gen)
    dA = -torch.rand(b, nh, nc, generator=gen)
    dout = torch.randn(b, nc, nh, dim, generator=gen)
    dfin = torch.randn(b, nh, dim, generator=gen)
    ref = S.state_passing_bwd(states, dA, dout, dfin, has_initial_states=has_init)
    dA_view = torch.empty(b, nh, nc, 4).copy_(dA[..., None])[..., -1]  # strided, like dA_cumsum[..., -1]
    got = _state_passing_bwd(states.to(device), dA_view.to(device), dout.to(device), dfinal_states=dfin.to(device),
                             has_initial_states=has_init)
    check_close("dstates", got[0], ref[0], F32)
    check_close("ddA_chunk_cumsum", got[1], ref[1], F32)
    if has_init:
        check_close("dinitstates", got[2], ref[2], F32)
    else:
        assert got[2] is None
    got0 = _state_passing_bwd(states.to(device), dA.to(device), dout.to(device))
    ref0 = S.state_passing_bwd(states, dA, dout)
    check_close("dstates, no dfinal", got0[0], ref0[0], F32)
    # states in bfloat16 (what the combined forward keeps): read as they are, same result as their
    # float32 copy
    s16 = states.to(BF16)
    got16 = _state_passing_bwd(s16.to(device), dA.to(device), dout.to(device), dfinal_states=dfin.to(device))
    ref16 = S.state_passing_bwd(s16.float(), dA, dout, dfin)
    check_close("dstates, bfloat16 states", got16[0], ref16[0], F32)
    check_close("ddA_chunk_cumsum, bfloat16 states", got16[1], ref16[1], F32)
    # all three state-sized tensors in bfloat16 (dstates_dtype / states_dtype of the reference's
    # launcher): the recurrence itself stays in float32, only what is stored is rounded
    d16 = dout.to(BF16)
    got16 = _state_passing_bwd(s16.to(device), dA.to(device), d16.to(device), dfinal_states=dfin.to(device),
                               has_initial_states=has_init)
    ref16 = S.state_passing_bwd(s16.float(), dA, d16.float(), dfin, has_initial_states=has_init)
    assert got16[0].dtype == BF16
    check_close("dstates, all bfloat16", got16[0], ref16[0], BF16)
    check_close("ddA_chunk_cumsum, all bfloat16", got16[1], ref16[1], F32)
    mixed = _state_passing_bwd(s16.to(device), dA.to(device), d16.to(device), dfinal_states=dfin.to(device),
                               dstates_dtype=F32)
    assert mixed[0].dtype == F32
    check_close("dstates, float32 out of bfloat16 in", mixed[0], ref16[0], F32)


WALK_CASES = [
    # b, L, nh, g, Q: bfloat16, hdim 64, dstate 128 (what the single kernel is written for)
    (2, 1024, 4, 1, 256),
    (1, 700, 3, 1, 256),    # last chunk ragged: three stages, the last of them 60 rows
    (1, 520, 2, 2, 128),    # two stages per chunk, the last chunk has one stage of 8 rows
    (2, 384, 4, 2, 192),    # three stages per chunk
    (1, 1536, 2, 1, 512),
    (1, 100, 2, 1, 128),    # a single, ragged chunk
    (1, 2100, 1, 1, 1024),
]


@pytest.mark.parametrize("has_init", [False, True])
@pytest.mark.parametrize("b,L,nh,g,Q", WALK_CASES)
def test_dstates_and_state_passing_in_one_kernel(b, L, nh, g, Q, has_init, device):
    """The reverse walk against the oracle's two stages with the reference's rounding, and against
    the two launchers with a float32 tensor between them (dstates bit for bit)."""
    from kernels.mamba_kernels_bwd import mamba_scan_state_passing_bwd as M
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates
    from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd

    P, N = 64, 128
    announce(f"ssd reverse walk b{b} L{L} nh{nh} g{g} Q{Q} init={has_init}")
    x, dt, dA_cs, B, C, D, dout, prev, _ = _inputs(b, L, nh, P, g, N, Q, BF16)
    nc = dA_cs.shape[2]
    states = prev.to(BF16)
    gen = torch.Generator().manual_seed(L)
    dfin = torch.randn(b, nh, P, N, generator=gen)
    d = lambda t: t.to(device)

    fused = M._fused(d(C), d(dA_cs), d(dout), d(states), d(dfin), has_init, F32)
    assert fused is not None, "the single kernel must take this case"
    got = M._chunk_scan_state_passing_bwd(d(C), d(dA_cs), d(dout), d(states), dfinal_states=d(dfin),
                                          has_initial_states=has_init, dstates_dtype=F32)
    assert torch.equal(got[0], fused[0])

    dprev_ref = S.bwd_dstates(C, dA_cs, dout, round_to=BF16)
    ref = S.state_passing_bwd(states.float().reshape(b, nc, nh, P * N), dA_cs[..., -1],
                              dprev_ref.reshape(b, nc, nh, P * N), dfin.reshape(b, nh, P * N),
                              has_initial_states=has_init)
    check_close("dstates", got[0].reshape(b, nc, nh, P * N), ref[0], BF16)
    check_close("ddA_chunk_cumsum", got[1], ref[1], BF16)
    if has_init:
        check_close("dinitstates", got[2].reshape(b, nh, P * N), ref[2], BF16)
    else:
        assert got[2] is None

    dprev = _chunk_scan_bwd_dstates(d(C), d(dA_cs), d(dout), dtype=F32)
    two = _state_passing_bwd(d(states).reshape(b, nc, nh, P * N), d(dA_cs)[..., -1], dprev.reshape(b, nc, nh, P * N),
                             dfinal_states=d(dfin).reshape(b, nh, P * N), has_initial_states=has_init,
                             dstates_dtype=F32)
    assert torch.equal(got[0].reshape(b, nc, nh, P * N), two[0]), "dstates differ from the two launchers'"
    check_close("ddA_chunk_cumsum against the two launchers", got[1], two[1].cpu(), F32)
    if has_init:
        assert torch.equal(got[2].reshape(b, nh, P * N), two[2])

    # bfloat16 out (the type of the states) and no gradient of the final state
    got16 = M._chunk_scan_state_passing_bwd(d(C), d(dA_cs), d(dout), d(states))
    assert got16[0].dtype == BF16
    ref0 = S.state_passing_bwd(states.float().reshape(b, nc, nh, P * N), dA_cs[..., -1],
                               dprev_ref.reshape(b, nc, nh, P * N))
    check_close("dstates, bfloat16, no dfinal", got16[0].reshape(b, nc, nh, P * N), ref0[0], BF16)
    check_close("ddA_chunk_cumsum, no dfinal", got16[1], ref0[1], BF16)


def test_reverse_walk_falls_back_to_the_two_launchers(device):
    """Shapes and types the single kernel does not take go through the two launchers."""
    from kernels.mamba_kernels_bwd import mamba_scan_state_passing_bwd as M

    b, L, nh, P, g, N, Q = 1, 300, 2, 64, 1, 64, 64
    for dtype in (F32, BF16):
        x, dt, dA_cs, B, C, D, dout, prev, _ = _inputs(b, L, nh, P, g, N, Q, dtype)
        nc = dA_cs.shape[2]
        d = lambda t: t.to(device)
        assert M._fused(d(C), d(dA_cs), d(dout), d(prev.to(dtype)), None, False, F32) is None
        got = M._chunk_scan_state_passing_bwd(d(C), d(dA_cs), d(dout), d(prev.to(dtype)), has_initial_states=True,
                                              dstates_dtype=F32)
        rt = None if dtype == F32 else dtype
        ref = S.state_passing_bwd(prev.to(dtype).float().reshape(b, nc, nh, P * N), dA_cs[..., -1],
                                  S.bwd_dstates(C, dA_cs, dout, round_to=rt).reshape(b, nc, nh, P * N),
                                  has_initial_states=True)
        check_close("dstates", got[0].reshape(b, nc, nh, P * N), ref[0], F32)
        check_close("ddA_chunk_cumsum", got[1], ref[1], F32)
        check_close("dinitstates", got[2].reshape(b, nh, P * N), ref[2], F32)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_dx_vs_oracle(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx

    announce(f"ssd bwd dx b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, dA_cs, B, C, D, dout, prev, dstates = _inputs(b, L, nh, P, g, N, Q, dtype)
    rt = None if dtype == F32 else dtype
    d = lambda t: t.to(device)
    cb = S.bmm_chunk(C, B, Q)
    dx_ref, ddt_ref, dD_ref = S.chunk_scan_chunk_state_bwd_dx(x, dt, dA_cs, B, cb, dout, dstates, D=D, round_to=rt)
    dx, ddt, dD = _chunk_scan_chunk_state_bwd_dx(d(x), d(dt), d(dA_cs), d(B), d(cb), d(dout), d(dstates), D=d(D))
    check_close("dx", dx, dx_ref, dtype)
    check_close("ddt", ddt, ddt_ref, dtype, loose=dtype == BF16)
    check_close("dD", dD, dD_ref, F32)
    if dtype == BF16:  # gradient states already in bfloat16
        dx16, ddt16, _ = _chunk_scan_chunk_state_bwd_dx(d(x), d(dt), d(dA_cs), d(B), d(cb), d(dout), d(dstates).to(BF16),
                                                        D=d(D))
        assert torch.equal(dx16, dx) and torch.equal(ddt16, ddt)
    D2 = torch.randn(nh, P, generator=torch.Generator().manual_seed(1))
    dx_ref2, _, dD_ref2 = S.chunk_scan_chunk_state_bwd_dx(x, dt, dA_cs, B, cb, dout, dstates, D=D2, round_to=rt)
    dx2, _, dD2 = _chunk_scan_chunk_state_bwd_dx(d(x), d(dt), d(dA_cs), d(B), d(cb), d(dout), d(dstates), D=d(D2))
    check_close("dx (D per feature)", dx2, dx_ref2, dtype)
    check_close("dD per feature", dD2, dD_ref2, F32)
    dx3, _, none = _chunk_scan_chunk_state_bwd_dx(d(x), d(dt), d(dA_cs), d(B), d(cb), d(dout), d(dstates))
    assert none is None
    check_close("dx (no D)", dx3, S.chunk_scan_chunk_state_bwd_dx(x, dt, dA_cs, B, cb, dout, dstates, round_to=rt)[0],
                dtype)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_ddAcs_vs_oracle(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_da import _chunk_scan_bwd_ddAcs_stable

    announce(f"ssd bwd ddAcs b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, dA_cs, B, C, D, dout, prev, dstates = _inputs(b, L, nh, P, g, N, Q, dtype)
    d = lambda t: t.to(device)
    cb = S.bmm_chunk(C, B, Q)
    ref = S.chunk_scan_bwd_ddAcs_stable(x, dt, dA_cs, dout, cb)
    got = _chunk_scan_bwd_ddAcs_stable(d(x), d(dt), d(dA_cs), d(dout), d(cb))
    check_close("ddA_cumsum (causal term)", got, ref, dtype, loose=dtype == BF16)


@pytest.mark.parametrize("kind", ["steep", "rising", "mixed"])
@pytest.mark.parametrize("Q", [64, 256])
def test_ddAcs_decays_outside_the_factored_form(kind, Q, device):
    """The kernel factors exp(dA_m - dA_n) below the diagonal blocks where dA falls along the chunk,
    and inside a diagonal block where it falls by little there.  Steep decays (dA falls by far more
    than float32's exponent range inside 32 positions), rising dA (A > 0: the clamp at 0 acts) and
    dA that changes direction take the other forms; all against the oracle in float32."""
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_da import _chunk_scan_bwd_ddAcs_stable

    b, L, nh, P, g, N = 1, 2 * Q, 2, 64, 1, 64
    announce(f"ssd bwd ddAcs {kind} Q{Q}")
    x, dt_raw, A, B, C, D, _ = S.make_inputs(b, L, nh, P, g, N, seed=7 + Q, dtype=F32)
    gen = torch.Generator().manual_seed(Q)
    if kind == "steep":
        dt_raw, A = torch.full_like(dt_raw, 2.0), torch.tensor([-6.0, -1.5])
    elif kind == "rising":
        A = torch.tensor([0.5, 0.05])
    dA_cs, dt = S.chunk_cumsum(dt_raw, A, Q)
    if kind == "mixed":  # no cumsum of one sign: what the launcher is given need not come from chunk_cumsum
        dA_cs = torch.randn(dA_cs.shape, generator=gen)
    dout = torch.randn(b, L, nh, P, generator=gen)
    cb = S.bmm_chunk(C, B, Q)
    d = lambda t: t.to(device)
    ref = S.chunk_scan_bwd_ddAcs_stable(x, dt, dA_cs, dout, cb)
    got = _chunk_scan_bwd_ddAcs_stable(d(x), d(dt), d(dA_cs), d(dout), d(cb))
    check_close("ddA_cumsum (causal term)", got, ref, F32)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
def test_backward_stages_on_views(dtype, device):
    """x, B, C as slices of one projected tensor and dout as a slice of a wider gradient: the
    position strides exceed the dense ones.  Strides only change addresses, so every backward
    launcher must return exactly what it returns for contiguous copies."""
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_da import _chunk_scan_bwd_ddAcs_stable
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_dc import _chunk_scan_bwd_dC
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx
    from kernels.mamba_kernels_bwd.mamba_chunk_state_bwd_db import _chunk_state_bwd_db
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates

    b, L, nh, P, g, N, Q = 2, 520, 4, 64, 2, 128, 256
    announce(f"ssd bwd on views b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, dA_cs, B, C, D, dout, prev, dstates = [t.to(device) for t in _inputs(b, L, nh, P, g, N, Q, dtype)]
    cb = S.bmm_chunk(C.cpu(), B.cpu(), Q).to(device)
    d_in = nh * P
    xbc = torch.zeros(b, L, d_in + 2 * g * N + 8, device=device, dtype=dtype)
    xbc[..., :d_in] = x.reshape(b, L, d_in)
    xbc[..., d_in:d_in + g * N] = B.reshape(b, L, g * N)
    xbc[..., d_in + g * N:d_in + 2 * g * N] = C.reshape(b, L, g * N)
    xv = xbc[..., :d_in].unflatten(-1, (nh, P))
    Bv = xbc[..., d_in:d_in + g * N].unflatten(-1, (g, N))
    Cv = xbc[..., d_in + g * N:d_in + 2 * g * N].unflatten(-1, (g, N))
    dwide = torch.zeros(b, L, 2 * d_in, device=device, dtype=dtype)
    dwide[..., d_in:] = dout.reshape(b, L, d_in)
    dv = dwide[..., d_in:].unflatten(-1, (nh, P))
    assert not xv.is_contiguous() and not dv.is_contiguous()

    def same(name, got, want):
        got = got if isinstance(got, tuple) else (got,)
        want = want if isinstance(want, tuple) else (want,)
        for i, (a, w) in enumerate(zip(got, want)):
            assert (a is None and w is None) or torch.equal(a, w), f"{name}[{i}] differs on views"

    same("dstates", _chunk_scan_bwd_dstates(Cv, dA_cs, dv), _chunk_scan_bwd_dstates(C, dA_cs, dout))
    same("dB", _chunk_state_bwd_db(xv, dt, dA_cs, dstates, B=Bv, ngroups=g),
         _chunk_state_bwd_db(x, dt, dA_cs, dstates, B=B, ngroups=g))
    same("dC", _chunk_scan_bwd_dC(prev, dA_cs, dv, C=Cv, ngroups=g),
         _chunk_scan_bwd_dC(prev, dA_cs, dout, C=C, ngroups=g))
    same("dx", _chunk_scan_chunk_state_bwd_dx(xv, dt, dA_cs, Bv, cb, dv, dstates, D=D),
         _chunk_scan_chunk_state_bwd_dx(x, dt, dA_cs, B, cb, dout, dstates, D=D))
    same("ddA", _chunk_scan_bwd_ddAcs_stable(xv, dt, dA_cs, dv, cb), _chunk_scan_bwd_ddAcs_stable(x, dt, dA_cs, dout, cb))


def test_config5_backward_stages_full_size(device):
    """b8 nh32 hdim64 dstate128 g1 L8192 Q256 bf16: every backward launcher runs on the whole
    workload; batch element 0 of each result is compared with the oracle."""
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_da import _chunk_scan_bwd_ddAcs_stable
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_dc import _chunk_scan_bwd_dC
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx
    from kernels.mamba_kernels_bwd.mamba_chunk_state_bwd_db import _chunk_state_bwd_db
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates
    from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd

    announce("ssd config 5 backward stages, full size")
    b, L, nh, P, g, N, Q = 8, 8192, 32, 64, 1, 128, 256
    C_ = L // Q
    x, dt_raw, A, B, C, _, _ = S.make_inputs(b, L, nh, P, g, N, seed=5, dtype=BF16)
    dA_cs, dt = S.chunk_cumsum(dt_raw, A, Q)
    gen = torch.Generator().manual_seed(55)
    dout = torch.randn(b, L, nh, P, generator=gen).to(BF16)
    d = lambda t: t.to(device)
    xd, dtd, dAd, Bd, Cd, doutd = d(x), d(dt), d(dA_cs), d(B), d(C), d(dout)
    one = lambda t: t[:1]

    # forward intermediates of element 0 from the oracle (float32), the rest from the GPU
    st0 = S.chunk_state(one(B), one(x), one(dt), one(dA_cs), round_to=BF16)
    prev0, _ = S.state_passing(st0.reshape(1, C_, nh, P * N), one(dA_cs)[..., -1])
    prev0 = prev0.reshape(1, C_, nh, P, N)
    cb0 = S.bmm_chunk(one(C), one(B), Q)
    from kernels.mamba_kernels.mamba_combined_fwd import _mamba_chunk_scan_combined_fwd
    from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd
    _, _, _, _, prevd, _ = _mamba_chunk_scan_combined_fwd(xd, d(dt_raw), d(A), Bd, Cd, Q)
    cbd = _bmm_chunk_fwd(Cd, Bd, Q, output_dtype=torch.float32)
    check_close("prev states[0] (forward)", prevd[:1], prev0, BF16)

    dprev = _chunk_scan_bwd_dstates(Cd, dAd, doutd, dtype=torch.float32)
    dprev0 = S.bwd_dstates(one(C), one(dA_cs), one(dout), round_to=BF16)
    check_close("dprev_states[0]", dprev[:1], dprev0, BF16)

    dstates, ddA_chunk, _ = _state_passing_bwd(prevd.view(b, C_, nh, P * N), dAd[..., -1], dprev.view(b, C_, nh, P * N))
    ds0, ddAc0, _ = S.state_passing_bwd(prev0.reshape(1, C_, nh, P * N), one(dA_cs)[..., -1],
                                        dprev0.reshape(1, C_, nh, P * N))
    check_close("dstates[0]", dstates[:1], ds0, BF16, loose=True)
    check_close("ddA_chunk[0]", ddA_chunk[:1], ddAc0, BF16, loose=True)
    dstates5, ds05 = dstates.view(b, C_, nh, P, N), ds0.reshape(1, C_, nh, P, N)

    dB, ddA_b = _chunk_state_bwd_db(xd, dtd, dAd, dstates5, B=Bd, ngroups=g)
    dB0, ddAb0 = S.chunk_state_bwd_db(one(x), one(dt), one(dA_cs), ds05, B=one(B), ngroups=g, round_to=BF16)
    check_close("dB[0]", dB[:1], dB0, BF16, loose=True)
    check_close("ddA (chunk state)[0]", ddA_b[:1], ddAb0, BF16, loose=True)

    dC, ddA_p = _chunk_scan_bwd_dC(prevd, dAd, doutd, C=Cd, ngroups=g)
    dC0, ddAp0 = S.chunk_scan_bwd_dC(prev0, one(dA_cs), one(dout), C=one(C), ngroups=g, round_to=BF16)
    check_close("dC[0]", dC[:1], dC0, BF16, loose=True)
    check_close("ddA_prev[0]", ddA_p[:1], ddAp0, BF16, loose=True)

    dx, ddt, _ = _chunk_scan_chunk_state_bwd_dx(xd, dtd, dAd, Bd, cbd, doutd, dstates5)
    dx0, ddt0, _ = S.chunk_scan_chunk_state_bwd_dx(one(x), one(dt), one(dA_cs), one(B), cb0, one(dout), ds05, round_to=BF16)
    check_close("dx[0]", dx[:1], dx0, BF16, loose=True)
    check_close("ddt[0]", ddt[:1], ddt0, BF16, loose=True)

    ddA_s = _chunk_scan_bwd_ddAcs_stable(xd, dtd, dAd, doutd, cbd)
    check_close("ddA (causal term)[0]", ddA_s[:1], S.chunk_scan_bwd_ddAcs_stable(one(x), one(dt), one(dA_cs), one(dout), cb0),
                BF16, loose=True)
    for name, t in (("dprev", dprev), ("dstates", dstates), ("dB", dB), ("dC", dC), ("dx", dx), ("ddt", ddt), ("ddA", ddA_s)):
        assert torch.isfinite(t.float()).all(), name
