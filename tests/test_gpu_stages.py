"""GPU parity of every per-stage launcher against the CPU oracle, on seeded inputs.

The shapes follow the reference's own per-stage tests (kernels/tests/ema/*.py,
kernels/tests/ema_bwd/*.py), shortened along the sequence where the oracle's dense
(Q x Q) formulas would need gigabytes; ragged lengths, small feature sizes, the headed
layout and bf16 inputs are added.  Each launcher gets the ORACLE's intermediates as
inputs, so a stage is judged on its own.
"""
import pytest
import torch

from oracle import ema_oracle as O
from parity_util import announce, check_close, flat_case, oracle_intermediates

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16

# (N, L, T, Q): reference stage-test shapes (L shortened) plus edge cases
STAGE_SHAPES = [
    (4, 2048, 512, 128),   # tests/ema/test_ema_scan_fwd.py:118-171 (B4 T512 Q128)
    (8, 1024, 16, 32),     # tests/ema/test_ema_state_fwd.py:158-191 (T16 Q32)
    (3, 1000, 64, 128),    # ragged last chunk
    (2, 777, 72, 64),      # ragged, T not a multiple of the 64-column tile
    (2, 1024, 256, 256),   # two row tiles per chunk
    (1, 1024, 128, 512),   # four row tiles per chunk
    (2, 96, 32, 32),       # tiny
    (1, 5, 8, 16),         # a single short chunk
]


def _dev(t, device):
    return t.to(device)


@pytest.fixture(scope="module", params=[F32, BF16], ids=["f32", "bf16"])
def dtype(request):
    return request.param


@pytest.fixture(scope="module", params=STAGE_SHAPES, ids=lambda s: "N%d_L%d_T%d_Q%d" % s)
def case(request, dtype):
    N, L, T, Q = request.param
    A, X, dy = flat_case(N, L, T, seed=1000 + L + Q, dtype=dtype)
    inter = oracle_intermediates(A, X, dy, Q)
    return dict(N=N, L=L, T=T, Q=Q, A=A, X=X, dy=dy, dtype=dtype, **inter)


def test_cumsum(case, device):
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd

    announce(f"cumsum {case['N']}x{case['L']} Q{case['Q']}")
    got = ema_chunk_cumsum_fwd(_dev(case["A"], device), case["Q"])
    check_close("cs", got, case["cs"], F32)


def test_cumsum_reference_shape(device):
    # tests/ema/test_ema_cumsum.py:86-95: B8, L8197 (ragged), Q64
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd

    announce("cumsum B8 L8197 Q64")
    A, _, _ = flat_case(8, 8197, 8, seed=3)
    got = ema_chunk_cumsum_fwd(_dev(A, device), 64)
    assert got.shape == (8, 129, 64)
    check_close("cs", got, O.chunk_cumsum(A, 64), F32)
    for Q in (1, 7, 100, 1000, 1024):
        got = ema_chunk_cumsum_fwd(_dev(A, device), Q)
        check_close(f"cs Q{Q}", got, O.chunk_cumsum(A, Q), F32)


def test_chunk_state(case, device):
    from kernels.ema_kernels.ema_state_fwd import _ema_chunk_state_fwd

    announce(f"chunk_state {case['N']}x{case['L']}x{case['T']} Q{case['Q']} {case['dtype']}")
    got = _ema_chunk_state_fwd(_dev(case["X"], device), _dev(case["cs"], device))
    assert got.dtype == F32
    check_close("states", got, case["states"], case["dtype"])


def test_state_passing(case, device):
    from kernels.ema_kernels.ema_state_pass import _ema_state_passing_fwd

    announce(f"state_passing N{case['N']} C{case['cs'].shape[1]} T{case['T']}")
    cs = _dev(case["cs"], device)
    out, final = _ema_state_passing_fwd(_dev(case["states"], device), cs[..., -1], out_dtype=F32)
    check_close("prev", out, case["prev"], F32)
    check_close("final", final, case["final"], F32)


def test_chunk_scan(case, device):
    from kernels.ema_kernels.ema_scan_fwd import _ema_scan_fwd

    announce(f"chunk_scan {case['N']}x{case['L']}x{case['T']} Q{case['Q']} {case['dtype']}")
    got = _ema_scan_fwd(_dev(case["X"], device), _dev(case["cs"], device), _dev(case["prev"], device))
    assert got.dtype == case["dtype"]
    ref = O.chunk_scan(case["X"].float(), case["cs"], case["prev"])
    check_close("y", got, ref, case["dtype"])


def test_bwd_dstates(case, device):
    from kernels.ema_kernels_bwd.ema_scan_bwd import _ema_chunk_scan_bwd_dstates

    announce(f"bwd_dstates {case['N']}x{case['L']}x{case['T']} Q{case['Q']} {case['dtype']}")
    got = _ema_chunk_scan_bwd_dstates(_dev(case["cs"], device), _dev(case["dy"], device))
    check_close("ds", got, case["ds"], case["dtype"])


def test_state_passing_bwd(case, device):
    from kernels.ema_kernels_bwd.ema_state_passing_bwd_dstates import _ema_state_passing_bwd

    announce(f"state_passing_bwd N{case['N']} C{case['cs'].shape[1]} T{case['T']}")
    cs = _dev(case["cs"], device)
    g, ddA_chunk, none = _ema_state_passing_bwd(
        _dev(case["prev"], device), cs[..., -1], _dev(case["ds"], device), chunk_size=case["Q"]
    )
    assert none is None
    check_close("g", g, case["g"], F32)
    check_close("ddA_chunk", ddA_chunk, case["ddA_chunk"], F32)


def test_bwd_dx(case, device):
    from kernels.ema_kernels_bwd.ema_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx

    announce(f"bwd_dx {case['N']}x{case['L']}x{case['T']} Q{case['Q']} {case['dtype']}")
    got = _chunk_scan_chunk_state_bwd_dx(
        _dev(case["X"], device), _dev(case["cs"], device), _dev(case["dy"], device), _dev(case["g"], device)
    )
    assert got.dtype == case["dtype"]
    ref = O.bwd_dx(case["cs"], case["dy"].float(), case["g"])
    check_close("dx", got, ref, case["dtype"])


def _valid(t, L):
    """Keeps only the slots of a (N, C, Q) tensor that lie inside the sequence."""
    N = t.shape[0]
    return t.reshape(N, -1)[:, :L]


def test_bwd_db(case, device):
    from kernels.ema_kernels_bwd.ema_chunk_state_bwd_db import _ema_chunk_state_bwd_db

    announce(f"bwd_db {case['N']}x{case['L']}x{case['T']} Q{case['Q']} {case['dtype']}")
    args = (_dev(case["X"], device), _dev(case["cs"], device), _dev(case["g"], device))
    got = _ema_chunk_state_bwd_db(*args)
    ref = O.bwd_db(case["X"].float(), case["cs"], case["g"])
    check_close("ddA_next", _valid(got, case["L"]), _valid(ref, case["L"]), case["dtype"])
    raw = _ema_chunk_state_bwd_db(*args, raw_scale_gradient=True)
    ref_raw = O.bwd_db(case["X"].float(), case["cs"], case["g"], raw=True)
    check_close("ddA_next raw", _valid(raw, case["L"]), _valid(ref_raw, case["L"]), case["dtype"])


def test_bwd_dc(case, device):
    from kernels.ema_kernels_bwd.ema_chunk_scan_bwd_dc import _ema_chunk_scan_bwd_dC

    announce(f"bwd_dc {case['N']}x{case['L']}x{case['T']} Q{case['Q']} {case['dtype']}")
    got = _ema_chunk_scan_bwd_dC(_dev(case["prev"], device), _dev(case["cs"], device), _dev(case["dy"], device))
    ref = O.bwd_dc(case["prev"], case["cs"], case["dy"].float())
    check_close("ddA_prev", got, ref, case["dtype"])


def test_bwd_da_intra(case, device):
    from kernels.ema_kernels_bwd.ema_scan_da import _ema_chunk_scan_bwd_ddAcs_stable

    announce(f"bwd_da_intra {case['N']}x{case['L']}x{case['T']} Q{case['Q']} {case['dtype']}")
    got = _ema_chunk_scan_bwd_ddAcs_stable(
        _dev(case["X"], device), _dev(case["cs"], device), _dev(case["dy"], device)
    )
    ref = O.bwd_da_intra(case["X"].float(), case["cs"], case["dy"].float())
    check_close("ddA_intra", _valid(got, case["L"]), _valid(ref, case["L"]), case["dtype"])
    assert float(got[..., 0].abs().max()) == 0.0


# (N, L, T, Q) for B6 alone: chunks of one to eight 128-row sub-tiles with ragged ends (up to four
# sub-tiles keep their x rows in registers, longer chunks read x twice) and a feature width that is
# no multiple of the column tile
DA_SHAPES = [
    (2, 1000, 320, 200),
    (1, 900, 1024, 300),
    (3, 1100, 264, 384),
    (2, 2048, 512, 512),
    (2, 1500, 136, 500),
    (1, 1300, 72, 640),
    (1, 2100, 264, 1000),
    (2, 2048, 512, 1024),
]


@pytest.mark.parametrize("rising", ["nowhere", "some_chunks", "everywhere"])
@pytest.mark.parametrize("shape", DA_SHAPES, ids=lambda s: "N%d_L%d_T%d_Q%d" % s)
def test_bwd_da_intra_forms(shape, rising, dtype, device):
    """B6 over both of its forms: a cumsum that never rises inside a chunk takes the factored form, a
    chunk in which it rises anywhere the product with the pairwise minimum
    (kernels/ema_kernels_bwd/ema_scan_da.py:92), and one call may hold both kinds."""
    from kernels.ema_kernels_bwd.ema_scan_da import _ema_chunk_scan_bwd_ddAcs_stable

    N, L, T, Q = shape
    announce(f"bwd_da_intra forms {N}x{L}x{T} Q{Q} {dtype} rising {rising}")
    A, X, dy = flat_case(N, L, T, seed=77 + L + Q, dtype=dtype)
    if rising == "everywhere":
        A = A.abs() * 0.05 - 0.02  # both signs in every chunk
    elif rising == "some_chunks":
        A = A.clone()
        C = -(-L // Q)
        for n in range(N):
            for c in range(n % 2, C, 3):  # every third chunk, one or two positive steps in it
                A[n, min(L - 1, c * Q + 1 + (37 * c) % (Q - 1))] = 0.3
                A[n, min(L - 1, c * Q + Q // 2)] = 0.01
    cs = O.chunk_cumsum(A, Q)
    got = _ema_chunk_scan_bwd_ddAcs_stable(_dev(X, device), _dev(cs, device), _dev(dy, device))
    ref = O.bwd_da_intra(X.float(), cs, dy.float())
    check_close("ddA_intra", _valid(got, L), _valid(ref, L), dtype)
    assert float(got[..., 0].abs().max()) == 0.0


@pytest.mark.parametrize("Q", [128, 256, 512, 640, 1024])
def test_bwd_da_intra_headed_layout(Q, dtype, device):
    """B6 on (b, L, nh, d) tensors consumed in place: the rows of a head are nh * d elements apart."""
    from kernels.ema_kernels_bwd.ema_scan_da import _ema_chunk_scan_bwd_ddAcs_stable

    announce(f"bwd_da_intra headed b2 L1100 nh3 d72 Q{Q} {dtype}")
    x, A, dy = O.make_inputs(2, 3, 1100, 72, seed=31 + Q, dtype=dtype)
    xf, Af = O.to_flat(x.float(), A)
    dyf, _ = O.to_flat(dy.float(), A)
    cs = O.chunk_cumsum(Af, Q)
    got = _ema_chunk_scan_bwd_ddAcs_stable(x.to(device), cs.to(device), dy.to(device))
    ref = O.bwd_da_intra(xf, cs, dyf)
    check_close("ddA_intra", _valid(got, 1100), _valid(ref, 1100), dtype)


@pytest.mark.parametrize("Q", [128, 256, 512, 1024])
def test_bwd_da_intra_bench_shape(Q, device):
    """B6 at the benchmark's size (b16 nh2 d1024 L4096, bfloat16): the factored form against the oracle's
    product form, which is evaluated here with torch on the device (268 MB of Q x Q blocks at Q = 512)."""
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd
    from kernels.ema_kernels_bwd.ema_scan_da import _ema_chunk_scan_bwd_ddAcs_stable

    announce(f"bwd_da_intra b16 nh2 d1024 L4096 Q{Q} bf16")
    gen = torch.Generator(device=device).manual_seed(400 + Q)
    N, L, T = 32, 4096, 1024
    X = torch.randn(N, L, T, generator=gen, device=device).to(BF16)
    dy = torch.randn(N, L, T, generator=gen, device=device).to(BF16)
    A = torch.nn.functional.logsigmoid(torch.randn(N, L, generator=gen, device=device) + 2.0)
    cs = ema_chunk_cumsum_fwd(A, Q)
    got = _ema_chunk_scan_bwd_ddAcs_stable(X, cs, dy)
    ref = torch.cat([O.bwd_da_intra(X[n0:n0 + 8].float(), cs[n0:n0 + 8], dy[n0:n0 + 8].float()) for n0 in range(0, N, 8)])
    check_close("ddA_intra", got, ref, BF16)
    # linearity in dy, which no chunking or tiling may break
    got2 = _ema_chunk_scan_bwd_ddAcs_stable(X, cs, (2 * dy.float()).to(BF16))
    check_close("ddA_intra(2 dy)", got2, 2 * got, F32)


def test_headed_layout_stages(device):
    """(b, L, nh, d) tensors and a (b, L, nh) log-decay are consumed in place (strided)."""
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd
    from kernels.ema_kernels.ema_scan_fwd import _ema_scan_fwd
    from kernels.ema_kernels.ema_state_fwd import _ema_chunk_state_fwd

    announce("headed stages b2 L300 nh3 d64 Q128")
    x, A, _ = O.make_inputs(2, 3, 300, 64, seed=9, dtype=BF16)
    xf, Af = O.to_flat(x.float(), A)
    cs_ref = O.chunk_cumsum(Af, 128)
    st_ref = O.chunk_state(xf, cs_ref)
    prev_ref, _ = O.state_passing(st_ref, cs_ref[..., -1])
    cs = ema_chunk_cumsum_fwd(A.to(device), 128)
    check_close("cs", cs, cs_ref, F32)
    st = _ema_chunk_state_fwd(x.to(device), cs)
    check_close("states", st, st_ref, BF16)
    y = _ema_scan_fwd(x.to(device), cs, prev_ref.to(device))
    assert y.shape == x.shape
    check_close("y", y, O.from_flat(O.chunk_scan(xf, cs_ref, prev_ref), 2, 3), BF16)
