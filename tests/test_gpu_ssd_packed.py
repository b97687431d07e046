"""GPU parity of the Mamba-2 SSD stages on packed batches (seq_idx), through the C ABI: every
forward and backward launcher against the CPU oracle with the same ids, and the five forward
stages together against running each sequence of the pack on its own."""
import pytest
import torch

from oracle import ssd_oracle as S
from parity_util import announce, check_close

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16


def pack_ids(b, L, Q, seed):
    """(b, L) int32 ids, counting up from 0 in each row: boundaries at random places, in the middle
    of the first chunk and, when the row is long enough, on a chunk edge, next to it and in the
    middle of the second chunk; row b-1 is left as a single sequence."""
    gen = torch.Generator().manual_seed(seed)
    rows = []
    for r in range(b):
        cuts = set()
        if r < b - 1 or b == 1:
            n = int(torch.randint(2, 6, (1,), generator=gen))
            cuts = {int(v) for v in torch.randint(1, L, (n,), generator=gen)}
            cuts.add(min(L, Q) // 2)  # the middle of the first chunk
            if L > Q:
                cuts |= {Q, min(L - 1, Q + 1), min(L - 1, Q + Q // 2)}
        ids = torch.zeros(L, dtype=torch.int32)
        for c in sorted(cuts):
            ids[c:] += 1
        rows.append(ids)
    return torch.stack(rows)


def slow(A):
    """Decay rates twenty times smaller than the configuration's, so that the state remembers
    hundreds of positions and a wrong mask changes results everywhere, not just next to a
    boundary."""
    return A * 0.05


CASES = [
    # b, L, nh, P, g, N, Q
    (2, 300, 4, 64, 1, 64, 64),
    (2, 200, 4, 64, 2, 128, 256),   # one ragged chunk
    (1, 520, 2, 128, 1, 64, 128),
    (1, 900, 2, 64, 1, 128, 512),   # two 256-row super-tiles per chunk, the last chunk ragged
    (2, 768, 2, 128, 2, 128, 256),
]


def _dev(device, *ts):
    return [None if t is None else t.to(device) for t in ts]


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_packed_forward_stages_vs_oracle(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd
    from kernels.mamba_kernels.mamba_scan_fwd import _chunk_scan_fwd
    from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd
    from kernels.mamba_kernels.mamba_state_pass import _state_passing_fwd

    announce(f"ssd packed fwd stages b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt_raw, A, B, C, D, z = S.make_inputs(b, L, nh, P, g, N, seed=L + N + Q, dtype=dtype, with_z=True)
    A = slow(A)
    seq = pack_ids(b, L, Q, seed=L)
    init = torch.randn(b, nh, P * N, generator=torch.Generator().manual_seed(3))
    dA_cs, dt = S.chunk_cumsum(dt_raw, A, Q)
    rt = None if dtype == F32 else dtype
    small = F32 if dtype == F32 else BF16
    xd, Bd, Cd, Dd, zd, dtd, dAd, seqd, initd = _dev(device, x, B, C, D, z, dt, dA_cs, seq, init)

    st_ref = S.chunk_state(B, x, dt, dA_cs, round_to=rt, seq_idx=seq)
    check_close("states", _chunk_state_fwd(Bd, xd, dtd, dAd, seq_idx=seqd), st_ref, small)
    assert (st_ref - S.chunk_state(B, x, dt, dA_cs, round_to=rt)).abs().max() > 0.1  # the ids matter

    flat = st_ref.reshape(b, -1, nh, P * N)
    prev_ref, fin_ref = S.state_passing(flat, dA_cs[..., -1], init, seq_idx=seq, chunk_size=Q)
    prev, fin = _state_passing_fwd(flat.to(device), dAd[..., -1], initial_states=initd, seq_idx=seqd, chunk_size=Q)
    check_close("prev states", prev, prev_ref, F32)
    check_close("final states", fin, fin_ref, F32)

    cb_ref = S.bmm_chunk(C, B, Q, seq_idx=seq)
    check_close("CB", _bmm_chunk_fwd(Cd, Bd, Q, seq_idx=seqd, output_dtype=torch.float32), cb_ref, small)
    # ids given as int64 and as a strided view are converted / addressed by strides
    wide = torch.zeros(b, L, 2, dtype=torch.int64, device=device)
    wide[..., 1] = seqd
    check_close("CB (int64 strided ids)", _bmm_chunk_fwd(Cd, Bd, Q, seq_idx=wide[..., 1], output_dtype=torch.float32),
                cb_ref, small)

    prev5 = prev_ref.reshape(b, -1, nh, P, N)
    out_ref, outx_ref = S.chunk_scan(cb_ref, x, dt, dA_cs, C, prev5, D, z, round_to=rt, seq_idx=seq)
    out, out_x = _chunk_scan_fwd(cb_ref.to(device), xd, dtd, dAd, Cd, prev5.to(device), D=Dd, z=zd, seq_idx=seqd)
    check_close("out_x", out_x, outx_ref, dtype)
    check_close("out", out, out_ref, dtype)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_packed_combined_equals_each_sequence_alone(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

    announce(f"ssd packed combined b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, A, B, C, D, z = S.make_inputs(b, L, nh, P, g, N, seed=11 + L + Q, dtype=dtype, with_z=True)
    A = slow(A)
    seq = pack_ids(b, L, Q, seed=L + 1)
    init = torch.randn(b, nh, P, N, generator=torch.Generator().manual_seed(4))
    xd, dtd, Ad, Bd, Cd, Dd, zd, seqd, initd = _dev(device, x, dt, A, B, C, D, z, seq, init)
    y, fin = mamba_chunk_scan_combined_fwd(xd, dtd, Ad, Bd, Cd, Q, D=Dd, z=zd, initial_states=initd, seq_idx=seqd,
                                           return_final_states=True)
    torch.cuda.synchronize()
    y_ref, fin_ref = S.ssd_loop(x.float(), dt, A, B.float(), C.float(), D, z.float(), init, seq_idx=seq)
    if dtype == BF16:
        y_rnd, fin_rnd = S.combined_fwd(x, dt, A, B, C, Q, D=D, z=z, initial_states=init, round_to=BF16, seq_idx=seq)
        # with the slow decay the sums reach ~100 and hide cancellations; a carried state that
        # rounds to the neighbouring bf16 value moves an output by a bf16 step of the terms, not
        # of the result, so the absolute term follows the largest magnitude
        check_close("y vs chunked oracle with the reference's roundings", y, y_rnd, BF16, loose=True)
        check_close("final states, same", fin, fin_rnd, BF16, loose=True)
    check_close("y vs recurrence", y, y_ref, dtype, loose=True)
    small = F32 if dtype == F32 else BF16
    check_close("final states vs recurrence", fin, fin_ref, small, loose=True)
    # the same kernels on every sequence by itself (other chunk alignment, no ids)
    for r in range(b):
        bounds = [0] + [t for t in range(1, L) if seq[r, t] != seq[r, t - 1]] + [L]
        for i in range(len(bounds) - 1):
            t0, t1 = bounds[i], bounds[i + 1]
            one = lambda t: t[r:r + 1, t0:t1].contiguous()
            yi, fi = mamba_chunk_scan_combined_fwd(one(xd), one(dtd), Ad, one(Bd), one(Cd), Q, D=Dd, z=one(zd),
                                                   initial_states=initd[r:r + 1] if i == 0 else None,
                                                   return_final_states=True)
            check_close(f"row {r} sequence {i} alone", y[r:r + 1, t0:t1], yi.float().cpu(), dtype, loose=True)
        check_close(f"row {r} final state alone", fin[r:r + 1], fi.cpu(), small, loose=True)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_packed_backward_stages_vs_oracle(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_da import _chunk_scan_bwd_ddAcs_stable
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_dc import _chunk_scan_bwd_dC
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx
    from kernels.mamba_kernels_bwd.mamba_chunk_state_bwd_db import _chunk_state_bwd_db
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates

    announce(f"ssd packed bwd stages b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt_raw, A, B, C, D, _ = S.make_inputs(b, L, nh, P, g, N, seed=2 * L + N + Q, dtype=dtype)
    dA_cs, dt = S.chunk_cumsum(dt_raw, slow(A), Q)
    seq = pack_ids(b, L, Q, seed=L + 2)
    gen = torch.Generator().manual_seed(L + Q)
    dout = torch.randn(b, L, nh, P, generator=gen).to(dtype)
    nc = dt.shape[2]
    prev = torch.randn(b, nc, nh, P, N, generator=gen)
    dstates = torch.randn(b, nc, nh, P, N, generator=gen)
    rt = None if dtype == F32 else dtype
    d = lambda t: t.to(device)
    seqd = d(seq)

    got = _chunk_scan_bwd_dstates(d(C), d(dA_cs), d(dout), seq_idx=seqd, dtype=torch.float32)
    check_close("dprev_states", got, S.bwd_dstates(C, dA_cs, dout, round_to=rt, seq_idx=seq), dtype)

    dB_ref, ddA_ref = S.chunk_state_bwd_db(x, dt, dA_cs, dstates, B=B, ngroups=g, round_to=rt, seq_idx=seq)
    dB, ddA = _chunk_state_bwd_db(d(x), d(dt), d(dA_cs), d(dstates), seq_idx=seqd, B=d(B), ngroups=g)
    check_close("dB", dB, dB_ref, dtype)
    check_close("ddA_cumsum (chunk state)", ddA, ddA_ref, dtype)

    dC_ref, ddAp_ref = S.chunk_scan_bwd_dC(prev, dA_cs, dout, C=C, ngroups=g, round_to=rt, seq_idx=seq)
    dC, ddAp = _chunk_scan_bwd_dC(d(prev), d(dA_cs), d(dout), seq_idx=seqd, C=d(C), ngroups=g)
    check_close("dC", dC, dC_ref, dtype)
    check_close("ddA_cumsum_prev", ddAp, ddAp_ref, dtype)

    cb = S.bmm_chunk(C, B, Q, seq_idx=seq)
    dx_ref, ddt_ref, _ = S.chunk_scan_chunk_state_bwd_dx(x, dt, dA_cs, B, cb, dout, dstates, D=D, round_to=rt,
                                                         seq_idx=seq)
    dx, ddt, _ = _chunk_scan_chunk_state_bwd_dx(d(x), d(dt), d(dA_cs), d(B), d(cb), d(dout), d(dstates), D=d(D),
                                                seq_idx=seqd)
    check_close("dx", dx, dx_ref, dtype)
    check_close("ddt", ddt, ddt_ref, dtype, loose=dtype == BF16)

    # the causal-term gradient only sees the ids through the masked cb
    ref = S.chunk_scan_bwd_ddAcs_stable(x, dt, dA_cs, dout, cb)
    got = _chunk_scan_bwd_ddAcs_stable(d(x), d(dt), d(dA_cs), d(dout), d(cb))
    check_close("ddA_cumsum (causal term)", got, ref, dtype, loose=dtype == BF16)


@pytest.mark.parametrize("has_init", [False, True])
@pytest.mark.parametrize("b,nc,nh,dim,Q,L", [(2, 5, 3, 64 * 64, 64, 300), (1, 33, 2, 64 * 128, 16, 520), (2, 7, 2, 100, 32, 200)])
def test_packed_state_passing_bwd_vs_oracle(b, nc, nh, dim, Q, L, has_init, device):
    from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd

    announce(f"ssd packed state passing bwd b{b} C{nc} nh{nh} dim{dim} init={has_init}")
    assert nc == (L + Q - 1) // Q
    gen = torch.Generator().manual_seed(dim + nc)
    states = torch.randn(b, nc, nh, dim, generator=gen)
    dA = -0.1 * torch.rand(b, nh, nc, generator=gen)
    dout = torch.randn(b, nc, nh, dim, generator=gen)
    dfin = torch.randn(b, nh, dim, generator=gen)
    seq = pack_ids(b, L, Q, seed=L + 3)
    seq[0] += 1  # row 0 does not continue the initial state
    ref = S.state_passing_bwd(states, dA, dout, dfin, has_initial_states=has_init, seq_idx=seq, chunk_size=Q)
    got = _state_passing_bwd(states.to(device), dA.to(device), dout.to(device), dfinal_states=dfin.to(device),
                             seq_idx=seq.to(device), has_initial_states=has_init, chunk_size=Q)
    check_close("dstates", got[0], ref[0], F32)
    check_close("ddA_chunk_cumsum", got[1], ref[1], F32)
    assert torch.equal(got[1][0, :, 0].cpu(), torch.zeros(nh))
    if has_init:
        check_close("dinitstates", got[2], ref[2], F32)
        assert torch.equal(got[2][0].cpu(), dout[0, 0])  # nothing flows back across the dropped state


VARLEN_CASES = [
    # L, nh, P, g, N, Q
    (300, 4, 64, 1, 64, 64),
    (520, 2, 128, 2, 128, 128),
    (200, 2, 64, 1, 128, 256),     # one ragged chunk that holds every sequence
    (333, 2, 48, 1, 20, 64),       # head and state sizes off the tile sizes
    (150, 2, 8, 1, 1, 32),
]


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("L,nh,P,g,N,Q", VARLEN_CASES)
def test_varlen_states(L, nh, P, g, N, Q, dtype, device):
    """The state at the end of each packed sequence (cu_seqlens): the launcher against the oracle on
    the oracle's intermediates, and the combined forward against each sequence run through the
    recurrence on its own."""
    from kernels.ema_chunk_state import chunk_state_varlen
    from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

    announce(f"ssd varlen states L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, A, B, C, _, _ = S.make_inputs(1, L, nh, P, g, N, seed=L + P, dtype=dtype)
    A = slow(A)
    seq = pack_ids(1, L, Q, seed=L)
    starts = (torch.nonzero(seq[0, 1:] != seq[0, :-1])[:, 0] + 1).tolist()
    cu = torch.tensor([0] + starts + [L], dtype=torch.int32)
    init = torch.randn(1, nh, P, N, generator=torch.Generator().manual_seed(6))
    rt = None if dtype == F32 else dtype
    small = F32 if dtype == F32 else BF16

    dA_cs, dt_out = S.chunk_cumsum(dt, A, Q)
    states = S.chunk_state(B, x, dt_out, dA_cs, rt, seq)
    prev, _ = S.state_passing(states.reshape(1, -1, nh, P * N), dA_cs[..., -1], init.reshape(1, nh, P * N), seq, Q)
    prev = prev.reshape(-1, nh, P, N)
    ref = S.chunk_state_varlen(B[0], x[0], dt_out[0], dA_cs[0], cu, prev, rt)
    got = chunk_state_varlen(*_dev(device, B[0], x[0], dt_out[0], dA_cs[0], cu, prev))
    assert got.shape == (len(cu) - 1, nh, P, N)
    check_close("varlen states vs oracle", got, ref, small)

    y, fin, varlen = mamba_chunk_scan_combined_fwd(
        *_dev(device, x, dt, A, B, C), Q, initial_states=init.to(device), seq_idx=seq.to(device),
        cu_seqlens=cu.to(device), return_final_states=True, return_varlen_states=True)
    for i in range(len(cu) - 1):
        sl = slice(int(cu[i]), int(cu[i + 1]))
        # the first sequence continues the initial state only if it reaches past chunk 0
        # (kernels/ema_chunk_state.py:563 of the reference)
        first = init if i == 0 and int(cu[1]) > Q else None
        _, fi = S.ssd_loop(x[:, sl].float(), dt[:, sl], A, B[:, sl].float(), C[:, sl].float(), initial_states=first)
        check_close(f"sequence {i} alone", varlen[i], fi[0], small, loose=dtype == BF16)
    check_close("last sequence = final state", varlen[-1], fin[0].float(), small)


def test_varlen_states_edge_cases(device):
    """A sequence of one position, an empty one, one that is the whole batch, and bounds that do
    not fit (zeros, no fault)."""
    from kernels.ema_chunk_state import chunk_state_varlen

    L, nh, P, g, N, Q = 100, 2, 64, 1, 64, 32
    x, dt, A, B, _, _, _ = S.make_inputs(1, L, nh, P, g, N, seed=1)
    dA_cs, dt_out = S.chunk_cumsum(dt, slow(A), Q)
    prev = torch.randn(4, nh, P, N, generator=torch.Generator().manual_seed(1))
    args = lambda cu: _dev(device, B[0], x[0], dt_out[0], dA_cs[0], cu, prev)
    cu = torch.tensor([0, 1, 1, 64, 100], dtype=torch.int32)
    got = chunk_state_varlen(*args(cu)).cpu()
    ref = S.chunk_state_varlen(B[0], x[0], dt_out[0], dA_cs[0], torch.tensor([0, 1]), prev)
    check_close("one position", got[0], ref[0], F32)
    assert torch.equal(got[1], torch.zeros(nh, P, N))  # empty
    ref = S.chunk_state_varlen(B[0], x[0], dt_out[0], dA_cs[0], torch.tensor([1, 64, 100]), prev)
    check_close("ends on a chunk edge / ragged last chunk", got[2:], ref, F32)
    whole = chunk_state_varlen(*args(torch.tensor([0, L], dtype=torch.int32)))
    check_close("whole batch", whole, S.chunk_state_varlen(B[0], x[0], dt_out[0], dA_cs[0], [0, L], prev), F32)
    odd = chunk_state_varlen(*args(torch.tensor([-5, 10, 5, 400], dtype=torch.int32))).cpu()
    assert torch.equal(odd[0], torch.zeros(nh, P, N)) and torch.equal(odd[1], torch.zeros(nh, P, N))
    ref = S.chunk_state_varlen(B[0], x[0], dt_out[0], dA_cs[0], torch.tensor([5, 100]), prev)
    check_close("end clamped to the length", odd[2], ref[0], F32)
