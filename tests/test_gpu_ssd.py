"""GPU parity of the Mamba-2 SSD forward stages (through the C ABI) against the CPU oracle:
each stage against its restatement on the same inputs, the five stages together against the
sequential state-space recurrence, and benchmark configuration 5 at full size through one
sequence checked against the recurrence plus chunk-size invariance for the rest."""
import pytest
import torch

from oracle import ssd_oracle as S
from parity_util import announce, check_close

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16


def _dev(device, *ts):
    return [None if t is None else t.to(device) for t in ts]


CASES = [
    # b, L, nh, P, g, N, Q
    (2, 300, 4, 64, 1, 64, 64),
    (1, 256, 2, 64, 2, 128, 128),
    (2, 200, 4, 64, 1, 128, 256),   # one ragged chunk
    (1, 520, 2, 128, 1, 64, 128),
    (1, 130, 2, 128, 2, 128, 64),
    (1, 900, 2, 64, 1, 64, 512),    # two 256-row super-tiles per chunk, the last chunk ragged
    (1, 512, 2, 128, 2, 128, 256),
    (1, 300, 3, 64, 1, 128, 256),   # an odd number of heads per group: one head per workgroup
    (1, 512, 6, 64, 2, 64, 256),
    (1, 150, 2, 64, 1, 64, 48),     # chunk sizes that are no multiple of the 64-row tiles
    (1, 333, 2, 64, 2, 64, 200),
    (1, 1100, 2, 64, 1, 128, 1024),  # the largest chunk size, second chunk ragged
    # head and state sizes the kernels do not take natively (split into sub-heads / zero-padded
    # around them); the reference's EMA tests and benchmarks call its Mamba launchers with
    # dstate = 1 and head sizes 8, 32 and 512
    (1, 200, 2, 32, 1, 1, 64),
    (1, 300, 2, 512, 1, 1, 128),
    (2, 150, 4, 8, 2, 16, 64),
    (1, 260, 2, 200, 1, 100, 256),
    (1, 100, 2, 6, 1, 1, 32),
]


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_stages_vs_oracle(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd
    from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd
    from kernels.mamba_kernels.mamba_scan_fwd import _chunk_scan_fwd
    from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd
    from kernels.mamba_kernels.mamba_state_pass import _state_passing_fwd

    announce(f"ssd stages b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt_raw, A, B, C, D, z = S.make_inputs(b, L, nh, P, g, N, seed=L + N + Q, dtype=dtype, with_z=True)
    gen = torch.Generator().manual_seed(3)
    bias = torch.randn(nh, generator=gen) * 0.1
    init = torch.randn(b, nh, P * N, generator=gen)
    xd, dtd, Ad, Bd, Cd, Dd, zd, biasd, initd = _dev(device, x, dt_raw, A, B, C, D, z, bias, init)
    small = F32 if dtype == F32 else BF16

    # stage 1 (dt given before softplus so that the option is exercised)
    pre = torch.log(torch.expm1(dt_raw)) - bias
    dA_ref, dt_ref = S.chunk_cumsum(pre, A, Q, bias, True, (1e-3, 0.5))
    dA_cs, dt_out = _chunk_cumsum_fwd(pre.to(device), Ad, Q, dt_bias=biasd, dt_softplus=True, dt_limit=(1e-3, 0.5))
    check_close("dt_out", dt_out, dt_ref, F32)
    check_close("dA_cumsum", dA_cs, dA_ref, F32)

    # the later stages take the oracle's intermediates, so each is checked on its own
    dA_d, dt_d = dA_ref.to(device), dt_ref.to(device)
    rt = None if dtype == F32 else dtype  # the roundings the reference applies before its dots
    st_ref = S.chunk_state(B, x, dt_ref, dA_ref, round_to=rt)
    st = _chunk_state_fwd(Bd, xd, dt_d, dA_d)
    check_close("states", st, st_ref, small)

    prev_ref, fin_ref = S.state_passing(st_ref.reshape(b, -1, nh, P * N), dA_ref[..., -1], init)
    prev, fin = _state_passing_fwd(st_ref.reshape(b, -1, nh, P * N).to(device), dA_d[..., -1], initial_states=initd)
    check_close("prev states", prev, prev_ref, F32)
    check_close("final states", fin, fin_ref, F32)

    if dtype == BF16:  # the carried states stored in the inputs' type, as the combined forward asks
        prev16, fin16 = _state_passing_fwd(st_ref.reshape(b, -1, nh, P * N).to(device), dA_d[..., -1],
                                           initial_states=initd, out_dtype=BF16)
        assert prev16.dtype == BF16 and torch.equal(prev16, prev.to(BF16)) and torch.equal(fin16, fin)

    cb_ref = S.bmm_chunk(C, B, Q)
    cb = _bmm_chunk_fwd(Cd, Bd, Q, output_dtype=torch.float32)
    check_close("CB", cb, cb_ref, small)
    if dtype == BF16:
        check_close("CB (bf16 out)", _bmm_chunk_fwd(Cd, Bd, Q), cb_ref, BF16)

    prev5 = prev_ref.reshape(b, -1, nh, P, N)
    out_ref, outx_ref = S.chunk_scan(cb_ref, x, dt_ref, dA_ref, C, prev5, D, z, round_to=rt)
    out, out_x = _chunk_scan_fwd(cb_ref.to(device), xd, dt_d, dA_d, Cd, prev5.to(device), D=Dd, z=zd)
    check_close("out_x", out_x, outx_ref, dtype)
    check_close("out", out, out_ref, dtype)
    if dtype == BF16:  # the product rounds the carried states to bfloat16 either way
        out16, _ = _chunk_scan_fwd(cb_ref.to(device), xd, dt_d, dA_d, Cd, prev5.to(device).to(BF16), D=Dd, z=zd)
        assert torch.equal(out16, out)
    D2 = torch.randn(nh, P, generator=gen)
    out_ref2, _ = S.chunk_scan(cb_ref, x, dt_ref, dA_ref, C, prev5, D2, None, round_to=rt)
    out2, none = _chunk_scan_fwd(cb_ref.to(device), xd, dt_d, dA_d, Cd, prev5.to(device), D=D2.to(device))
    assert none is None
    check_close("out (D per feature, no gate)", out2, out_ref2, dtype)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", CASES)
def test_combined_vs_recurrence(b, L, nh, P, g, N, Q, dtype, device):
    from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

    announce(f"ssd combined b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, A, B, C, D, z = S.make_inputs(b, L, nh, P, g, N, seed=7 + L + Q, dtype=dtype, with_z=True)
    init = torch.randn(b, nh, P, N, generator=torch.Generator().manual_seed(4))
    y_ref, fin_ref = S.ssd_loop(x.float(), dt, A, B.float(), C.float(), D, z.float(), init)
    xd, dtd, Ad, Bd, Cd, Dd, zd, initd = _dev(device, x, dt, A, B, C, D, z, init)
    y, fin = mamba_chunk_scan_combined_fwd(xd, dtd, Ad, Bd, Cd, Q, D=Dd, z=zd, initial_states=initd,
                                           return_final_states=True)
    torch.cuda.synchronize()
    # The kernels round the weighted B, the weighted CB and the carried states to bf16 before the
    # products, as the reference does; the recurrence rounds nothing, so it gets the loose bar and
    # the chunked oracle that makes the same roundings gets the tight one.
    if dtype == BF16:
        y_rnd, fin_rnd = S.combined_fwd(x, dt, A, B, C, Q, D=D, z=z, initial_states=init, round_to=BF16)
        check_close("y vs chunked oracle with the reference's roundings", y, y_rnd, BF16)
        check_close("final states, same", fin, fin_rnd, BF16)
    check_close("y", y, y_ref, dtype, loose=True)
    check_close("final states", fin, fin_ref, F32 if dtype == F32 else BF16, loose=True)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
def test_views_of_a_fused_projection(dtype, device):
    """x, B, C and z as a Mamba-2 layer holds them: slices of one projected tensor, so the position
    stride exceeds nheads * hdim while the heads stay dense (the chunk scan then pairs heads), and
    x with every other head of a wider tensor (head stride 2 * hdim: one head per workgroup).
    Strides only change addresses, so the results must equal those of contiguous copies."""
    from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

    b, L, nh, P, g, N, Q = 2, 520, 4, 64, 1, 128, 256
    announce(f"ssd strided views b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype}")
    x, dt, A, B, C, D, z = S.make_inputs(b, L, nh, P, g, N, seed=99, dtype=dtype, with_z=True)
    xd, dtd, Ad, Bd, Cd, Dd, zd = _dev(device, x, dt, A, B, C, D, z)
    y0, fin0 = mamba_chunk_scan_combined_fwd(xd, dtd, Ad, Bd, Cd, Q, D=Dd, z=zd, return_final_states=True)

    d_in = nh * P
    zxbc = torch.zeros(b, L, 2 * d_in + 2 * g * N + 8, device=device, dtype=dtype)
    zxbc[..., :d_in] = zd.reshape(b, L, d_in)
    zxbc[..., d_in:2 * d_in] = xd.reshape(b, L, d_in)
    zxbc[..., 2 * d_in:2 * d_in + g * N] = Bd.reshape(b, L, g * N)
    zxbc[..., 2 * d_in + g * N:2 * d_in + 2 * g * N] = Cd.reshape(b, L, g * N)
    zv = zxbc[..., :d_in].unflatten(-1, (nh, P))
    xv = zxbc[..., d_in:2 * d_in].unflatten(-1, (nh, P))
    Bv = zxbc[..., 2 * d_in:2 * d_in + g * N].unflatten(-1, (g, N))
    Cv = zxbc[..., 2 * d_in + g * N:2 * d_in + 2 * g * N].unflatten(-1, (g, N))
    assert not xv.is_contiguous() and xv.stride(2) == P
    y1, fin1 = mamba_chunk_scan_combined_fwd(xv, dtd, Ad, Bv, Cv, Q, D=Dd, z=zv, return_final_states=True)
    assert torch.equal(y1, y0) and torch.equal(fin1, fin0)

    wide = torch.zeros(b, L, 2 * nh, P, device=device, dtype=dtype)
    wide[:, :, ::2] = xd
    xs = wide[:, :, ::2]
    assert xs.stride(2) == 2 * P
    y2, fin2 = mamba_chunk_scan_combined_fwd(xs, dtd, Ad, Bd, Cd, Q, D=Dd, z=zd, return_final_states=True)
    assert torch.equal(y2, y0) and torch.equal(fin2, fin0)


def test_converted_operands_stay_alive_until_the_launch(device):
    """CB in bfloat16 together with dt and dA_cumsum as strided views: every operand the chunk scan
    has to convert is converted into a temporary, and all of them must still be there when the
    kernel is enqueued.  The result must equal that of float32, contiguous operands."""
    from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd
    from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd
    from kernels.mamba_kernels.mamba_scan_fwd import _chunk_scan_fwd
    from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd
    from kernels.mamba_kernels.mamba_state_pass import _state_passing_fwd

    b, L, nh, P, g, N, Q = 2, 512, 4, 64, 1, 128, 256
    announce(f"ssd chunk scan with converted operands b{b} L{L} nh{nh} P{P} N{N} Q{Q}")
    x, dt, A, B, C, D, _ = S.make_inputs(b, L, nh, P, g, N, seed=21, dtype=BF16)
    xd, dtd, Ad, Bd, Cd = _dev(device, x, dt, A, B, C)
    dA_cs, dt_out = _chunk_cumsum_fwd(dtd, Ad, Q)
    states = _chunk_state_fwd(Bd, xd, dt_out, dA_cs)
    nchunks = L // Q
    prev, _ = _state_passing_fwd(states.view(b, nchunks, nh, P * N), dA_cs[..., -1], out_dtype=BF16)
    prev = prev.view(b, nchunks, nh, P, N)
    cb32 = _bmm_chunk_fwd(Cd, Bd, Q, output_dtype=F32)
    ref, _ = _chunk_scan_fwd(cb32, xd, dt_out, dA_cs, Cd, prev)
    # the same values in the shapes that need converting
    cb16 = cb32.to(BF16)
    ref16, _ = _chunk_scan_fwd(cb16.float(), xd, dt_out, dA_cs, Cd, prev)
    wide_dt = torch.zeros(b, nh, nchunks, 2 * Q, device=device)
    wide_dA = torch.zeros(b, nh, nchunks, 2 * Q, device=device)
    wide_dt[..., ::2] = dt_out
    wide_dA[..., ::2] = dA_cs
    dt_view, dA_view = wide_dt[..., ::2], wide_dA[..., ::2]
    assert not dt_view.is_contiguous() and not dA_view.is_contiguous()
    for rep in range(3):  # the allocator reuses the blocks of earlier temporaries
        got, _ = _chunk_scan_fwd(cb16, xd, dt_view, dA_view, Cd, prev)
        assert torch.equal(got, ref16), rep
    check_close("y with bf16 CB", got, ref, BF16, loose=True)


def test_chunk_states_into_a_given_buffer(device):
    """A preallocated float32 result is written in place (no second tensor, no copy)."""
    from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd
    from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd

    b, L, nh, P, g, N, Q = 1, 512, 2, 64, 1, 128, 256
    x, dt, A, B, C, D, _ = S.make_inputs(b, L, nh, P, g, N, seed=22, dtype=BF16)
    xd, dtd, Ad, Bd = _dev(device, x, dt, A, B)
    dA_cs, dt_out = _chunk_cumsum_fwd(dtd, Ad, Q)
    ref = _chunk_state_fwd(Bd, xd, dt_out, dA_cs)
    buf = torch.full_like(ref, float("nan"))
    ptr = buf.data_ptr()
    before = torch.cuda.memory_allocated(device)
    out = _chunk_state_fwd(Bd, xd, dt_out, dA_cs, states=buf)
    assert out is buf and buf.data_ptr() == ptr and torch.equal(buf, ref)
    assert torch.cuda.memory_allocated(device) - before < ref.numel() * 4, "no second result tensor"
    half = torch.empty(ref.shape, device=device, dtype=BF16)  # another dtype still goes through a copy
    assert torch.equal(_chunk_state_fwd(Bd, xd, dt_out, dA_cs, states=half), ref.to(BF16))


WALK_CASES = [
    # b, L, nh, P, g, N, Q
    (2, 300, 4, 64, 1, 64, 64),     # last chunk ragged, last stage ragged
    (1, 256, 2, 64, 2, 128, 128),
    (2, 200, 4, 64, 1, 128, 256),   # a single ragged chunk
    (1, 520, 2, 128, 1, 64, 128),
    (1, 130, 2, 128, 2, 128, 64),
    (1, 900, 3, 64, 1, 64, 512),
    (1, 1100, 2, 64, 1, 128, 1024),
    (3, 64, 2, 64, 1, 128, 64),     # one stage in all
    (1, 50, 2, 64, 1, 64, 64),      # less than one stage
    (1, 8256, 1, 64, 1, 128, 256),  # 129 stages: rounds of the ring and a remainder
    (1, 640, 2, 64, 1, 128, 64),    # every stage begins a chunk (the state stores of two chunks in the queue at a time)
    (2, 1000, 2, 64, 2, 128, 128),  # two stages per chunk, last chunk and last stage ragged
]


@pytest.mark.parametrize("dtype,out_dtype", [(F32, F32), (BF16, F32), (BF16, BF16)],
                         ids=["f32-out_f32", "bf16-out_f32", "bf16-out_bf16"])  # float32 inputs carry float32 states
@pytest.mark.parametrize("b,L,nh,P,g,N,Q", WALK_CASES)
def test_chunk_state_passing_in_one_kernel(b, L, nh, P, g, N, Q, dtype, out_dtype, device):
    """The kernel that keeps the chunk-local states on chip against the two launchers it replaces:
    the same bits, with and without an initial state, and the oracle's restatements on top."""
    from kernels.mamba_kernels.mamba_combined_fwd import _chunk_state_passing_fwd
    from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd
    from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd
    from kernels.mamba_kernels.mamba_state_pass import _state_passing_fwd

    announce(f"ssd state walk b{b} L{L} nh{nh} P{P} g{g} N{N} Q{Q} {dtype} -> {out_dtype}")
    x, dt, A, B, _, _, _ = S.make_inputs(b, L, nh, P, g, N, seed=L + N + Q, dtype=dtype)
    init = torch.randn(b, nh, P, N, generator=torch.Generator().manual_seed(9))
    xd, dtd, Ad, Bd, initd = _dev(device, x, dt, A, B, init)
    dA_cs, dt_out = _chunk_cumsum_fwd(dtd, Ad, Q)
    C = dA_cs.shape[2]
    for ini in (None, initd):
        local = _chunk_state_fwd(Bd, xd, dt_out, dA_cs)
        ref, ref_fin = _state_passing_fwd(local.view(b, C, nh, P * N), dA_cs[..., -1],
                                          initial_states=None if ini is None else ini.view(b, nh, P * N),
                                          out_dtype=out_dtype)
        got, fin = _chunk_state_passing_fwd(Bd, xd, dt_out, dA_cs, initial_states=ini, out_dtype=out_dtype)
        torch.cuda.synchronize()
        assert got.dtype == out_dtype and got.shape == (b, C, nh, P, N) and fin.shape == (b, nh, P, N)
        assert torch.equal(got.view(b, C, nh, P * N), ref), "states entering the chunks differ from the two launchers"
        assert torch.equal(fin.view(b, nh, P * N), ref_fin), "final states differ from the two launchers"
    # against the oracle (no initial state)
    dA_ref, dt_ref = S.chunk_cumsum(dt, A, Q)
    st_ref = S.chunk_state(B, x, dt_ref, dA_ref, round_to=None if dtype == F32 else BF16)
    prev_ref, fin_ref = S.state_passing(st_ref.reshape(b, C, nh, P * N), dA_ref[..., -1])
    got, fin = _chunk_state_passing_fwd(Bd, xd, dt_out, dA_cs, out_dtype=F32)
    check_close("states entering the chunks", got, prev_ref.view(b, C, nh, P, N), dtype)
    check_close("final states", fin, fin_ref.view(b, nh, P, N), dtype)


def test_chunk_state_passing_views_and_limits(device):
    """x and B as slices of a wider projection give the bits of contiguous copies; chunk sizes the
    kernel does not take are left to the two launchers (None)."""
    from kernels.mamba_kernels.mamba_combined_fwd import _chunk_state_passing_fwd
    from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd

    b, L, nh, P, g, N, Q = 2, 384, 4, 64, 1, 128, 128
    x, dt, A, B, _, _, _ = S.make_inputs(b, L, nh, P, g, N, seed=31, dtype=BF16)
    xd, dtd, Ad, Bd = _dev(device, x, dt, A, B)
    wide = torch.randn(b, L, nh * P + g * N + 24, device=device).to(BF16)
    xv = wide[..., : nh * P].view(b, L, nh, P)
    Bv = wide[..., nh * P : nh * P + g * N].view(b, L, g, N)
    xv.copy_(xd)
    Bv.copy_(Bd)
    dA_cs, dt_out = _chunk_cumsum_fwd(dtd, Ad, Q)
    a = _chunk_state_passing_fwd(Bd, xd, dt_out, dA_cs, out_dtype=BF16)
    v = _chunk_state_passing_fwd(Bv, xv, dt_out, dA_cs, out_dtype=BF16)
    assert torch.equal(a[0], v[0]) and torch.equal(a[1], v[1])
    dA48, dt48 = _chunk_cumsum_fwd(dtd, Ad, 48)
    assert _chunk_state_passing_fwd(Bd, xd, dt48, dA48) is None




def test_unsupported_shapes_are_refused(device):
    from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd

    x = torch.zeros(1, 64, 2, 64, device=device)
    B = torch.zeros(1, 64, 1, 64, device=device)
    dt = torch.zeros(1, 2, 1, 64, device=device)
    with pytest.raises(NotImplementedError):  # a state larger than 128
        _chunk_state_fwd(torch.zeros(1, 64, 1, 256, device=device), x, dt, dt)
    with pytest.raises(NotImplementedError):  # a chunk size that is no multiple of 4
        _chunk_state_fwd(B[:, :62], x[:, :62], dt[..., :62], dt[..., :62])
    with pytest.raises(AssertionError):  # ids must be (batch, seqlen)
        _chunk_state_fwd(B, torch.zeros(1, 64, 2, 64, device=device), dt, dt, seq_idx=torch.zeros(1, 32, device=device))


def test_config5_full_size(device):
    """b8 nh32 hdim64 dstate128 g1 L8192 Q256 bf16, D = 0: every batch element against the chunked
    oracle that makes the reference's roundings (at the bar for computations that round the same
    operands at different points of a sum), batch element 0 also against the sequential
    recurrence, and the whole against the same computation at chunk size 128."""
    from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

    announce("ssd config 5 full size")
    b, L, nh, P, g, N = 8, 8192, 32, 64, 1, 128
    x, dt, A, B, C, _, _ = S.make_inputs(b, L, nh, P, g, N, seed=5, dtype=BF16)
    xd, dtd, Ad, Bd, Cd = _dev(device, x, dt, A, B, C)
    y256, fin256 = mamba_chunk_scan_combined_fwd(xd, dtd, Ad, Bd, Cd, 256, return_final_states=True)
    y128, fin128 = mamba_chunk_scan_combined_fwd(xd, dtd, Ad, Bd, Cd, 128, return_final_states=True)
    torch.cuda.synchronize()
    check_close("chunk 256 vs chunk 128", y256, y128.float(), BF16, loose=True)
    check_close("final states 256 vs 128", fin256, fin128, BF16, loose=True)
    for i in range(0, b, 2):
        y_rnd, fin_rnd = S.combined_fwd(x[i:i + 2], dt[i:i + 2], A, B[i:i + 2], C[i:i + 2], 256, round_to=BF16)
        check_close(f"y[{i}:{i + 2}] vs chunked oracle with the reference's roundings", y256[i:i + 2], y_rnd, BF16,
                    regrouped=True)
        check_close(f"final[{i}:{i + 2}], same", fin256[i:i + 2], fin_rnd, BF16)
    y_ref, fin_ref = S.ssd_loop(x[:1].float(), dt[:1], A, B[:1].float(), C[:1].float())
    check_close("y[0] vs recurrence", y256[:1], y_ref, BF16, loose=True)
    check_close("final[0] vs recurrence", fin256[:1], fin_ref, BF16, loose=True)
