"""GPU parity of the sequence-level entry points (ema_seq_fwd / ema_seq_bwd through the C ABI)
against the sequential CPU oracle: both forms of the coefficient, boundary states, flat and
headed layouts, ragged lengths, and the bench shape through size-independent properties."""
import pytest
import torch

from oracle import ema_oracle as O
from parity_util import announce, check_close

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16


def _case(N, L, T, seed, dtype, form):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, L, T, generator=g).to(dtype)
    u = torch.randn(N, L, generator=g) + 2.0
    coef = torch.sigmoid(-u) if form == "probability" else torch.nn.functional.logsigmoid(u)
    init = torch.randn(N, T, generator=g)
    dy = torch.randn(N, L, T, generator=g).to(dtype)
    dfinal = torch.randn(N, T, generator=g)
    return X, coef, init, dy, dfinal


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("form", ["log_decay", "probability"])
@pytest.mark.parametrize("states", [False, True], ids=["zero_init", "with_states"])
@pytest.mark.parametrize("N,L,T", [(3, 1000, 264), (2, 128, 8), (2, 129, 512), (1, 1, 16), (4, 2048, 1024)])
def test_seq_fwd_bwd_vs_oracle(N, L, T, states, form, dtype, device):
    from kernels.ema_seq import ema_seq_bwd, ema_seq_fwd

    announce(f"seq N{N} L{L} T{T} {form} states={states} {dtype}")
    X, coef, init, dy, dfinal = _case(N, L, T, 11 + L + T, dtype, form)
    y, fin, prev128 = ema_seq_fwd(coef.to(device), X.to(device), form, init.to(device) if states else None)
    dx, dc, dinit = ema_seq_bwd(dy.to(device), X.to(device), coef.to(device), prev128, form,
                                dfinal_states=dfinal.to(device) if states else None, want_dinit=states)
    torch.cuda.synchronize()
    y_ref, fin_ref = O.ema_seq_loop(X.float(), coef, form, init if states else None)
    dx_ref, dc_ref, dinit_ref = O.ema_seq_loop_bwd(dy.float(), X.float(), coef, form,
                                                   init if states else None, dfinal if states else None)
    small = F32 if dtype == F32 else BF16
    check_close("y", y, y_ref, dtype)
    check_close("final", fin, fin_ref, small)
    check_close("dx", dx, dx_ref, dtype)
    check_close("dcoef", dc, dc_ref, dtype)
    if states:
        check_close("dinit", dinit, dinit_ref, small)
    C = -(-L // 128)
    y0 = init if states else torch.zeros(N, T)
    ref_prev = torch.stack([y_ref[:, c * 128 - 1] if c else y0 for c in range(C)], 1)
    check_close("prev128", prev128, ref_prev, small)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("form", ["log_decay", "probability"])
def test_seq_autograd_headed(form, dtype, device):
    """Headed (b, L, nh, d) tensors through the autograd function, with gradients flowing
    through the final states and into the initial states."""
    from kernels.ema_seq import ema_seq_scan

    b, nh, L, d = 2, 3, 700, 64
    announce(f"seq autograd headed b{b} nh{nh} L{L} d{d} {form} {dtype}")
    g = torch.Generator().manual_seed(5)
    x = torch.randn(b, L, nh, d, generator=g).to(dtype)
    u = torch.randn(b, L, nh, generator=g) + 2.0
    coef = torch.sigmoid(-u) if form == "probability" else torch.nn.functional.logsigmoid(u)
    init = torch.randn(b, nh, d, generator=g)
    dy = torch.randn(b, L, nh, d, generator=g).to(dtype)
    dfin = torch.randn(b, nh, d, generator=g)
    xg, cg, ig = (t.to(device).requires_grad_() for t in (x, coef, init))
    y, fin = ema_seq_scan(cg, xg, form, initial_states=ig, return_final_states=True)
    ((y.float() * dy.to(device).float()).sum() + (fin * dfin.to(device)).sum()).backward()
    torch.cuda.synchronize()
    xf, cf = O.to_flat(x.float(), coef)
    dyf, _ = O.to_flat(dy.float(), coef)
    i2, df2 = init.reshape(b * nh, d), dfin.reshape(b * nh, d)
    y_ref, fin_ref = O.ema_seq_loop(xf, cf, form, i2)
    dx_ref, dc_ref, di_ref = O.ema_seq_loop_bwd(dyf, xf, cf, form, i2, df2)
    small = F32 if dtype == F32 else BF16
    check_close("y", y, O.from_flat(y_ref, b, nh), dtype)
    check_close("final", fin, fin_ref.reshape(b, nh, d), small)
    check_close("dx", xg.grad, O.from_flat(dx_ref, b, nh), dtype)
    check_close("dcoef", cg.grad, dc_ref.reshape(b, nh, L).permute(0, 2, 1), dtype)
    check_close("dinit", ig.grad, di_ref.reshape(b, nh, d), small)


def test_ema_scan_combined_xp_entry(device):
    """The (x, p) entry point of the reference's first implementation (kernels/ema.py:370),
    now one pass and differentiable."""
    from kernels.ema import ema_scan_combined

    B, L, D = 3, 777, 96
    announce(f"ema_scan_combined(x, p) B{B} L{L} D{D}")
    g = torch.Generator().manual_seed(9)
    x = torch.randn(B, L, D, generator=g)
    p = torch.sigmoid(torch.randn(B, L, 1, generator=g) - 2.0)
    dy = torch.randn(B, L, D, generator=g)
    xg, pg = x.to(device).requires_grad_(), p.to(device).requires_grad_()
    z = ema_scan_combined(xg, pg)
    z.backward(dy.to(device))
    torch.cuda.synchronize()
    z_ref, _ = O.ema_seq_loop(x, p.squeeze(-1), "probability")
    dx_ref, dp_ref, _ = O.ema_seq_loop_bwd(dy, x, p.squeeze(-1), "probability")
    check_close("z", z, z_ref, F32)
    check_close("dx", xg.grad, dx_ref, F32)
    check_close("dp", pg.grad, dp_ref[..., None], F32)


def test_seq_probability_extremes(device):
    """p = 0 keeps the state, p = 1 replaces it (log(1 - p) = -inf inside the chained scan)."""
    from kernels.ema_seq import ema_seq_fwd

    N, L, T = 2, 400, 64
    g = torch.Generator().manual_seed(2)
    X = torch.randn(N, L, T, generator=g)
    p = torch.sigmoid(torch.randn(N, L, generator=g))
    p[:, 100:140] = 0.0
    p[:, 200] = 1.0
    p[:, 255:257] = 1.0
    y, fin, _ = ema_seq_fwd(p.to(device), X.to(device), "probability")
    torch.cuda.synchronize()
    y_ref, fin_ref = O.ema_seq_loop(X, p, "probability")
    check_close("y", y, y_ref, F32)
    # (equal up to the rounding of the group and tile combination, not bit for bit)
    assert torch.allclose(y[:, 139].cpu(), y[:, 99].cpu(), rtol=1e-5, atol=1e-6)
    assert torch.allclose(y[:, 200].cpu(), X[:, 200], rtol=1e-6, atol=1e-6)


def test_seq_bench_shape_properties(device):
    """b16 nh2 d1024 L4096 bf16: the two forms agree under A = log(1 - p), X = p * x, the final
    state is the last output row, and a split scan (first half, then second half from the first
    half's final state) equals the whole scan."""
    from kernels.ema_seq import ema_seq_fwd

    b, nh, L, d = 16, 2, 4096, 1024
    announce("seq bench shape properties")
    g = torch.Generator(device="cpu").manual_seed(1128)
    x = torch.randn(b, L, nh, d, generator=g).to(BF16).to(device)
    p = torch.sigmoid(-(torch.randn(b, L, nh, generator=g) + 2.0)).to(device)
    y_p, fin_p, _ = ema_seq_fwd(p, x, "probability")
    # (p * x) rounded to bf16 costs up to 2^-9 relative per term: compare at the bf16 bar
    y_a, fin_a, _ = ema_seq_fwd(torch.log1p(-p), (p[..., None] * x.float()).to(BF16), "log_decay")
    check_close("probability form vs log-decay form", y_p, y_a.float(), BF16)
    check_close("final is last row", fin_p, y_p[:, -1].float(), BF16)
    h = 2048 + 128 * 3
    y1, f1, _ = ema_seq_fwd(p[:, :h], x[:, :h], "probability")
    y2, f2, _ = ema_seq_fwd(p[:, h:], x[:, h:], "probability", initial_states=f1)
    torch.cuda.synchronize()
    check_close("split scan, first part", y1, y_p[:, :h].float(), BF16)
    check_close("split scan, second part", y2, y_p[:, h:].float(), BF16)
    check_close("split scan, final", f2, fin_p, BF16)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
def test_seq_packed_sequences(dtype, device):
    """seq_idx: sequences packed along the length axis scan as if each were alone, forward and
    backward; boundaries fall inside tiles, on tile edges and inside 8-row groups."""
    from kernels.ema_seq import ema_seq_scan

    B, L, T = 2, 1000, 72
    announce(f"seq packed sequences {dtype}")
    g = torch.Generator().manual_seed(17)
    x = torch.randn(B, L, T, generator=g).to(dtype)
    A = torch.nn.functional.logsigmoid(torch.randn(B, L, generator=g) + 2.0)
    dy = torch.randn(B, L, T, generator=g).to(dtype)
    cuts = [[0, 3, 128, 131, 640, 1000], [0, 255, 256, 257, 900, 1000]]
    seq_idx = torch.zeros(B, L, dtype=torch.int32)
    for bi, cs in enumerate(cuts):
        for k in range(len(cs) - 1):
            seq_idx[bi, cs[k]:cs[k + 1]] = k
    xg, Ag = x.to(device).requires_grad_(), A.to(device).requires_grad_()
    y = ema_seq_scan(Ag, xg, "log_decay", seq_idx=seq_idx.to(device))
    y.backward(dy.to(device))
    torch.cuda.synchronize()
    y_ref, dx_ref, dA_ref = torch.zeros(B, L, T), torch.zeros(B, L, T), torch.zeros(B, L)
    for bi, cs in enumerate(cuts):
        for k in range(len(cs) - 1):
            sl = slice(cs[k], cs[k + 1])
            y_ref[bi, sl] = O.ema_loop(x[bi:bi + 1, sl].float(), A[bi:bi + 1, sl])[0]
            dxs, dAs = O.ema_loop_bwd(dy[bi:bi + 1, sl].float(), x[bi:bi + 1, sl].float(), A[bi:bi + 1, sl])
            dx_ref[bi, sl], dA_ref[bi, sl] = dxs[0], dAs[0]
    check_close("y", y, y_ref, dtype)
    check_close("dx", xg.grad, dx_ref, dtype)
    check_close("dA", Ag.grad, dA_ref, dtype)


@pytest.mark.parametrize("dtype", [F32, BF16], ids=["f32", "bf16"])
def test_seq_packed_sequences_probability_form(dtype, device):
    """seq_idx in the probability form (a set sign bit on p at sequence starts): forward, the
    gradients of x and p, initial state (reaches the first sequence only), final state (the last
    sequence's) and the gradients through both, against each sequence scanned alone.  One
    sequence starts with p = 0 (encoded as -0.0) and one with p = 1."""
    from kernels.ema_seq import ema_seq_scan

    B, L, T = 2, 1000, 72
    announce(f"seq packed sequences, probability form {dtype}")
    g = torch.Generator().manual_seed(23)
    x = torch.randn(B, L, T, generator=g).to(dtype)
    p = torch.sigmoid(-(torch.randn(B, L, generator=g) + 2.0))
    p[0, 128] = 0.0
    p[1, 257] = 1.0
    dy = torch.randn(B, L, T, generator=g).to(dtype)
    init = torch.randn(B, T, generator=g)
    dfin = torch.randn(B, T, generator=g)
    cuts = [[0, 3, 128, 131, 640, 1000], [0, 255, 256, 257, 900, 1000]]
    seq_idx = torch.zeros(B, L, dtype=torch.int32)
    for bi, cs in enumerate(cuts):
        for k in range(len(cs) - 1):
            seq_idx[bi, cs[k]:cs[k + 1]] = k
    xg, pg = x.to(device).requires_grad_(), p.to(device).requires_grad_()
    ig = init.to(device).requires_grad_()
    y, fin = ema_seq_scan(pg, xg, "probability", initial_states=ig, return_final_states=True,
                          seq_idx=seq_idx.to(device))
    ((y.float() * dy.to(device).float()).sum() + (fin * dfin.to(device)).sum()).backward()
    torch.cuda.synchronize()
    y_ref, dx_ref, dp_ref = torch.zeros(B, L, T), torch.zeros(B, L, T), torch.zeros(B, L)
    fin_ref, dinit_ref = torch.zeros(B, T), torch.zeros(B, T)
    for bi, cs in enumerate(cuts):
        for k in range(len(cs) - 1):
            sl = slice(cs[k], cs[k + 1])
            first, last = k == 0, k == len(cs) - 2
            one = lambda t: t[bi:bi + 1, sl].float()
            i0 = init[bi:bi + 1] if first else None
            df = dfin[bi:bi + 1] if last else None
            ys, fs = O.ema_seq_loop(one(x), p[bi:bi + 1, sl], "probability", i0)
            dxs, dps, dis = O.ema_seq_loop_bwd(one(dy), one(x), p[bi:bi + 1, sl], "probability", i0, df)
            y_ref[bi, sl], dx_ref[bi, sl], dp_ref[bi, sl] = ys[0], dxs[0], dps[0]
            if first:
                dinit_ref[bi] = dis[0]
            if last:
                fin_ref[bi] = fs[0]
    check_close("y", y, y_ref, dtype)
    check_close("final state", fin, fin_ref, dtype)
    check_close("dx", xg.grad, dx_ref, dtype)
    check_close("dp", pg.grad, dp_ref, dtype)
    check_close("dinit", ig.grad, dinit_ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("form", ["log_decay", "probability"])
def test_workspace_ready_or_not(form, dtype, device):
    """A call on a fresh buffer of unknown contents (workspace_ready = 0: the call clears what it
    uses) and calls on one zero-filled buffer that forward and backward share call after call
    (workspace_ready = 1: no clearing launch, words of earlier calls are told apart by their epoch)
    give bit-identical results; so do the autograd entry points, which use the shared buffer."""
    from kernels import _lib
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined
    from kernels.ema_seq import ema_seq_bwd, ema_seq_fwd, ema_seq_scan

    announce(f"workspace ready / not ready {form} {dtype}")
    b, L, nh, d = 2, 700, 2, 320  # ragged last tile, two column tiles
    gen = torch.Generator().manual_seed(11)
    x = torch.randn(b, L, nh, d, generator=gen).to(dtype).to(device)
    dy = torch.randn(b, L, nh, d, generator=gen).to(dtype).to(device)
    p = torch.sigmoid(torch.randn(b, L, nh, generator=gen) - 1.0)
    coef = (p if form == "probability" else torch.log1p(-p)).to(device)
    dfin = torch.randn(b, nh, d, generator=gen).to(device)

    def fresh():  # a buffer of unknown contents (here: all bits set)
        n = _lib.lib().ema_seq_bwd_workspace_bytes(b, nh, L, d)
        return torch.full((n,), 0xFF, dtype=torch.uint8, device=device), 0

    y0, fin0, prev0 = ema_seq_fwd(coef, x, form, workspace=fresh())
    ref = ema_seq_bwd(dy, x, coef, prev0, form, workspace=fresh())
    ref_f = ema_seq_bwd(dy, x, coef, prev0, form, dfinal_states=dfin, workspace=fresh())

    n = _lib.lib().ema_seq_bwd_workspace_bytes(b, nh, L, d)
    shared = torch.zeros(n, dtype=torch.uint8, device=device)
    for rep in range(3):  # the same buffer, forward and backward in turn, never cleared
        y1, fin1, prev1 = ema_seq_fwd(coef, x, form, workspace=(shared, 1))
        assert torch.equal(y0, y1) and torch.equal(fin0, fin1) and torch.equal(prev0, prev1), rep
        got = ema_seq_bwd(dy, x, coef, prev1, form, workspace=(shared, 1))
        assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1]), rep
        got_f = ema_seq_bwd(dy, x, coef, prev1, form, dfinal_states=dfin, workspace=(shared, 1))
        assert torch.equal(got_f[0], ref_f[0]) and torch.equal(got_f[1], ref_f[1]), rep
    hdr = shared[:256].view(torch.int32).cpu()
    assert hdr[0] == 0 and hdr[1] == 0, "ticket and exit counters are left at zero"
    assert hdr[2] == 9, "one epoch per call"
    assert hdr[3] == 0, "no wait ran out"

    # autograd: two backward passes through one forward, on the wrappers' own shared buffer
    xg, cg = x.clone().requires_grad_(), coef.clone().requires_grad_()
    y = ema_seq_scan(cg, xg, form=form)
    y.backward(dy, retain_graph=True)
    g1 = (xg.grad.clone(), cg.grad.clone())
    xg.grad = cg.grad = None
    y.backward(dy)
    assert torch.equal(xg.grad, g1[0]) and torch.equal(cg.grad, g1[1])
    assert torch.equal(g1[0], ref[0]) and torch.equal(g1[1], ref[1])
    if form == "log_decay":
        xg, cg = x.clone().requires_grad_(), coef.clone().requires_grad_()
        ema_matmul_scan_combined(cg, xg, 128).backward(dy)
        assert torch.equal(xg.grad, ref[0]) and torch.equal(cg.grad, ref[1])
        with torch.no_grad():
            assert torch.equal(ema_matmul_scan_combined(coef, x, 128), y0)
    _lib.check_chain_errors(device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_unused_final_state_brings_no_gradient_tensor(dtype, device):
    """When only y is used, autograd hands the backward None for the final state's gradient (not
    zeros), and the result equals that of a call without it."""
    from kernels.ema_seq import EMASeqFn, ema_seq_bwd, ema_seq_fwd

    gen = torch.Generator().manual_seed(3)
    x = torch.randn(1, 300, 2, 64, generator=gen).to(dtype).to(device)
    dy = torch.randn(1, 300, 2, 64, generator=gen).to(dtype).to(device)
    A = torch.nn.functional.logsigmoid(torch.randn(1, 300, 2, generator=gen) + 2).to(device)
    xg, Ag = x.clone().requires_grad_(), A.clone().requires_grad_()
    y, fin = EMASeqFn.apply(Ag, xg, None, "log_decay")
    seen = []
    fin.register_hook(lambda g: seen.append(g))
    y.backward(dy)
    assert seen in ([], [None]), "no tensor of zeros is made up for the unused final state"
    _, _, prev = ema_seq_fwd(A, x)
    dx, dA, _ = ema_seq_bwd(dy, x, A, prev)
    assert torch.equal(xg.grad, dx) and torch.equal(Ag.grad, dA)
    # only the final state is used: dy arrives as None
    xg, Ag = x.clone().requires_grad_(), A.clone().requires_grad_()
    y, fin = EMASeqFn.apply(Ag, xg, None, "log_decay")
    dfin = torch.randn_like(fin)
    fin.backward(dfin)
    dx2, dA2, _ = ema_seq_bwd(torch.zeros_like(x), x, A, prev, dfinal_states=dfin)
    assert torch.equal(xg.grad, dx2) and torch.equal(Ag.grad, dA2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("form", ["log_decay", "probability"])
@pytest.mark.parametrize("row", [126, 127, 128, 254, 255])
def test_single_reset_near_tile_end(form, dtype, row, device):
    """One sequence boundary at a row whose position inside its 128-row tile is 126, 127 or 0,
    with nothing reset in the tile that follows (and the same with p = 1 there): the tile's total
    decay is exactly zero, the later tiles must not see anything from before the boundary, and
    the gradients follow the per-sequence oracle."""
    from kernels.ema_seq import ema_seq_scan

    announce(f"single reset at row {row} {form} {dtype}")
    b, L, nh, d = 2, 640, 1, 256
    gen = torch.Generator().manual_seed(100 + row)
    x = torch.randn(b, L, nh, d, generator=gen).to(dtype)
    dy = torch.randn(b, L, nh, d, generator=gen).to(dtype)
    p = torch.sigmoid(torch.randn(b, L, nh, generator=gen) - 3.0)  # long memory: a leak would show
    seq_idx = torch.zeros(b, L, dtype=torch.int32)
    seq_idx[:, row:] = 1
    for variant in ("seq_idx", "p_is_one"):
        if variant == "p_is_one":
            if form != "probability":
                continue
            pv = p.clone()
            pv[:, row] = 1.0  # y[row] = x[row]: the state before is dropped without any flag
            ids = None
        else:
            pv, ids = p, seq_idx
        coef = pv if form == "probability" else torch.log1p(-pv)
        xg = x.to(device).requires_grad_()
        cg = coef.to(device).requires_grad_()
        y = ema_seq_scan(cg, xg, form=form, seq_idx=None if ids is None else ids.to(device))
        y.backward(dy.to(device))
        # oracle: every piece on its own
        xf, cf = O.to_flat(x.float(), coef)
        dyf, _ = O.to_flat(dy.float(), coef)
        if ids is None:
            y_ref, _ = O.ema_seq_loop(xf, cf, form)
            dx_ref, dc_ref, _ = O.ema_seq_loop_bwd(dyf, xf, cf, form)
        else:
            ys, dxs, dcs = [], [], []
            for sl in (slice(0, row), slice(row, L)):
                yy, _ = O.ema_seq_loop(xf[:, sl], cf[:, sl], form)
                dxx, dcc, _ = O.ema_seq_loop_bwd(dyf[:, sl], xf[:, sl], cf[:, sl], form)
                ys.append(yy), dxs.append(dxx), dcs.append(dcc)
            y_ref, dx_ref, dc_ref = torch.cat(ys, 1), torch.cat(dxs, 1), torch.cat(dcs, 1)
        check_close(f"y[{variant}]", O.to_flat(y.detach().cpu().float(), coef)[0], y_ref, dtype)
        check_close(f"dx[{variant}]", O.to_flat(xg.grad.cpu().float(), coef)[0], dx_ref, dtype)
        dc = cg.grad.cpu().permute(0, 2, 1).reshape(b * nh, L)
        if form == "log_decay" and ids is not None:
            # the gradient with respect to the -inf that marks the boundary is 0 * <...> = 0
            assert torch.equal(dc[:, row], torch.zeros(b * nh))
        check_close(f"dcoef[{variant}]", dc, dc_ref, dtype)


def test_chain_error_is_reported(device):
    """A tile whose predecessor never publishes gives up after spin_limit polls, raises the error
    word of the workspace header and hands on NaN; every kernel still ends.  Forced from the host:
    the ticket counter of a ready workspace is set past the first chunk's tiles, so those tiles
    are never processed and the tiles of the second chunk wait in vain."""
    from kernels import _lib
    from kernels.ema_seq import ema_seq_fwd

    announce("chained scan: bounded wait runs out")
    b, L, nh, d = 1, 512, 2, 256
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(b, L, nh, d, generator=gen).to(device)
    A = torch.nn.functional.logsigmoid(torch.randn(b, L, nh, generator=gen) + 2).to(device)
    n = _lib.lib().ema_seq_fwd_workspace_bytes(b, nh, L, d)
    ws = torch.zeros(n, dtype=torch.uint8, device=device)
    y_ok, _, _ = ema_seq_fwd(A, x, workspace=(ws, 1))
    assert not _lib.chain_error(ws)
    hdr = ws[:256].view(torch.int32)
    cols = b * nh * 2  # sequences x column tiles of 128 float32 columns
    hdr[0] = cols      # tickets of chunk 0 are skipped
    hdr[4] = 64        # polls before a wait gives up
    torch.cuda.synchronize()
    y_bad, _, _ = ema_seq_fwd(A, x, workspace=(ws, 1))
    torch.cuda.synchronize()
    assert _lib.chain_error(ws), "the error word must be raised"
    assert torch.isnan(y_bad[:, 128:]).all(), "everything computed from the missing state is NaN"
    # clearing the workspace puts it back in order
    _lib._clear(ws, device)
    y_again, _, _ = ema_seq_fwd(A, x, workspace=(ws, 1))
    assert torch.equal(y_again, y_ok) and not _lib.chain_error(ws)
