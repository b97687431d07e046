"""The entry point that allocates nothing (ema_seq_fwd_static): its results against those of
ema_seq_fwd, which takes a caller-allocated workspace, through the C ABI, on two calls in a
row, the second on a smaller problem, so that the second call meets whatever the first one
left in the shared file-scope scratch.  The two entry points run the same arithmetic in the
same order, so the outputs must be identical bit for bit; y is also held against the
sequential oracle."""
import pytest
import torch

from kernels import _lib
from oracle import ema_oracle as O
from parity_util import announce, check_close

pytestmark = pytest.mark.gpu


def _call(entry, form, coef, x, init, dev):
    """One forward through `entry` ("workspace" or "static"); returns (y, final, prev128)."""
    lib = _lib.lib()
    x, xs, batch, nh, L, T = _lib.seq_view(x)
    cs_, *_ = _lib.decay_view(coef)
    N = batch * nh
    y = torch.full_like(x, float("nan"))
    _, ys, *_ = _lib.seq_view(y)
    final = torch.full((N, T), float("nan"), dtype=torch.float32, device=dev)
    prev128 = torch.full((N, -(-L // 128), T), float("nan"), dtype=torch.float32, device=dev)
    init_ptr = None if init is None else init.data_ptr()
    stream = _lib.stream_ptr(dev)
    with torch.cuda.device(dev):
        if entry == "static":
            st = lib.ema_seq_fwd_static(form, *cs_, *xs, _lib.dtype_code(x), *ys, init_ptr, final.data_ptr(),
                                        prev128.data_ptr(), batch, nh, L, T, stream)
        else:
            nbytes = lib.ema_seq_fwd_workspace_bytes(batch, nh, L, T)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            st = lib.ema_seq_fwd(form, *cs_, *xs, _lib.dtype_code(x), *ys, init_ptr, final.data_ptr(),
                                 prev128.data_ptr(), ws.data_ptr(), nbytes, 0, batch, nh, L, T, stream,
                                 None, None)
    _lib.check(st, "ema_seq_fwd_" + entry)
    torch.cuda.synchronize(dev)
    return y, final, prev128


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("form", ["log_decay", "probability"])
def test_static_entry_matches_workspace_entry_twice(device, dtype, form):
    code = _lib.EMA_FORM_LOG_DECAY if form == "log_decay" else _lib.EMA_FORM_PROBABILITY
    # first a problem of several tiles per column set and several column tiles, then a smaller,
    # ragged one whose status words lie inside the region the first call has written
    for k, (b, nh, L, T) in enumerate([(2, 2, 1000, 320), (1, 3, 300, 64)]):
        announce(f"ema_seq_fwd_static {form} {dtype} call {k}: b{b} nh{nh} L{L} d{T}")
        x, A, _ = O.make_inputs(b, nh, L, T, seed=40 + k, dtype=dtype)
        coef = A if form == "log_decay" else -torch.expm1(A)  # p = 1 - exp(A)
        g = torch.Generator().manual_seed(7 + k)
        init = torch.randn(b * nh, T, generator=g)
        xd, cd, idv = x.to(device), coef.to(device), init.to(device)
        got = _call("static", code, cd, xd, idv, device)
        want = _call("workspace", code, cd, xd, idv, device)
        for name, a, w in zip(("y", "final", "prev128"), got, want):
            assert torch.isfinite(a.float()).all(), name
            assert torch.equal(a, w), f"{name}: the two entry points disagree"
        # and against the sequential recurrence
        xf, cf = O.to_flat(x.float(), coef)
        y_ref, fin_ref = O.ema_seq_loop(xf, cf, form=form, init=init)
        check_close("y", O.to_flat(got[0].cpu().float(), coef)[0], y_ref, dtype)
        check_close("final", got[1].cpu(), fin_ref, torch.float32 if dtype == torch.float32 else dtype)


def test_static_entry_rejects_what_does_not_fit(device):
    lib = _lib.lib()
    cap = lib.ema_seq_fwd_static_max_workspace_bytes()
    assert cap == 16 << 20
    b, nh, L, T = 16, 4, 8192, 1024  # needs more status words than the array holds
    assert lib.ema_seq_fwd_workspace_bytes(b, nh, L, T) > cap
    fake = 0x1000
    st = lib.ema_seq_fwd_static(_lib.EMA_FORM_LOG_DECAY, fake, L * nh, nh, 1, fake, L * nh * T, nh * T, T,
                                _lib.EMA_BF16, fake, L * nh * T, nh * T, T, None, None, fake, b, nh, L, T, None)
    assert st == -7
    with pytest.raises(ValueError):
        _lib.check(st, "ema_seq_fwd_static")


def test_static_entry_in_a_hip_graph_and_its_companions(device):
    """After ema_seq_fwd_static_init nothing but kernel launches happens in a call, so it can be
    captured; every replay must give the bits of ema_seq_fwd.  The error word reads 0 after normal
    calls, and a reset leaves the array usable."""
    import ctypes

    lib = _lib.lib()
    with torch.cuda.device(device):
        assert lib.ema_seq_fwd_static_init() == 0
    b, nh, L, T = 2, 2, 1024, 256
    x, A, _ = O.make_inputs(b, nh, L, T, seed=51, dtype=torch.bfloat16)
    xs, As = x.to(device), A.to(device)
    y = torch.zeros_like(xs)
    final = torch.zeros(b * nh, T, dtype=torch.float32, device=device)
    prev128 = torch.zeros(b * nh, L // 128, T, dtype=torch.float32, device=device)
    _, xa, *_ = _lib.seq_view(xs)
    _, ya, *_ = _lib.seq_view(y)
    ca, *_ = _lib.decay_view(As)

    def launch():
        with torch.cuda.device(device):
            _lib.check(lib.ema_seq_fwd_static(_lib.EMA_FORM_LOG_DECAY, *ca, *xa, _lib.EMA_BF16, *ya, None,
                                              final.data_ptr(), prev128.data_ptr(), b, nh, L, T,
                                              _lib.stream_ptr(device)), "ema_seq_fwd_static")

    announce("ema_seq_fwd_static captured into a graph")
    launch()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    for rep in range(3):
        x2, A2, _ = O.make_inputs(b, nh, L, T, seed=60 + rep, dtype=torch.bfloat16)
        xs.copy_(x2.to(device)); As.copy_(A2.to(device))
        want = _call("workspace", _lib.EMA_FORM_LOG_DECAY, As, xs, None, device)
        y.zero_(); final.zero_(); prev128.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, w in zip(("y", "final", "prev128"), (y, final, prev128), want):
            assert torch.equal(a, w), f"replay {rep}: {name} differs from ema_seq_fwd"
    err = ctypes.c_int(-1)
    with torch.cuda.device(device):
        assert lib.ema_seq_fwd_static_error(ctypes.byref(err), _lib.stream_ptr(device)) == 0 and err.value == 0
        assert lib.ema_seq_fwd_static_error(None, _lib.stream_ptr(device)) == -1
        assert lib.ema_seq_fwd_static_reset(_lib.stream_ptr(device)) == 0
    launch()
    torch.cuda.synchronize()
    assert torch.equal(y, want[0]), "after a reset the entry point gives the same bits"
