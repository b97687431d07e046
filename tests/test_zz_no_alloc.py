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
