"""The wrappers' shared workspaces are kept per (device, stream, shape): calls of one shape issued
on two streams must not share a ticket counter or an epoch (the reference launches on the current
stream with no state shared between calls, kernels/ema_kernels/ema_state_fwd.py:146), and a
buffer whose address a captured HIP graph holds is never dropped."""
import pytest
import torch

from oracle import ema_oracle as O
from parity_util import announce, check_close

pytestmark = pytest.mark.gpu


def _reference(x, A, dy, b, nh):
    xf, Af = O.to_flat(x.float(), A)
    dyf, _ = O.to_flat(dy.float(), A)
    y = O.from_flat(O.ema_loop(xf, Af), b, nh)
    dx, dA = O.ema_loop_bwd(dyf, xf, Af)
    L = x.shape[1]
    return y, O.from_flat(dx, b, nh), dA.reshape(b, nh, L).permute(0, 2, 1)


def test_same_shape_on_two_streams(device):
    from kernels import _lib
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    announce("two streams, one shape, autograd steps overlapping in time")
    b, nh, L, d = 4, 2, 4096, 512
    dtype = torch.bfloat16
    cases, streams = [], [torch.cuda.Stream(device), torch.cuda.Stream(device)]
    for s in range(2):
        x, A, dy = O.make_inputs(b, nh, L, d, seed=70 + s, dtype=dtype)
        cases.append((x, A, dy, x.to(device).requires_grad_(), A.to(device).requires_grad_(), dy.to(device)))
    torch.cuda.synchronize()
    outs = [None, None]
    for rep in range(6):  # the two streams' launches are enqueued alternately and run side by side
        for s, st in enumerate(streams):
            _, _, _, xg, Ag, dyg = cases[s]
            with torch.cuda.stream(st):
                xg.grad = None
                Ag.grad = None
                y = ema_matmul_scan_combined(Ag, xg, 128)
                y.backward(dyg)
                outs[s] = (y.detach(), xg.grad, Ag.grad)
    torch.cuda.synchronize()
    _lib.check_chain_errors(device)
    keys = [k for k in _lib._shared if k[2:] == (b * nh, L // 128, d)]
    assert len({k[1] for k in keys}) >= 2, "the two streams must not share a workspace"
    for s in range(2):
        x, A, dy = cases[s][:3]
        y_ref, dx_ref, dA_ref = _reference(x, A, dy, b, nh)
        check_close(f"stream {s} y", outs[s][0], y_ref, dtype)
        check_close(f"stream {s} dx", outs[s][1], dx_ref, dtype)
        check_close(f"stream {s} dA", outs[s][2], dA_ref, dtype)


def test_buffer_held_by_a_graph_is_never_dropped(device):
    from kernels import _lib
    from kernels.ema_seq import ema_seq_fwd

    announce("workspace handed out during capture stays, whatever is created afterwards")
    b, nh, L, d = 2, 2, 1024, 256
    x, A, _ = O.make_inputs(b, nh, L, d, seed=81, dtype=torch.float32)
    xs, As = x.to(device), A.to(device)
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        y_e = ema_seq_fwd(As, xs)[0].clone()  # creates the buffer of (side, shape)
    torch.cuda.synchronize()
    key = (device.index, side.cuda_stream, b * nh, L // 128, d)
    assert key in _lib._shared and not _lib._shared[key].pinned
    held = _lib._shared[key].buf
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        y_g = ema_seq_fwd(As, xs)[0]
    assert _lib._shared[key].pinned and _lib._shared[key].buf is held
    # more shapes than the cache keeps: unpinned buffers go, the pinned one stays where it is
    for k in range(_lib._MAX_SHARED + 4):
        xk, Ak, _ = O.make_inputs(1, 1, 128, 256 * (k + 2), seed=k, dtype=torch.float32)
        ema_seq_fwd(Ak.to(device), xk.to(device))
    torch.cuda.synchronize()
    assert key in _lib._shared and _lib._shared[key].buf is held
    assert sum(not e.pinned for e in _lib._shared.values()) <= _lib._MAX_SHARED
    for rep in range(3):
        x2, A2, _ = O.make_inputs(b, nh, L, d, seed=90 + rep, dtype=torch.float32)
        xs.copy_(x2.to(device)); As.copy_(A2.to(device))
        y_ref = ema_seq_fwd(As, xs)[0].clone()
        torch.cuda.synchronize()
        y_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_ref), f"replay {rep} differs from the eager result"
    _lib.check_chain_errors(device)
    xf, Af = O.to_flat(x2, A2)
    check_close("last replay vs oracle", y_g, O.from_flat(O.ema_loop(xf, Af), b, nh), torch.float32)
    assert torch.isfinite(y_e).all()
