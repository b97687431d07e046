"""The EMA entry points enqueue kernels only (no allocation, no host synchronisation, no memset
nodes), so a forward + backward step can be captured into a HIP graph, as the reference's
benchmarks do with do_bench_cudagraph (kernels/benchmarks/ema_bench.py:102).  The graph is
replayed several times with eager work and synchronisations in between and every replay is
checked against the eager result."""
import pytest
import torch

from oracle import ema_oracle as O
from parity_util import announce, check_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_step_in_hip_graph(dtype, device):
    from kernels.ema_kernels.ema_combined_fwd import _ema_matmul_scan_combined_fwd
    from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_chunk_scan_combined_bwd

    announce(f"hip graph step {dtype}")
    b, nh, L, d, Q = 2, 2, 1024, 256, 128
    x, A, dy = O.make_inputs(b, nh, L, d, seed=21, dtype=dtype)
    xs, As, dys = x.to(device), A.to(device), dy.to(device)  # static inputs of the graph

    def step():
        y, cs, prev, final, p128 = _ema_matmul_scan_combined_fwd(As, xs, Q, return_prev128=True)
        dx, ddA = _ema_chunk_scan_combined_bwd(dys, xs, As, Q, prev128=p128)[:2]
        return y, dx, ddA

    y_e, dx_e, dA_e = (t.clone() for t in step())
    torch.cuda.synchronize()

    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up on the capture stream
            step()
    torch.cuda.current_stream(device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_g, dx_g, dA_g = step()

    for rep in range(3):
        # new inputs in the static buffers, eager work and a synchronisation between replays
        x2, A2, dy2 = O.make_inputs(b, nh, L, d, seed=30 + rep, dtype=dtype)
        xs.copy_(x2.to(device)); As.copy_(A2.to(device)); dys.copy_(dy2.to(device))
        y_ref, dx_ref, dA_ref = (t.clone() for t in step())
        torch.cuda.synchronize()
        y_g.zero_(); dx_g.zero_(); dA_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_ref), f"replay {rep}: y differs from the eager result"
        assert torch.equal(dx_g, dx_ref), f"replay {rep}: dx differs from the eager result"
        check_close(f"replay {rep} dA", dA_g, dA_ref, torch.float32)
    xf, Af = O.to_flat(x2.float(), A2)
    check_close("last replay vs oracle", y_g, O.from_flat(O.ema_loop(xf, Af), b, nh), dtype)
