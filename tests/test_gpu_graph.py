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


@pytest.mark.parametrize("Q", [128, 512, 640])
def test_da_intra_in_hip_graph(Q, device):
    """The B6 launcher in a graph: the factored form (copies into LDS, a flag per chunk, nothing cleared
    by memset) and, for the chunks of the replay inputs whose cumsum rises, the product form behind it.
    Replays see new inputs, some with rising chunks and some without."""
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd
    from kernels.ema_kernels_bwd.ema_scan_da import _ema_chunk_scan_bwd_ddAcs_stable
    from parity_util import flat_case

    announce(f"hip graph: B6 Q{Q}")
    N, L, T = 3, 1100, 264
    dtype = torch.bfloat16

    def inputs(seed, rising):
        A, X, dy = flat_case(N, L, T, seed=seed, dtype=dtype)
        if rising:
            A = A.clone()
            A[:, 5::Q] = 0.2  # one rising step in every chunk
        return A.to(device), X.to(device), dy.to(device)

    As, Xs, dys = inputs(1, False)

    def run():
        cs = ema_chunk_cumsum_fwd(As, Q)
        return _ema_chunk_scan_bwd_ddAcs_stable(Xs, cs, dys), cs

    run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        for _ in range(2):
            run()
    torch.cuda.current_stream(device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g, cs_g = run()
    for rep, rising in enumerate([True, False, True]):
        A2, X2, dy2 = inputs(50 + rep, rising)
        As.copy_(A2); Xs.copy_(X2); dys.copy_(dy2)
        ref, _ = run()
        ref = ref.clone()
        torch.cuda.synchronize()
        out_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, ref), f"replay {rep}: differs from the eager result"
        want = O.bwd_da_intra(X2.float().cpu(), cs_g.cpu(), dy2.float().cpu())
        check_close(f"replay {rep} vs oracle", out_g.reshape(N, -1)[:, :L], want.reshape(N, -1)[:, :L], dtype)


@pytest.mark.parametrize("packed", [False, True], ids=["plain", "packed"])
def test_ssd_forward_and_backward_stages_in_hip_graph(packed, device):
    """The Mamba-2 SSD launchers enqueue kernels only as well: the five forward stages and the six
    backward stage launchers captured in one graph, replayed with new inputs in the static buffers
    and eager work in between, every replay bit-identical to the eager run."""
    from kernels.mamba_kernels.mamba_combined_fwd import _mamba_chunk_scan_combined_fwd
    from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_da import _chunk_scan_bwd_ddAcs_stable
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_dc import _chunk_scan_bwd_dC
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx
    from kernels.mamba_kernels_bwd.mamba_chunk_state_bwd_db import _chunk_state_bwd_db
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates
    from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd
    from oracle import ssd_oracle as S

    announce(f"hip graph: ssd forward + backward stages, packed={packed}")
    b, L, nh, P, g, N, Q = 2, 600, 4, 64, 1, 128, 256
    BF16 = torch.bfloat16

    def inputs(seed):
        x, dt, A, B, C, _, _ = S.make_inputs(b, L, nh, P, g, N, seed=seed, dtype=BF16)
        dout = torch.randn(b, L, nh, P, generator=torch.Generator().manual_seed(seed)).to(BF16)
        return [t.to(device) for t in (x, dt, A, B, C, dout)]

    static = inputs(1)
    seq = None
    if packed:
        ids = torch.zeros(b, L, dtype=torch.int32)
        ids[0, 100:] += 1
        ids[0, 256:] += 1
        ids[1, 300:] += 1
        seq = ids.to(device)

    def step():
        x, dt, A, B, C, dout = static
        out, _, dt_out, dA_cs, states, final = _mamba_chunk_scan_combined_fwd(x, dt, A, B, C, Q, seq_idx=seq)
        nc = dt_out.shape[2]
        cb = _bmm_chunk_fwd(C, B, Q, seq_idx=seq, output_dtype=torch.float32)
        dprev = _chunk_scan_bwd_dstates(C, dA_cs, dout, seq_idx=seq)
        dstates, ddA_chunk, _ = _state_passing_bwd(states.view(b, nc, nh, P * N), dA_cs[..., -1],
                                                   dprev.view(b, nc, nh, P * N), seq_idx=seq, chunk_size=Q)
        dstates = dstates.view(b, nc, nh, P, N)
        dB, ddA_b = _chunk_state_bwd_db(x, dt_out, dA_cs, dstates, seq_idx=seq, B=B, ngroups=g)
        dC, ddA_c = _chunk_scan_bwd_dC(states, dA_cs, dout, seq_idx=seq, C=C, ngroups=g)
        dx, ddt, _ = _chunk_scan_chunk_state_bwd_dx(x, dt_out, dA_cs, B, cb, dout, dstates, seq_idx=seq)
        ddA = _chunk_scan_bwd_ddAcs_stable(x, dt_out, dA_cs, dout, cb)
        return out, final, dstates, ddA_chunk, dB, ddA_b, dC, ddA_c, dx, ddt, ddA

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream(device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    names = "out final dstates ddA_chunk dB ddA_b dC ddA_c dx ddt ddA".split()
    for rep in range(3):
        for dst, src in zip(static, inputs(10 + rep)):
            dst.copy_(src)
        ref = [t.clone() for t in step()]
        torch.cuda.synchronize()
        for t in captured:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, want in zip(names, captured, ref):
            assert torch.equal(got, want), f"replay {rep}: {name} differs from the eager result"
    x, dt, A, B, C, _ = [t.cpu() for t in static]
    y_ref, _ = S.ssd_loop(x.float(), dt, A, B.float(), C.float(), seq_idx=None if seq is None else seq.cpu())
    check_close("last replay vs the recurrence", captured[0], y_ref, BF16, loose=True)
