"""The EMA kernels against the Mamba-2 SSD kernels on the same problem, both through the C ABI
on the GPU: the reference's own EMA tests hold its EMA launchers against its Mamba launchers
this way (kernels/tests/ema/test_ema_state_fwd.py:120-141,
kernels/tests/ema_bwd/test_ema_scan_bwd_dstates.py:95-125): with dt = -log(1 - p), A = -1,
B = p, C = 1 and x = X / dt per head, the SSD recurrence h = exp(dt A) h + dt B x, y = C h is the
EMA y = (1 - p) y + p X.  The state size is 1, as in the reference's tests (head sizes 32 and
512 there), or 64 with B and C carrying their value in component 0, which is the shape the SSD
kernels take as it is.  float32, where both families compute in full precision."""
import pytest
import torch

from parity_util import announce, check_close

pytestmark = pytest.mark.gpu

F32 = torch.float32


def _encode(b, L, nh, P, nstate, seed, device):
    gen = torch.Generator().manual_seed(seed)
    X = torch.randn(b, L, nh * P, generator=gen)
    p = torch.sigmoid(torch.randn(b, L, generator=gen) - 1.0)
    dt1 = -torch.log1p(-p)                                    # (b, L)
    ema = dict(A=torch.log1p(-p), X=X * p[..., None])         # the EMA kernels' inputs
    Bm = torch.zeros(b, L, 1, nstate)
    Bm[..., 0, 0] = p
    Cm = torch.zeros(b, L, 1, nstate)
    Cm[..., 0, 0] = 1.0
    ssd = dict(x=(X / dt1[..., None]).reshape(b, L, nh, P), dt=dt1[..., None].expand(b, L, nh).contiguous(),
               A=-torch.ones(nh), B=Bm, C=Cm)
    to = lambda d: {k: v.to(device) for k, v in d.items()}
    return to(ema), to(ssd)


CASES = [  # b, L, nh, P, Q, state size
    (2, 512, 2, 64, 128, 64), (1, 700, 4, 64, 256, 64), (2, 300, 2, 128, 64, 64),
    (2, 512, 16, 32, 128, 1),   # HEAD_DIM 512 as 16 heads of 32: kernels/tests/ema/test_ema_scan_fwd.py:73-74
    (1, 640, 2, 512, 128, 1),   # 1024 features as 2 heads: kernels/benchmarks/ema/scan_fwd/scan_fwd_bench.py:20-42
]


@pytest.mark.parametrize("b,L,nh,P,Q,nstate", CASES)
def test_forward_agrees(b, L, nh, P, Q, nstate, device):
    from kernels.ema_kernels.ema_combined_fwd import _ema_matmul_scan_combined_fwd
    from kernels.mamba_kernels.mamba_combined_fwd import _mamba_chunk_scan_combined_fwd

    announce(f"ema vs ssd forward b{b} L{L} nh{nh} P{P} Q{Q}")
    ema, ssd = _encode(b, L, nh, P, nstate, seed=L + Q, device=device)
    y_e, cs_e, prev_e, fin_e = _ema_matmul_scan_combined_fwd(ema["A"], ema["X"], Q)
    y_s, _, dt_out, dA_cs, prev_s, fin_s = _mamba_chunk_scan_combined_fwd(ssd["x"], ssd["dt"], ssd["A"], ssd["B"],
                                                                          ssd["C"], Q)
    torch.cuda.synchronize()
    nc = cs_e.shape[1]
    check_close("y", y_s.reshape(b, L, nh * P), y_e.cpu(), F32)
    check_close("dA_cumsum", dA_cs[:, 0], cs_e.cpu(), F32)                      # the heads share one decay
    check_close("states entering the chunks", prev_s[..., 0].reshape(b, nc, nh * P), prev_e.cpu(), F32)
    check_close("final state", fin_s[..., 0].reshape(b, nh * P), fin_e.cpu(), F32)
    if nstate > 1:
        assert float(prev_s[..., 1:].abs().max()) == 0.0 and float(fin_s[..., 1:].abs().max()) == 0.0


@pytest.mark.parametrize("b,L,nh,P,Q,nstate", CASES)
def test_backward_stages_agree(b, L, nh, P, Q, nstate, device):
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd
    from kernels.ema_kernels_bwd.ema_scan_bwd import _ema_chunk_scan_bwd_dstates
    from kernels.ema_kernels_bwd.ema_state_passing_bwd_dstates import _ema_state_passing_bwd
    from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates
    from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd

    announce(f"ema vs ssd backward stages b{b} L{L} nh{nh} P{P} Q{Q}")
    ema, ssd = _encode(b, L, nh, P, nstate, seed=2 * L + Q, device=device)
    gen = torch.Generator().manual_seed(L)
    dout = torch.randn(b, L, nh * P, generator=gen).to(device)
    cs_e = ema_chunk_cumsum_fwd(ema["A"], Q)
    dA_cs, _ = _chunk_cumsum_fwd(ssd["dt"], ssd["A"], Q)
    nc = cs_e.shape[1]

    # gradient of the states entering the chunks: component 0 of the SSD result (C = e_0)
    ds_e = _ema_chunk_scan_bwd_dstates(cs_e, dout)
    ds_s = _chunk_scan_bwd_dstates(ssd["C"], dA_cs, dout.reshape(b, L, nh, P), dtype=F32)
    check_close("dstates of the chunk scan", ds_s[..., 0].reshape(b, nc, nh * P), ds_e.cpu(), F32)
    if nstate > 1:
        assert float(ds_s[..., 1:].abs().max()) == 0.0

    # reverse inter-chunk recurrence on the same flattened states
    states = torch.randn(b, nc, nh * P, generator=gen).to(device)
    g_e, ddA_e, _ = _ema_state_passing_bwd(states, cs_e[:, :, -1], ds_e, chunk_size=Q)
    st4 = states.reshape(b, nc, nh, P)
    g_s, ddA_s, _ = _state_passing_bwd(st4, dA_cs[:, :, :, -1], ds_e.reshape(b, nc, nh, P), chunk_size=Q)
    check_close("dstates of state passing", g_s.reshape(b, nc, nh * P), g_e.cpu(), F32)
    check_close("ddA of the chunk decays (summed over heads)", ddA_s.sum(1), ddA_e.cpu(), F32)


def test_main_script_flow(device):
    """The three providers of the reference's main.py:77-143 on its own shapes (batch 2, length
    512, 64 features as 2 heads of 32, chunk size 8): the (x, p) entry point, the Mamba-encoded
    EMA entry point and the Mamba forward itself (main.py takes that one from mamba_ssm) against
    the loop z = (1 - p) z + p x."""
    from kernels.ema import ema_scan_combined
    from kernels.ema_combined import ema_chunk_scan_combined
    from kernels.mamba_kernels.mamba_combined_fwd import mamba_chunk_scan_combined_fwd

    announce("main.py flow: ema_scan_combined, ema_chunk_scan_combined, mamba forward")
    b, L, D, hd, nh, Q = 2, 512, 64, 32, 2, 8
    gen = torch.Generator().manual_seed(42)
    X = torch.randn(b, L, D, generator=gen)
    P = torch.rand(b, L, 1, generator=gen) * 0.98 + 0.01
    ref = torch.empty_like(X)
    z = torch.zeros(b, D)
    for t in range(L):
        z = (1 - P[:, t]) * z + P[:, t] * X[:, t]
        ref[:, t] = z
    dt1 = -torch.log(1 - P).squeeze(-1)
    X_m = (X / dt1[..., None]).reshape(b, L, nh, hd).to(device)
    dt = dt1[..., None].expand(b, L, nh).contiguous().to(device)
    A = -torch.ones(nh, device=device)
    B_m = P.reshape(b, L, 1, 1).to(device)
    C_m = torch.ones_like(B_m)
    check_close("ema_scan_combined(X, P)", ema_scan_combined(X.to(device), P.to(device)), ref, F32)
    got = ema_chunk_scan_combined(X_m, dt, A, B_m, C_m, chunk_size=Q, seq_idx=None)
    check_close("ema_chunk_scan_combined", got.reshape(b, L, D), ref, F32)
    got = mamba_chunk_scan_combined_fwd(X_m, dt, A, B_m, C_m, Q)
    check_close("mamba forward", got.reshape(b, L, D), ref, F32)


def test_legacy_stage_modules(device):
    """The stage launchers under the module paths of the reference's legacy headed path, run in the
    order of kernels/ema_combined.py:43-55 with an A that must be ignored, against the same loop."""
    from kernels.ema_bmm import _bmm_chunk_fwd
    from kernels.ema_chunk_scan import _chunk_scan_fwd
    from kernels.ema_chunk_state import _chunk_cumsum_fwd, _simplified_chunk_state_fwd
    from kernels.ema_state_passing import _state_passing_fwd

    announce("legacy stage modules: cumsum, simplified chunk state, state passing, bmm, chunk scan")
    b, L, nh, P, Q = 2, 300, 2, 32, 64
    ema, ssd = _encode(b, L, nh, P, 1, seed=3, device=device)
    x, dt, Bm, Cm = ssd["x"], ssd["dt"], ssd["B"], ssd["C"]
    dA_cs, dt_out = _chunk_cumsum_fwd(dt, torch.full((nh,), -7.0, device=device), Q)
    states = _simplified_chunk_state_fwd(Bm, x, dt_out, dA_cs, states_in_fp32=True)
    states, final = _state_passing_fwd(states.reshape(b, -1, nh, P), dA_cs[:, :, :, -1], chunk_size=Q,
                                       out_dtype=torch.float32)
    CB = _bmm_chunk_fwd(Cm, Bm, Q, output_dtype=torch.float32)
    out, _ = _chunk_scan_fwd(CB, x, dt_out, dA_cs, Cm, states.reshape(b, -1, nh, P, 1))
    ref = torch.empty(b, L, nh * P)
    z = torch.zeros(b, nh * P)
    Xc, Ac = ema["X"].cpu(), ema["A"].cpu()
    for t in range(L):
        z = torch.exp(Ac[:, t, None]) * z + Xc[:, t]
        ref[:, t] = z
    check_close("out", out.reshape(b, L, nh * P), ref, F32)
    check_close("final", final.reshape(b, nh * P), ref[:, -1], F32)
