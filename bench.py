#!/usr/bin/env python3
"""Benchmark of the EMA chunked scan, forward + backward, on one MI355X.

One step = one forward and one backward through the autograd entry point
(ema_matmul_scan_combined(...).backward(dy)) of benchmark configuration 3 at chunk size 128:
b16 nh2 d1024 L4096, bf16 x / dy, fp32 log-decay and accumulation.  The forward is one pass
over x, the backward one pass over x and dy (three launches per step: the two single-pass
kernels and the small reduction of the log-decay gradient).  Inputs are synthetic and resident
in HBM before the timed region; the steps run back to back and rotate over several input sets,
so that no step finds its inputs in the 256 MB last-level cache and every kernel runs while the
output of the one before is still on its way to HBM, as in a training loop.  The outputs of the
last few launches stay allocated, as activations and gradients do in a training step: a timed loop
that drops each output at once makes the allocator hand the same block to the next launch, whose
stores the last-level cache then absorbs, and reads up to 20 % faster than the kernel is.

Prints ONE JSON line.  `roofline` describes the kernel with the largest share of the step; its
duration is that of the very dispatches of the timed steps (events that the runtime stamps with
start and end of the dispatch, collected in a second pass of the same loop).  `configs` holds
the other benchmark configurations: chunk sizes 256 and 512 (step, and the three per-stage
contraction launchers with their dense-FLOP rate), the long-sequence configuration 4, the
Mamba-2 SSD configuration 5 and `ref_f32_fwd`, the forward on the workload of the reference's own
benchmark script (float32, b16 L8192 d1024) beside the only figures the reference publishes.
`stage_launchers` times every per-stage launcher of the reference's interface on its own, and
the copies that bound what a kernel can reach here: a linear one, torch's, and four that move the
tensor in the tile order of the single-pass kernels (in the kernels' own shape, with fewer and
longer waves, with the rows interleaved as the memory system prefers them, and interleaved with an
exchange through LDS).  `cpu_baseline` is the sequential CPU
oracle timed on a bounded sample and scaled to the full workload.
"""
import argparse
import json
import os
import platform
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "triton-kernels_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (summaries and commands under
# profiles/), scaled by what the same counters read for a plain 268 435 456-byte device copy
# (FETCH_SIZE reads 131 085 KiB for it, factor 1.99982; WRITE_SIZE reads 262 144 KiB, factor 1).
TRAFFIC_BYTES = {"fwd_single_pass": 570370042, "bwd_single_pass": 841222651}
TRAFFIC_SOURCE = "profiles/single_pass_tile_kernels_b16_nh2_d1024_L4096_c128_hbm_traffic.txt (rocprofv3 --pmc, not measured by this run)"
# the same for the SSD stage kernels at configuration 5 (finishing kernels added to their stage)
SSD_TRAFFIC_BYTES = {
    "chunk_cumsum": 25320408, "chunk_state": 571591572, "state_passing": 419465499, "bmm_chunk": 100772767,
    "chunk_scan": 742930943, "bwd_dstates": 446640967, "bwd_state_passing": 409601722, "bwd_db": 496071800,
    "bwd_dc": 469831534, "bwd_dx": 1029628081, "bwd_ddAcs": 599926788,
}

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--chunk", type=int, default=128)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--nheads", type=int, default=2)
    ap.add_argument("--seqlen", type=int, default=4096)
    ap.add_argument("--dim", type=int, default=1024)
    ap.add_argument("--u-mean", type=float, default=2.0, help="mean of u in the decay sigmoid(u)")
    ap.add_argument("--sets", type=int, default=3, help="input sets the steps rotate over")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-stage launcher timing")
    ap.add_argument("--no-configs", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--workload", default="ema", choices=["ema", "ssd"],
                    help="ema: the headline EMA scan step (default); ssd: the Mamba-2 SSD stages at "
                    "benchmark configuration 5 (b8 nh32 hdim64 dstate128 g1 L8192 chunk256, bf16) alone")
    ap.add_argument("--stage", default=None,
                    help="time only this stage (a name from the stage tables, or fwd, bwd, bwd_saved, step, copy) "
                    "and print a short JSON line; used for profiles and counter collection")
    return ap.parse_args()


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return platform.processor() or "unknown"


def ema_inputs(torch, dev, b, nh, L, T, seed, u_mean=2.0, dtype=None):
    """Synthetic inputs of the EMA benchmark configurations, generated on the device:
    x, dy ~ N(0,1) (b, L, nh, T) bf16; A = log(sigmoid(u)), u ~ N(u_mean, 1), (b, L, nh) fp32."""
    dtype = dtype or torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn(b, L, nh, T, generator=g, device=dev, dtype=torch.float32).to(dtype)
    u = torch.randn(b, L, nh, generator=g, device=dev, dtype=torch.float32) + u_mean
    A = torch.nn.functional.logsigmoid(u)
    dy = torch.randn(b, L, nh, T, generator=g, device=dev, dtype=torch.float32).to(dtype)
    return x, A, dy


def algorithmic_bytes(N, L, T, Q, esize):
    """Compulsory HBM bytes per launch of each stage (every input read once, every output
    written once), and of the whole forward / backward."""
    C = -(-L // Q)
    x = N * L * T * esize
    a = N * L * 4
    st = N * C * T * 4
    return {
        "cumsum": 2 * a,
        "chunk_state": x + a + st,
        "state_passing_fwd": 2 * st + N * C * 4 + N * T * 4,
        "chunk_scan": 2 * x + a + st,
        "bwd_dstates": x + a + st,
        "state_passing_bwd": 3 * st + 2 * N * C * 4,
        "bwd_dx": 2 * x + a + st,
        "bwd_db": x + st + 2 * a,
        "bwd_dc": x + st + 2 * a,
        "bwd_da_intra": 2 * x + 2 * a,
        "bwd_fused_dx_dA": 3 * x + 2 * a + 2 * st,
        "fwd": 2 * x + a,
        "bwd": 3 * x + 2 * a,
    }


KEEP_ALIVE = 4  # results of the last launches that stay allocated (see time_region)


def time_region(fn, iters, torch):
    """Average milliseconds of fn() over `iters` calls, HIP events on the current stream.

    What fn returns stays alive for a few more calls, as the outputs of a kernel do in a training
    step.  Dropped at once, an output tensor goes back to the allocator and the next launch writes
    into the very block the launch before has just written, which the 256 MB last-level cache
    still holds: the stores are absorbed there and a kernel that writes as much as it reads looks
    up to 20 % faster than it is (forward kernel 86 us instead of 107 us at b16 nh2 d1024 L4096)."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    alive = [None] * KEEP_ALIVE
    torch.cuda.synchronize()
    start.record()
    for i in range(iters):
        alive[i % KEEP_ALIVE] = fn(i)
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def cpu_baseline(args, torch):
    """Sequential CPU oracle (forward + closed-form reverse recurrence) on a sample of the
    workload's sequences, scaled linearly to all of them."""
    from oracle import ema_oracle as O

    threads = torch.get_num_threads()
    nseq_total = args.batch * args.nheads
    sample_b = min(4, args.batch)  # about 10 s of CPU work: 20 to 30 repetitions of a quarter of the batch
    x, A, dy = O.make_inputs(sample_b, args.nheads, args.seqlen, args.dim, seed=1, dtype=torch.bfloat16)
    xf, Af = O.to_flat(x.float(), A)
    dyf, _ = O.to_flat(dy.float(), A)
    t0 = time.perf_counter()
    reps = 0
    while True:
        O.ema_loop(xf, Af)
        O.ema_loop_bwd(dyf, xf, Af)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 40:
            break
    per = (time.perf_counter() - t0) / reps
    scale = nseq_total / (sample_b * args.nheads)
    return {
        "value": per * scale * 1e3,
        "unit": "ms",
        "cores": threads,
        "cpu_model": cpu_model(),
        "threads": threads,
        "kind": "port",
        "sample": f"{sample_b * args.nheads} of {nseq_total} sequences (L={args.seqlen}, d={args.dim}), "
        f"fwd + bwd sequential recurrence in fp32 torch, {reps} repetitions, scaled x{scale:g}",
    }


# ------------------------------------------------------------------------------------------------
# EMA step on one configuration
# ------------------------------------------------------------------------------------------------

class EmaRun:
    """Input sets and step functions of one EMA configuration."""

    def __init__(self, torch, dev, b, nh, L, T, Q, nsets, u_mean, seed0):
        from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined
        from kernels.ema_seq import ema_seq_bwd, ema_seq_fwd

        self.torch, self.dev = torch, dev
        self.b, self.nh, self.L, self.T, self.Q = b, nh, L, T, Q
        self.N = b * nh
        self.sets = [ema_inputs(torch, dev, b, nh, L, T, seed0 + s, u_mean) for s in range(nsets)]
        self.grad_sets = [(x.clone().requires_grad_(), A.clone().requires_grad_(), dy) for x, A, dy in self.sets]
        self._apply, self._fwd, self._bwd = ema_matmul_scan_combined, ema_seq_fwd, ema_seq_bwd
        self._saved = None

    def step(self, i):
        # one training step through the autograd entry point: the forward keeps the states entering
        # each 128-row chunk (4 MB) and the backward reuses them
        x, A, dy = self.grad_sets[i % len(self.grad_sets)]
        x.grad = None
        A.grad = None
        self._apply(A, x, self.Q).backward(dy)

    def fwd_only(self, i, events=None, workspace=None):
        x, A, dy = self.sets[i % len(self.sets)]
        return self._fwd(A, x, kernel_events=events, workspace=workspace)

    def bwd_saved(self, i, events=None, workspace=None):  # backward as the autograd step runs it, with the forward's states
        if self._saved is None:
            self._saved = [self._fwd(A, x)[2] for x, A, dy in self.sets]
        x, A, dy = self.sets[i % len(self.sets)]
        return self._bwd(dy, x, A, self._saved[i % len(self.sets)], kernel_events=events, workspace=workspace)

    def ready_workspace(self):
        """A zero-filled workspace of the caller's own (passed as ready): what code that captures
        its step into a HIP graph creates once before the capture, so that the graph holds no
        clearing launches."""
        from kernels import _lib

        n = _lib.lib().ema_seq_bwd_workspace_bytes(self.b, self.nh, self.L, self.T)
        return (self.torch.zeros(n, dtype=self.torch.uint8, device=self.dev), 1)

    def step_kernels(self, iters):
        """The same two launches per step as `step` makes (sequence-level forward, then backward
        with the forward's states), back to back, with the runtime's start / stop stamps of every
        dispatch: in-sequence durations of the two single-pass kernels, in ms."""
        torch = self.torch
        self.bwd_saved(0)
        evs = []
        for i in range(2 * iters):
            ev = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            ev[0].record()
            ev[1].record()  # materialise the handles before the timed launches
            evs.append(ev)
        alive = [None] * (2 * KEEP_ALIVE)  # outputs stay allocated for a few steps, as in time_region
        for i in range(3):
            self.fwd_only(i)
            self.bwd_saved(i)
        torch.cuda.synchronize()
        for i in range(iters):
            alive[(2 * i) % len(alive)] = self.fwd_only(i, evs[2 * i])
            alive[(2 * i + 1) % len(alive)] = self.bwd_saved(i, evs[2 * i + 1])
        torch.cuda.synchronize()
        f = sum(evs[2 * i][0].elapsed_time(evs[2 * i][1]) for i in range(iters)) / iters
        bw = sum(evs[2 * i + 1][0].elapsed_time(evs[2 * i + 1][1]) for i in range(iters)) / iters
        return f, bw

    def measure(self, steps, warmup):
        torch = self.torch
        for i in range(warmup):
            self.step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ms_events = time_region(self.step, steps, torch)
        wall = (time.perf_counter() - t0) * 1e3 / steps
        ab = algorithmic_bytes(self.N, self.L, self.T, self.Q, 2)
        ms_step = max(ms_events, wall)
        kf, kb = self.step_kernels(steps)
        # inputs read once, outputs written once; the chunk-entry states the forward saves for the
        # backward (N * ceil(L / 128) * T floats, under 1 % of the tensors) are not counted
        fb, bb = ab["fwd"], ab["bwd"]
        return {
            "ms_per_step": ms_step,
            "hbm_frac_of_peak_fwd+bwd": (ab["fwd"] + ab["bwd"]) / ms_step / 1e6 / HBM_PEAK_GBS,
            "algorithmic_bytes_fwd+bwd": ab["fwd"] + ab["bwd"],
            "step_kernels": {
                "fwd_single_pass": {"ms": kf, "bytes": fb, "GBps": fb / kf / 1e6, "hbm_frac": fb / kf / 1e6 / HBM_PEAK_GBS},
                "bwd_single_pass": {"ms": kb, "bytes": bb, "GBps": bb / kb / 1e6, "hbm_frac": bb / kb / 1e6 / HBM_PEAK_GBS},
            },
        }


def ref_f32_forward(torch, dev, iters):
    """Forward of ema_matmul_scan_combined on the reference benchmark's own workload and inputs
    (kernels/benchmarks/ema_bench.py:96-98,134-138), with its byte model (:141-143)."""
    from kernels.ema_kernels.ema_combined_fwd import ema_matmul_scan_combined

    B, L, T, Q = 16, 8192, 1024, 128
    gen = torch.Generator(device=dev).manual_seed(8192)
    sets = []
    for _ in range(2):
        x = torch.randn(B, L, T, device=dev, generator=gen)
        p = torch.sigmoid(torch.randn(B, L, 1, device=dev, generator=gen))
        sets.append((torch.log(1 - p).squeeze(-1), x * p))
    with torch.no_grad():
        fn = lambda i: ema_matmul_scan_combined(*sets[i % 2], Q)
        for i in range(3):
            fn(i)
        ms = time_region(fn, iters, torch)
    nbytes = 2 * B * L * T * 4 + B * L * 4
    return {
        "workload": "EMA forward, float32, B16 L8192 T1024 chunk128, flat (B, L, T) layout, inputs as in the reference's bench",
        "ms": ms, "bytes_reference_model": nbytes, "GBps": nbytes / ms / 1e6, "hbm_frac": nbytes / ms / 1e6 / HBM_PEAK_GBS,
        "reference_published": {"hardware": "H100 80GB HBM3", "ms": 0.638, "GBps": 1684.37,
                                "source": "bench_dump/H100_80GB_HBM3/raw_triton_matmul_b16_seq8192_chunk128_h1024_nh2.bench:3"},
    }


def make_stages(sets, Q, torch):
    """name -> callable(i) launching one stage through its per-stage launcher (one kernel each,
    plus at most one tiny finishing kernel) on input set i; `copy` is a plain device copy of
    one x-sized tensor."""
    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd
    from kernels.ema_kernels.ema_scan_fwd import _ema_scan_fwd
    from kernels.ema_kernels.ema_state_fwd import _ema_chunk_state_fwd
    from kernels.ema_kernels.ema_state_pass import _ema_state_passing_fwd
    from kernels.ema_kernels_bwd.ema_chunk_scan_bwd_dc import _ema_chunk_scan_bwd_dC
    from kernels.ema_kernels_bwd.ema_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx
    from kernels.ema_kernels_bwd.ema_chunk_state_bwd_db import _ema_chunk_state_bwd_db
    from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_bwd_dx_dA_fused
    from kernels.ema_kernels_bwd.ema_scan_bwd import _ema_chunk_scan_bwd_dstates
    from kernels.ema_kernels_bwd.ema_scan_da import _ema_chunk_scan_bwd_ddAcs_stable
    from kernels.ema_kernels_bwd.ema_state_passing_bwd_dstates import _ema_state_passing_bwd

    inter = []
    for x, A, dy in sets:
        cs = ema_chunk_cumsum_fwd(A, Q)
        states = _ema_chunk_state_fwd(x, cs)
        prev, _ = _ema_state_passing_fwd(states, cs[..., -1], out_dtype=torch.float32)
        ds = _ema_chunk_scan_bwd_dstates(cs, dy)
        g, _, _ = _ema_state_passing_bwd(prev, cs[..., -1], ds)
        if Q == 128:
            fused_in = (cs, prev, g)
        else:  # the fused backward kernel always works on 128-row chunks
            cs1 = ema_chunk_cumsum_fwd(A, 128)
            prev1, _ = _ema_state_passing_fwd(_ema_chunk_state_fwd(x, cs1), cs1[..., -1], out_dtype=torch.float32)
            g1, _, _ = _ema_state_passing_bwd(prev1, cs1[..., -1], _ema_chunk_scan_bwd_dstates(cs1, dy))
            fused_in = (cs1, prev1, g1)
        inter.append((cs, states, prev, ds, g, fused_in))

    def pick(i):
        k = i % len(sets)
        return sets[k] + inter[k]

    stages = {
        "cumsum": lambda i: ema_chunk_cumsum_fwd(pick(i)[1], Q),
        "chunk_state": lambda i: _ema_chunk_state_fwd(pick(i)[0], pick(i)[3]),
        "state_passing_fwd": lambda i: _ema_state_passing_fwd(pick(i)[4], pick(i)[3][..., -1]),
        "chunk_scan": lambda i: _ema_scan_fwd(pick(i)[0], pick(i)[3], pick(i)[5]),
        "bwd_dstates": lambda i: _ema_chunk_scan_bwd_dstates(pick(i)[3], pick(i)[2]),
        "state_passing_bwd": lambda i: _ema_state_passing_bwd(pick(i)[5], pick(i)[3][..., -1], pick(i)[6]),
        "bwd_dx": lambda i: _chunk_scan_chunk_state_bwd_dx(pick(i)[0], pick(i)[3], pick(i)[2], pick(i)[7]),
        "bwd_db": lambda i: _ema_chunk_state_bwd_db(pick(i)[0], pick(i)[3], pick(i)[7]),
        "bwd_dc": lambda i: _ema_chunk_scan_bwd_dC(pick(i)[5], pick(i)[3], pick(i)[2]),
        "bwd_da_intra": lambda i: _ema_chunk_scan_bwd_ddAcs_stable(pick(i)[0], pick(i)[3], pick(i)[2]),
        "bwd_fused_dx_dA": lambda i: _ema_bwd_dx_dA_fused(
            pick(i)[0], pick(i)[8][0], pick(i)[2], pick(i)[8][1], pick(i)[8][2]),
    }
    outs = [torch.empty_like(s[0]) for s in sets]
    stages["copy"] = lambda i: outs[i % len(sets)].copy_(sets[i % len(sets)][0])
    # the plainest streaming kernels, as ceilings: x -> out (the forward's traffic) and
    # x, dy -> out (the backward's)
    from kernels import _lib

    def stream(i, two):
        x, A, dy = sets[i % len(sets)]
        o = outs[i % len(sets)]
        _lib.check(_lib.lib().ema_stream_copy(x.data_ptr(), dy.data_ptr() if two else None, o.data_ptr(),
                                              x.numel() * x.element_size(), _lib.stream_ptr(x.device)), "ema_stream_copy")

    stages["stream_copy"] = lambda i: stream(i, False)
    stages["stream_2in_1out"] = lambda i: stream(i, True)

    # the same bytes in the access pattern of the single-pass kernels (tiles of 128 rows x 512
    # bytes, one persistent workgroup per compute unit): in the shape the two kernels load and
    # store in (sixteen waves with 8 consecutive rows each; also with two inputs, as the backward
    # kernel has), with eight waves of 16 rows, in the order the memory system likes best, and in
    # that order with the rows handed on through LDS
    def tile_copy(i, rowmap, two=False):
        x, A, dy = sets[i % len(sets)]
        o = outs[i % len(sets)]
        b, L, nh, d = x.shape
        _lib.check(_lib.lib().ema_tile_pattern_copy(x.data_ptr(), dy.data_ptr() if two else None, o.data_ptr(), b, L,
                                                    nh * d * x.element_size(), rowmap, _lib.stream_ptr(x.device)),
                   "ema_tile_pattern_copy")

    x0 = sets[0][0]
    if x0.shape[1] % 128 == 0 and (x0.shape[2] * x0.shape[3] * x0.element_size()) % 512 == 0:
        stages["tile_copy_scan_order"] = lambda i: tile_copy(i, 0)
        stages["tile_copy_scan_order_2in_1out"] = lambda i: tile_copy(i, 0, two=True)
        stages["tile_copy_scan_order_8_waves"] = lambda i: tile_copy(i, 3)
        stages["tile_copy_best_order"] = lambda i: tile_copy(i, 1)
        stages["tile_copy_exchange"] = lambda i: tile_copy(i, 2)
    return stages


def time_stages(sets, Q, iters, torch, only=None):
    """Per-stage timing with HIP events on the launch stream (back-to-back launches over the
    rotating input sets)."""
    stages = make_stages(sets, Q, torch)
    x = sets[0][0]
    N, L, T = x.shape[0] * x.shape[2], x.shape[1], x.shape[3]
    xb = x.numel() * x.element_size()
    ab = dict(algorithmic_bytes(N, L, T, Q, 2), copy=2 * xb, stream_copy=2 * xb, stream_2in_1out=3 * xb,
              tile_copy_scan_order=2 * xb, tile_copy_scan_order_2in_1out=3 * xb, tile_copy_scan_order_8_waves=2 * xb,
              tile_copy_best_order=2 * xb, tile_copy_exchange=2 * xb)
    res = {}
    for name, fn in stages.items():
        if only and name not in only:
            continue
        for i in range(3):
            fn(i)
        ms = time_region(fn, iters, torch)
        gbps = ab[name] / ms / 1e6
        res[name] = {"ms": ms, "GBps": gbps, "hbm_frac": gbps / HBM_PEAK_GBS, "bytes": ab[name]}
    flops = 2.0 * Q * L * T * N
    for name in ("chunk_scan", "bwd_dx", "bwd_da_intra"):  # dense-equivalent count, Q*Q per chunk
        if name in res:
            tf = flops / res[name]["ms"] / 1e9
            res[name]["dense_TFLOPs"] = tf
            res[name]["mfma_frac_dense"] = tf / MFMA_BF16_PEAK_TFLOPS
    return res


# ------------------------------------------------------------------------------------------------
# Mamba-2 SSD stages at configuration 5
# ------------------------------------------------------------------------------------------------

def ssd_stages(torch, steps, warmup, only=None):
    """The five forward stage launchers, their combined forward and the six backward stage
    launchers at benchmark configuration 5, timed with events on the launch stream; per stage the
    algorithmic bytes (inputs read once, outputs written once) against the HBM peak and, for the
    MFMA stages, dense FLOPs against the bf16 MFMA peak."""
    from kernels.mamba_kernels.mamba_bmm import _bmm_chunk_fwd
    from kernels.mamba_kernels.mamba_combined_fwd import _chunk_state_passing_fwd, _mamba_chunk_scan_combined_fwd
    from kernels.mamba_kernels.mamba_cumsum import _chunk_cumsum_fwd
    from kernels.mamba_kernels.mamba_scan_fwd import _chunk_scan_fwd
    from kernels.mamba_kernels.mamba_state_fwd import _chunk_state_fwd
    from kernels.mamba_kernels.mamba_state_pass import _state_passing_fwd
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_da import _chunk_scan_bwd_ddAcs_stable
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_bwd_dc import _chunk_scan_bwd_dC
    from kernels.mamba_kernels_bwd.mamba_chunk_scan_chunk_state_bwd_dx import _chunk_scan_chunk_state_bwd_dx
    from kernels.mamba_kernels_bwd.mamba_chunk_state_bwd_db import _chunk_state_bwd_db
    from kernels.mamba_kernels_bwd.mamba_scan_bwd import _chunk_scan_bwd_dstates
    from kernels.mamba_kernels_bwd.mamba_scan_state_passing_bwd import _chunk_scan_state_passing_bwd
    from kernels.mamba_kernels_bwd.mamba_state_passing_bwd_dstates import _state_passing_bwd

    dev = torch.device("cuda:0")
    b, L, nh, P, g, N, Q = 8, 8192, 32, 64, 1, 128, 256
    C = L // Q
    sets = []
    for s in range(2):
        gen = torch.Generator(device=dev).manual_seed(5 + s)
        x = torch.randn(b, L, nh, P, generator=gen, device=dev).to(torch.bfloat16)
        B = torch.randn(b, L, g, N, generator=gen, device=dev).to(torch.bfloat16)
        Cm = torch.randn(b, L, g, N, generator=gen, device=dev).to(torch.bfloat16)
        dt = torch.nn.functional.softplus(torch.randn(b, L, nh, generator=gen, device=dev) * 0.5 - 2.0)
        A = -torch.exp(torch.rand(nh, generator=gen, device=dev) * 2.772588722239781)  # -exp(U(log 1, log 16))
        sets.append((x, dt, A, B, Cm))
    inter = []
    for x, dt, A, B, Cm in sets:
        out, _, dt_out, dA_cs, states, _ = _mamba_chunk_scan_combined_fwd(x, dt, A, B, Cm, Q)
        st = _chunk_state_fwd(B, x, dt_out, dA_cs)
        cb = _bmm_chunk_fwd(Cm, B, Q, output_dtype=torch.float32)
        dout = torch.randn_like(x)
        dprev = _chunk_scan_bwd_dstates(Cm, dA_cs, dout)  # state-sized gradients travel in bf16 too
        dstates, _, _ = _state_passing_bwd(states.view(b, C, nh, P * N), dA_cs[..., -1], dprev.view(b, C, nh, P * N))
        inter.append((dt_out, dA_cs, st, states, cb, dout, dprev, dstates.view(b, C, nh, P, N)))
    del out, dprev, dstates

    def pick(i):
        k = i % len(sets)
        return sets[k] + inter[k]

    stages = {
        "chunk_cumsum": lambda i: _chunk_cumsum_fwd(pick(i)[1], pick(i)[2], Q),
        "chunk_state": lambda i: _chunk_state_fwd(pick(i)[3], pick(i)[0], pick(i)[5], pick(i)[6]),
        "state_passing": lambda i: _state_passing_fwd(pick(i)[7].view(b, C, nh, P * N), pick(i)[6][..., -1],
                                                      out_dtype=torch.bfloat16),
        # the two stages above as the combined forward runs them: one kernel, local states kept on chip
        "chunk_state_passing": lambda i: _chunk_state_passing_fwd(pick(i)[3], pick(i)[0], pick(i)[5], pick(i)[6],
                                                                  out_dtype=torch.bfloat16),
        "bmm_chunk": lambda i: _bmm_chunk_fwd(pick(i)[4], pick(i)[3], Q, output_dtype=torch.float32),
        "chunk_scan": lambda i: _chunk_scan_fwd(pick(i)[9], pick(i)[0], pick(i)[5], pick(i)[6], pick(i)[4], pick(i)[8]),
        "forward": lambda i: _mamba_chunk_scan_combined_fwd(*pick(i)[:5], Q),
        # backward stages (the reference has no combined backward): x dt A B C | dt_out dA st states cb dout dprev dstates
        "bwd_dstates": lambda i: _chunk_scan_bwd_dstates(pick(i)[4], pick(i)[6], pick(i)[10]),
        "bwd_state_passing": lambda i: _state_passing_bwd(pick(i)[8].view(b, C, nh, P * N), pick(i)[6][..., -1],
                                                          pick(i)[11].view(b, C, nh, P * N)),
        # the two stages above in one kernel: the chunk's gradient stays in the accumulators
        "bwd_dstates_state_passing": lambda i: _chunk_scan_state_passing_bwd(pick(i)[4], pick(i)[6], pick(i)[10],
                                                                             pick(i)[8]),
        "bwd_db": lambda i: _chunk_state_bwd_db(pick(i)[0], pick(i)[5], pick(i)[6], pick(i)[12], B=pick(i)[3], ngroups=g),
        "bwd_dc": lambda i: _chunk_scan_bwd_dC(pick(i)[8], pick(i)[6], pick(i)[10], C=pick(i)[4], ngroups=g),
        "bwd_dx": lambda i: _chunk_scan_chunk_state_bwd_dx(pick(i)[0], pick(i)[5], pick(i)[6], pick(i)[3], pick(i)[9],
                                                           pick(i)[10], pick(i)[12]),
        "bwd_ddAcs": lambda i: _chunk_scan_bwd_ddAcs_stable(pick(i)[0], pick(i)[5], pick(i)[6], pick(i)[10], pick(i)[9]),
    }

    def backward_pass(i):
        """The backward stages chained as a caller would chain them (the reference has no combined
        backward): the reverse walk's dstates feed dx and dB; one timed region, five launchers."""
        x, _, _, B, Cm, dt_out, dA_cs, _, states, cb, dout = pick(i)[:11]
        dstates, _, _ = _chunk_scan_state_passing_bwd(Cm, dA_cs, dout, states)
        dstates = dstates.view(b, C, nh, P, N)
        _chunk_scan_chunk_state_bwd_dx(x, dt_out, dA_cs, B, cb, dout, dstates)
        _chunk_state_bwd_db(x, dt_out, dA_cs, dstates, B=B, ngroups=g)
        _chunk_scan_bwd_dC(states, dA_cs, dout, C=Cm, ngroups=g)
        _chunk_scan_bwd_ddAcs_stable(x, dt_out, dA_cs, dout, cb)

    stages["backward_pass"] = backward_pass
    xb = b * L * nh * P * 2
    bc = b * L * g * N * 2
    dtb = b * L * nh * 4
    stb = b * C * nh * P * N * 4
    cbb = b * C * g * Q * Q * 4
    # the states entering the chunks travel in bf16, as in the reference's combined forward, and so
    # do the state-sized gradients of the backward stages (their dtype / dstates_dtype arguments)
    pvb = stb // 2
    nbytes = {
        "chunk_cumsum": 3 * dtb, "chunk_state": xb + bc + 2 * dtb + stb, "state_passing": stb + pvb + dtb // Q,
        "chunk_state_passing": xb + bc + 2 * dtb + pvb,
        "bmm_chunk": 2 * bc + cbb, "chunk_scan": cbb + 2 * xb + bc + pvb + 2 * dtb,
        "forward": 2 * xb + 2 * bc + dtb,
        "bwd_dstates": xb + bc + dtb + pvb, "bwd_state_passing": 3 * pvb + 2 * dtb // Q,
        "bwd_dstates_state_passing": xb + bc + dtb + 2 * pvb + dtb // Q,
        "bwd_db": xb + pvb + 2 * dtb + bc + 2 * bc + dtb, "bwd_dc": xb + pvb + dtb + bc + 2 * bc + dtb,
        "bwd_dx": cbb + 3 * xb + bc + pvb + 3 * dtb, "bwd_ddAcs": 2 * xb + 3 * dtb + cbb,
    }
    # in and out of the chained backward: x, dout, B, C, cb, dt, dA, states read; dx, dB, dC, ddt, ddA (x2) written
    nbytes["backward_pass"] = 3 * xb + 4 * bc + cbb + 5 * dtb + pvb
    units = b * C * nh
    flops = {"chunk_state": 2 * Q * P * N * units, "chunk_state_passing": 2 * Q * P * N * units, "bmm_chunk": 2 * Q * Q * N * b * C * g,
             "chunk_scan": (2 * Q * Q * P + 2 * Q * N * P) * units, "bwd_dstates": 2 * Q * P * N * units,
             "bwd_dstates_state_passing": 2 * Q * P * N * units,
             "bwd_db": 2 * Q * P * N * units, "bwd_dc": 2 * Q * P * N * units,
             "bwd_dx": (2 * Q * Q * P + 2 * Q * N * P) * units, "bwd_ddAcs": 2 * Q * Q * P * units}
    res = {}
    for name, fn in stages.items():
        if only and name != only:
            continue
        for i in range(warmup):
            fn(i)
        ms = time_region(fn, steps, torch)
        res[name] = {"ms": ms, "bytes": nbytes[name], "GBps": nbytes[name] / ms / 1e6,
                     "hbm_frac": nbytes[name] / ms / 1e6 / HBM_PEAK_GBS}
        if name in flops:
            res[name]["dense_TFLOPs"] = flops[name] / ms / 1e9
            res[name]["mfma_frac"] = flops[name] / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS
    if not only:
        six = ("bwd_dstates", "bwd_state_passing", "bwd_db", "bwd_dc", "bwd_dx", "bwd_ddAcs")
        res["backward_stages_sum"] = {"ms": sum(res[k]["ms"] for k in six)}
        # the same work with the first two stages in one kernel
        res["backward_sum_with_reverse_walk"] = {
            "ms": res["bwd_dstates_state_passing"]["ms"] + sum(res[k]["ms"] for k in six[2:])}
    return res


def ssd_main(args):
    import torch

    from oracle import ssd_oracle as S

    res = ssd_stages(torch, args.steps, args.warmup, args.stage)
    if args.stage:
        print(json.dumps({"stage": args.stage, **res[args.stage], "steps": args.steps}))
        return
    # the roofline entry is for the dominant kernel of the timed region, which is the forward
    dom = max((k for k in res if not k.startswith(("forward", "bwd_", "backward"))),
              key=lambda k: res[k]["ms"])
    out = {
        "metric": "Mamba-2 SSD fwd ms @ b8 nh32 hdim64 dstate128 g1 L8192 c256",
        "value": res["forward"]["ms"], "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["forward"]["ms"], "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Mamba-2 SSD chunked scan forward, five stages, b8 nh32 hdim64 dstate128 g1 L8192 "
                   "chunk256, bf16 x/B/C, fp32 dt/A, D = 0, no gate"},
        "stages": res,
        "roofline": {"kernel": dom, "bound": "hbm", "achieved": res[dom]["GBps"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": res[dom]["hbm_frac"], "traffic": SSD_TRAFFIC_BYTES.get(dom),
                     "traffic_source": "profiles/ssd_stages_b8_nh32_hd64_ds128_L8192_c256_hbm_traffic.txt"},
    }
    if not args.no_cpu_baseline:
        b, L, nh, P, g, N = 8, 8192, 32, 64, 1, 128
        x, dt, A, B, Cm, _, _ = S.make_inputs(1, 512, nh, P, g, N, seed=5, dtype=torch.bfloat16)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 10.0 and reps < 400:  # about 10 s of CPU work
            S.ssd_loop(x.float(), dt, A, B.float(), Cm.float())
            reps += 1
        per = (time.perf_counter() - t0) / reps
        scale = b * L / 512
        out["cpu_baseline"] = {"value": per * scale * 1e3, "unit": "ms", "cores": torch.get_num_threads(),
                               "cpu_model": cpu_model(), "threads": torch.get_num_threads(), "kind": "port",
                               "sample": f"1 of {b} sequences, 512 of {L} positions, sequential recurrence in fp32 "
                               f"torch, {reps} repetitions, scaled x{scale:g}"}
    print(json.dumps(out))


# ------------------------------------------------------------------------------------------------

# ------------------------------------------------------------------------------------------------
# Per-tile phases of the two single-pass kernels (development build with timestamps)
# ------------------------------------------------------------------------------------------------

TIMING_LIB = os.path.join(ROOT, "triton-kernels_amd", "lib", "libema_hip_timing.so")


def tile_phases(args):
    """Loads the timestamp build of the library (python triton-kernels_amd/build.py --timing) and prints, for
    the forward and the backward single-pass kernel, how a tile's time divides into phases as
    thread 0 of the workgroup sees them (it belongs to a wave that looks back), and how much of
    the launch is lost at its start and end.  Stamps are the 100 MHz constant clock."""
    if not os.path.exists(TIMING_LIB):
        print("tile_phases needs the timestamp build: python triton-kernels_amd/build.py --timing", file=sys.stderr)
        sys.exit(2)
    os.environ["EMA_HIP_LIB"] = TIMING_LIB
    import ctypes

    import numpy as np
    import torch

    from kernels import _lib
    from kernels.ema_seq import ema_seq_bwd, ema_seq_fwd

    dev = torch.device("cuda:0")
    b, nh, L, T = args.batch, args.nheads, args.seqlen, args.dim
    sets = [ema_inputs(torch, dev, b, nh, L, T, 1000 + args.chunk + s, args.u_mean) for s in range(args.sets)]
    lib = _lib.lib()
    lib.ema_debug_set_timing.restype = ctypes.c_int
    lib.ema_debug_set_timing.argtypes = [ctypes.c_void_p]
    tiles = b * nh * (-(-L // 128)) * (-(-T // 256))
    stamps = torch.zeros(tiles, 16, dtype=torch.int64, device=dev)
    prevs = [ema_seq_fwd(A, x)[2] for x, A, dy in sets]
    def pct(v, q):
        return float(np.percentile(v, q)) if len(v) else float("nan")

    def report(name, launch, phases, s0, s1):
        """phases: (label, from slot, to slot); s0 / s1: the slots that open and close a tile."""
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for e in ev:
            e[0].record(), e[1].record()
        lib.ema_debug_set_timing(None)
        for i in range(args.warmup):
            launch(i, None)
        torch.cuda.synchronize()
        # the launch whose stamps are read is the last of a back-to-back series, as in the bench
        lib.ema_debug_set_timing(stamps.data_ptr())
        for i in range(args.steps):
            launch(i, ev[i])
        torch.cuda.synchronize()
        lib.ema_debug_set_timing(None)
        ms = [e[0].elapsed_time(e[1]) for e in ev]
        ts = stamps.cpu().numpy().astype(np.int64)
        wg = ts[:, 7]
        t0, tend = ts[:, s0], ts[:, s1]
        tick = 0.01  # us per stamp unit
        span = (tend.max() - t0.min()) * tick
        print(f"\n{name}: {tiles} tiles on {len(set(wg.tolist()))} workgroups; launch {ms[-1] * 1e3:.1f} us by events "
              f"(mean of {args.steps}: {sum(ms) / len(ms) * 1e3:.1f}), first stamp to last stamp {span:.1f} us")
        print(f"  {'phase':66s} {'median':>8s} {'p95':>8s} {'mean':>8s}  us")
        first = np.zeros(tiles, dtype=bool)
        order = np.lexsort((t0, wg))
        first[order[np.r_[True, wg[order][1:] != wg[order][:-1]]]] = True
        for label, a, bb in phases:
            ok = (ts[:, a] > 0) & (ts[:, bb] > 0) & ~first
            v = (ts[ok, bb] - ts[ok, a]) * tick
            print(f"  {label:66s} {pct(v, 50):8.2f} {pct(v, 95):8.2f} {float(v.mean()) if len(v) else float('nan'):8.2f}")
        same = wg[order][1:] == wg[order][:-1]
        per = (t0[order][1:] - t0[order][:-1])[same] * tick
        print(f"  {'tile period (start to start, same workgroup)':66s} {pct(per, 50):8.2f} {pct(per, 95):8.2f} {float(per.mean()):8.2f}")
        v = (ts[first, s1] - ts[first, s0]) * tick
        print(f"  {'first tile of a workgroup, start to end':66s} {pct(v, 50):8.2f} {pct(v, 95):8.2f} {float(v.mean()):8.2f}")
        ids = np.unique(wg)
        starts = np.array([t0[wg == w].min() for w in ids])
        ends = np.array([tend[wg == w].max() for w in ids])
        stagger = (starts - starts.min()) * tick
        idle = (ends.max() - ends) * tick
        ntile = np.array([(wg == w).sum() for w in ids])
        print(f"  workgroup start after the first one: median {pct(stagger, 50):.2f}, max {stagger.max():.2f} us")
        print(f"  workgroup idle before the last one ends: median {pct(idle, 50):.2f}, mean {idle.mean():.2f}, max {idle.max():.2f} us "
              f"(tiles per workgroup {ntile.min()}..{ntile.max()})")
        print(f"  launch by events minus first-to-last stamp: {ms[-1] * 1e3 - span:.1f} us (dispatch before the first stamp, "
              "stores in flight and end of kernel after the last)")
        return ts

    # the outputs of the last few launches stay alive, as they do in a training step: an output
    # written into the block that the launch before has just written is absorbed by the
    # last-level cache and the kernel looks 20 % faster than it is
    alive = [None] * 4

    def fwd_launch(i, e):
        alive[i % 4] = ema_seq_fwd(sets[i % len(sets)][1], sets[i % len(sets)][0], kernel_events=e)

    def bwd_launch(i, e):
        k = i % len(sets)
        alive[i % 4] = ema_seq_bwd(sets[k][2], sets[k][0], sets[k][1], prevs[k], kernel_events=e)

    fwd_ph = [("start -> coefficients and rows of the tile have arrived", 0, 5),
              ("local pass, LDS, barrier 1", 5, 1),
              ("chain over the 16 row groups, publish aggregate", 1, 4),
              ("look-back (first look to state known)", 4, 6),
              ("publish prefix, store states, request next rows, barrier 2", 6, 2),
              ("final pass, stores issued", 2, 3),
              ("whole tile", 0, 3)]
    report("fwd_tile_kernel (thread 0, a wave that owns rows and looks back)", fwd_launch, fwd_ph, 0, 3)
    bwd_ph = [("start -> coefficients and rows of the tile have arrived", 0, 5),
              ("two local passes, LDS, barrier 1", 5, 1),
              ("chains over the row groups, publish, first look, barrier 2", 1, 2),
              ("forward values again; look-back done (thread 0)", 2, 6),
              ("publish prefix, barrier 3", 6, 3),
              ("final pass: stores, dots, next rows requested", 3, 4),
              ("whole tile", 0, 4)]
    report("bwd_tile_kernel (thread 0)", bwd_launch, bwd_ph, 0, 4)


def main():
    args = parse()
    if args.stage == "tile_phases":
        return tile_phases(args)
    if args.gpus != 1:
        print("bench.py measures one GPU only: the EMA scan has no multi-GPU path in this build "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if args.workload == "ssd":
        return ssd_main(args)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    b, nh, L, T, Q = args.batch, args.nheads, args.seqlen, args.dim, args.chunk
    run = EmaRun(torch, dev, b, nh, L, T, Q, args.sets, args.u_mean, seed0=1000 + Q)

    if args.stage:
        from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_chunk_scan_combined_bwd

        stages = {"fwd": run.fwd_only, "bwd_saved": run.bwd_saved, "step": run.step,
                  "bwd": lambda i: _ema_chunk_scan_combined_bwd(run.sets[i % len(run.sets)][2], run.sets[i % len(run.sets)][0],
                                                                run.sets[i % len(run.sets)][1], Q)}
        if args.stage not in stages:
            stages = make_stages(run.sets, Q, torch)
        fn = stages[args.stage]
        for i in range(args.warmup):
            fn(i)
        ms = time_region(fn, args.steps, torch)
        print(json.dumps({"stage": args.stage, "ms": ms, "steps": args.steps}))
        return

    head = run.measure(args.steps, args.warmup)
    ms_step = head["ms_per_step"]
    main_k = head["step_kernels"]
    ab = algorithmic_bytes(run.N, L, T, Q, 2)

    # the same step (forward launcher, then backward launcher with the forward's states) captured
    # once per input set into a HIP graph and replayed, as the reference's benchmarks time their
    # kernels (do_bench_cudagraph, kernels/benchmarks/ema_bench.py:102)
    ms_graph = None
    try:
        run.bwd_saved(0)
        graphs, keep = [], []
        ws = run.ready_workspace()  # the graphs replay one after the other on one stream: one buffer serves all
        torch.cuda.synchronize()
        for k in range(len(run.sets)):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                keep.append((run.fwd_only(k, workspace=ws), run.bwd_saved(k, workspace=ws)))
            graphs.append(gr)
        for i in range(args.warmup):
            graphs[i % len(graphs)].replay()
        ms_graph = time_region(lambda i: graphs[i % len(graphs)].replay(), args.steps, torch)
        del graphs, keep
    except Exception as exc:  # capture is an extra; the eager figure stands without it
        print(f"graph capture skipped: {exc}", file=sys.stderr)

    ms_fwd = time_region(run.fwd_only, args.steps, torch)
    ms_bwd_saved = time_region(run.bwd_saved, args.steps, torch)
    from kernels.ema_kernels_bwd.ema_combined_bwd import _ema_chunk_scan_combined_bwd

    ms_bwd = time_region(lambda i: _ema_chunk_scan_combined_bwd(run.sets[i % len(run.sets)][2], run.sets[i % len(run.sets)][0],
                                                                run.sets[i % len(run.sets)][1], Q), args.steps, torch)

    kernels = {} if args.no_kernels else time_stages(run.sets, Q, args.steps, torch)

    shape = f"b{b} nh{nh} d{T} L{L} c{Q}"
    out = {
        "metric": f"EMA scan fwd+bwd ms @ {shape}",
        "value": ms_step,
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"EMA chunked scan fwd+bwd, b{b} nh{nh} d{T} L{L} chunk{Q}, bf16 x/dy, fp32 log-decay",
            "batch": b, "nheads": nh, "seqlen": L, "dim": T, "chunk": Q,
        },
        "graph_replay_ms_per_step": ms_graph,
        "fwd_ms": ms_fwd,
        "bwd_ms": ms_bwd_saved,
        "bwd_standalone_ms": ms_bwd,
        "hbm_algorithmic_GBps": {
            "fwd": ab["fwd"] / ms_fwd / 1e6,
            "bwd": ab["bwd"] / ms_bwd_saved / 1e6,
            "fwd+bwd": (ab["fwd"] + ab["bwd"]) / ms_step / 1e6,
        },
        "hbm_frac_of_peak_fwd+bwd": head["hbm_frac_of_peak_fwd+bwd"],
        "step_kernels": main_k,
        "stage_launchers": kernels,
    }
    dom = max(main_k, key=lambda k: main_k[k]["ms"])
    out["roofline"] = {
        "kernel": dom,
        "bound": "hbm",
        "achieved": main_k[dom]["GBps"],
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": main_k[dom]["GBps"] / HBM_PEAK_GBS,
        "traffic": TRAFFIC_BYTES.get(dom),
        "traffic_source": TRAFFIC_SOURCE,
        "duration": "mean over the timed fwd,bwd sequence of the time between events recorded on the launch stream directly before and after the launch",
    }
    del run
    torch.cuda.empty_cache()

    if not args.no_configs:
        cfgs = {}
        # configuration 3 at the other chunk sizes: the step, and the three contraction launchers
        for q in (256, 512):
            r = EmaRun(torch, dev, 16, 2, 4096, 1024, q, 2, 2.0, seed0=1000 + q)
            m = r.measure(max(10, args.steps // 2), 3)
            st = time_stages(r.sets, q, max(10, args.steps // 2), torch, only=("chunk_scan", "bwd_dx", "bwd_da_intra"))
            cfgs[f"c{q}"] = {"workload": f"b16 nh2 d1024 L4096 chunk{q}", "step_ms": m["ms_per_step"],
                             "hbm_frac": m["hbm_frac_of_peak_fwd+bwd"], "step_kernels": m["step_kernels"],
                             "contraction_launchers": st}
            del r, st
            torch.cuda.empty_cache()
        # configuration 4: long sequence, long memory
        r = EmaRun(torch, dev, 4, 2, 32768, 1024, 256, 2, 4.0, seed0=4000)
        m = r.measure(max(10, args.steps // 2), 3)
        cfgs["cfg4"] = {"workload": "b4 nh2 d1024 L32768 chunk256, u ~ N(4,1)", "step_ms": m["ms_per_step"],
                        "hbm_frac": m["hbm_frac_of_peak_fwd+bwd"], "algorithmic_bytes": m["algorithmic_bytes_fwd+bwd"],
                        "step_kernels": m["step_kernels"]}
        del r
        torch.cuda.empty_cache()
        # the one workload the reference publishes numbers for (kernels/benchmarks/ema_bench.py:134-145): forward
        # only, float32, B16 L8192 T1024 chunk 128, flat layout, rate under its byte model 2|x| + |p|
        cfgs["ref_f32_fwd"] = ref_f32_forward(torch, dev, max(10, args.steps // 2))
        torch.cuda.empty_cache()
        # configuration 5: Mamba-2 SSD stages
        s5 = ssd_stages(torch, max(10, args.steps // 2), 3)
        cfgs["cfg5"] = {"workload": "Mamba-2 SSD b8 nh32 hdim64 dstate128 g1 L8192 chunk256, bf16",
                        "forward_ms": s5["forward"]["ms"],
                        # the combined forward runs chunk_cumsum, chunk_state_passing (chunk_state and
                        # state_passing in one kernel), bmm_chunk and chunk_scan
                        "forward_stages_ms": {k: s5[k]["ms"] for k in ("chunk_cumsum", "chunk_state", "state_passing",
                                                                      "chunk_state_passing", "bmm_chunk", "chunk_scan")},
                        "backward_stages_ms": {k: v["ms"] for k, v in s5.items() if k.startswith("bwd_")},
                        "backward_stages_sum_ms": s5["backward_stages_sum"]["ms"],
                        # with bwd_dstates and bwd_state_passing replaced by bwd_dstates_state_passing
                        "backward_sum_with_reverse_walk_ms": s5["backward_sum_with_reverse_walk"]["ms"],
                        # the same five launchers chained in one timed region, dstates flowing from the
                        # reverse walk into dx and dB
                        "backward_pass_ms": s5["backward_pass"]["ms"],
                        "stages": s5}
        torch.cuda.empty_cache()
        out["configs"] = cfgs

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args, torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
