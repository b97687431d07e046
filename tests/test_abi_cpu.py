"""CPU-side checks of the C ABI: the built library loads, exports every symbol that
include/ema_hip.h and include/ssd_hip.h declare, and validates its arguments before launching anything (so the
refusals can be exercised without a GPU)."""
import os
import re

import pytest

from kernels import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", "ema_hip.h"), os.path.join(ROOT, "include", "ssd_hip.h")]


def declared_functions():
    names = set()
    for header in HEADERS:
        src = open(header).read()
        src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
        names |= set(re.findall(r"\b((?:ema|ssd)_[a-z_A-Z0-9]+)\s*\(", src))
    return sorted(names)


def test_header_and_binding_agree():
    assert declared_functions() == _lib.exported_symbols()


def test_library_exports_every_declared_symbol():
    handle = _lib.lib()
    for name in declared_functions():
        assert hasattr(handle, name), name
    assert b"gfx950" in handle.ema_version()


def test_status_strings():
    handle = _lib.lib()
    assert handle.ema_status_string(0) == b"ok"
    for code in range(-7, 0):
        assert handle.ema_status_string(code) not in (b"ok", b"unknown status")


def test_workspace_sizes():
    handle = _lib.lib()
    # config 2: N=32, C=32, T=1024, Q=128
    # header + one word per (sequence, 128-row tile) + one per (sequence, tile, column), then scratch
    chain = 256 + 32 * 32 * 8 + 32 * 32 * 1024 * 8
    assert handle.ema_seq_fwd_workspace_bytes(16, 2, 4096, 1024) == chain
    assert handle.ema_fwd_workspace_bytes(16, 2, 4096, 1024, 64) == chain + 32 * 64 * 1024 * 4
    assert handle.ema_fwd_workspace_bytes(16, 2, 4096, 1024, 128) == chain + 32 * 32 * 1024 * 4
    assert handle.ema_seq_bwd_workspace_bytes(16, 2, 4096, 1024) == chain + 8 * 32 * 4096 * 4  # partials per 128 (float32) columns
    assert handle.ema_state_passing_bwd_workspace_bytes(32, 32, 1024) == 32 * 32 * 16 * 4
    # B6: column sums per row tile and row sums of the product form, dots per column tile (4 of 256
    # bfloat16 columns, 8 of 128 float32 columns) and one flag per chunk of the factored form
    da = 2 * 32 * 32 * 128 * 4
    assert handle.ema_chunk_scan_bwd_ddAcs_workspace_bytes(16, 2, 4096, 1024, 128, _lib.EMA_BF16) == da + 4 * 32 * 32 * 128 * 4 + 32 * 32 * 4
    assert handle.ema_chunk_scan_bwd_ddAcs_workspace_bytes(16, 2, 4096, 1024, 128, _lib.EMA_F32) == da + 8 * 32 * 32 * 128 * 4 + 32 * 32 * 4
    assert handle.ema_chunk_scan_bwd_ddAcs_workspace_bytes(16, 2, 4096, 1024, 1024, _lib.EMA_BF16) == (8 + 1 + 4) * 32 * 4 * 1024 * 4 + 32 * 4 * 4
    assert handle.ema_chunk_scan_bwd_ddAcs_workspace_bytes(16, 2, 4096, 1024, 128, 7) == 0
    assert handle.ema_bwd_workspace_bytes(16, 2, 4096, 1024, 128) > 4 * 32 * 32 * 1024 * 4
    assert handle.ema_bwd_workspace_bytes(16, 2, 4096, 1024, 512) == handle.ema_bwd_workspace_bytes(16, 2, 4096, 1024, 128)
    # refused shapes report 0 bytes
    assert handle.ema_fwd_workspace_bytes(0, 2, 4096, 1024, 128) == 0
    assert handle.ema_bwd_workspace_bytes(16, 2, 4096, 1024, _lib.EMA_MAX_CHUNK + 1) == 0


def test_validation_happens_before_any_launch():
    handle = _lib.lib()
    fake = 0x1000  # 16-byte aligned, never dereferenced: every call below is refused
    # null pointers
    assert handle.ema_chunk_cumsum_fwd(None, 1, 1, 0, fake, 1, 1, 8, 4, None) == -1
    # bad shapes
    assert handle.ema_chunk_cumsum_fwd(fake, 8, 1, 0, fake, 0, 1, 8, 4, None) == -2
    assert handle.ema_chunk_cumsum_fwd(fake, 8, 1, 0, fake, 1, 1, 8, 0, None) == -2
    assert handle.ema_chunk_cumsum_fwd(fake, 8, 1, 0, fake, 1, 1, 8, 2048, None) == -2
    # feature size / strides that break 16-byte rows
    assert handle.ema_chunk_state_fwd(fake, 48, 6, 0, _lib.EMA_F32, fake, fake, 1, 1, 8, 6, 4, None) == -3
    assert handle.ema_chunk_state_fwd(fake, 64, 8, 0, _lib.EMA_BF16, fake, fake, 1, 1, 8, 4, 4, None) == -3
    assert handle.ema_chunk_state_fwd(fake + 2, 64, 8, 0, _lib.EMA_BF16, fake, fake, 1, 1, 8, 8, 4, None) == -3
    # unknown dtype
    assert handle.ema_chunk_state_fwd(fake, 64, 8, 0, 7, fake, fake, 1, 1, 8, 8, 4, None) == -4
    # workspace too small
    assert (
        handle.ema_fwd(fake, 8, 1, 0, fake, 64, 8, 0, _lib.EMA_F32, fake, 64, 8, 0, fake, fake, fake,
                       None, fake, 16, 0, 1, 1, 8, 8, 4, None, None, None)
        == -2
    )
    seq = [fake, 64, 8, 0]
    coef = [fake, 8, 1, 0]
    assert (
        handle.ema_seq_bwd(0, *seq, *seq, *coef, fake, None, _lib.EMA_F32, *seq, *coef, None, fake, 16, 1,
                           1, 1, 8, 8, None, None, None)
        == -2
    )
    # unknown form of the recurrence, misaligned workspace
    assert (
        handle.ema_seq_bwd(5, *seq, *seq, *coef, fake, None, _lib.EMA_F32, *seq, *coef, None, fake, 1 << 30, 1,
                           1, 1, 8, 8, None, None, None)
        == -5
    )
    assert handle.ema_workspace_clear(fake + 4, 64, None) == -3
    assert handle.ema_workspace_clear(None, 64, None) == -1


def test_chain_header_layout():
    # the header the library declares, the one the kernels use and the binding's view agree
    src = open(HEADERS[0]).read()
    body = src[src.index("typedef struct {"):src.index("} ema_chain_header;")]
    fields = re.findall(r"uint32_t\s+(\w+)(?:\[(\d+)\])?;", body)
    assert [f[0] for f in fields] == ["ticket", "done", "epoch", "error", "spin_limit", "reserved"]
    assert 4 * (5 + int(fields[-1][1])) == _lib.HEADER_BYTES == 256


def test_ssd_validation_happens_before_any_launch():
    handle = _lib.lib()
    fake = 0x1000
    seq = [fake, 64 * 2 * 64, 2 * 64, 64]
    grp = [fake, 64 * 64, 64, 64]
    ids = [None, 0, 0]  # not a packed batch
    # null pointer, bad shape, unsupported head size, misaligned strides, unknown dtype
    assert handle.ssd_chunk_cumsum_fwd(None, 0, 2, 2, 1, fake, None, fake, fake, 1, 64, 2, 64, 0, 0.0, 1.0, None) == -1
    assert handle.ssd_chunk_cumsum_fwd(fake, 0, 2, 2, 1, fake, None, fake, fake, 1, 0, 2, 64, 0, 0.0, 1.0, None) == -2
    assert handle.ssd_chunk_state_fwd(*grp, *seq, 0, fake, fake, fake, 1, 64, 2, 1, 48, 64, 64, *ids, None) == -5
    assert handle.ssd_chunk_state_fwd(*grp, fake, 8190, 130, 65, 1, fake, fake, fake, 1, 64, 2, 1, 64, 64, 64, *ids, None) == -3
    assert handle.ssd_chunk_state_fwd(*grp, *seq, 9, fake, fake, fake, 1, 64, 2, 1, 64, 64, 64, *ids, None) == -4
    assert handle.ssd_chunk_state_fwd(*grp, *seq, 0, fake, fake, fake, 1, 64, 3, 2, 64, 64, 64, *ids, None) == -2
    assert handle.ssd_bmm_chunk_fwd(*grp, *grp, 0, fake, 1, 1, 64, 1, 64, 64, *ids, None) == -4  # bf16 out of f32 in
    assert handle.ssd_state_passing_fwd(fake, fake, 2, 1, 1, None, fake, 0, fake, 1, 1, 2, 6, *ids, 0, 0, None) == -3
    assert handle.ssd_state_passing_fwd(fake, fake, 2, 1, 1, None, fake, 7, fake, 1, 1, 2, 8, *ids, 0, 0, None) == -4
    # carried states are float32 or of the inputs' type: bfloat16 states with float32 inputs are refused
    assert handle.ssd_chunk_scan_bwd_dc(*seq, 0, fake, fake, 1, *grp, fake, fake, 1, 64, 2, 1, 64, 64, 64, *ids, None) == -4
    # the fused chunk-state + state-passing entry: chunk sizes off the 64-row stages, float32 inputs and head size 128 go to the staged entries
    walk = lambda dtype, chunk, out_dtype=0: handle.ssd_chunk_state_passing_fwd(
        *grp, *seq, dtype, fake, fake, None, fake, out_dtype, fake, 1, 64, 2, 1, 64, 64, chunk, None)
    assert walk(0, 48) == -5 and walk(1, 64, 9) == -4 and walk(1, 0) == -2
    assert handle.ssd_chunk_state_passing_fwd(*grp, *seq, 1, None, fake, None, fake, 1, fake, 1, 64, 2, 1, 64, 64, 64, None) == -1
    # dt and the decay sums are fetched in 16-byte pieces by the kernels that copy straight into LDS
    assert handle.ssd_chunk_state_passing_fwd(*grp, *seq, 1, fake + 4, fake, None, fake, 1, fake, 1, 64, 2, 1, 64, 64, 64, None) == -3
    assert handle.ssd_chunk_state_passing_fwd(*grp, *seq, 1, fake, fake + 8, None, fake, 1, fake, 1, 64, 2, 1, 64, 64, 64, None) == -3
    # a packed batch must come with the chunking that gives nchunks
    assert handle.ssd_state_passing_fwd(fake, fake, 2, 1, 1, None, fake, 0, fake, 1, 2, 2, 8, fake, 64, 1, 64, 16, None) == -2
    # the reverse walk (dstates + state passing in one kernel): what it is not written for goes to the two launchers
    grp128 = [fake, 64 * 128, 128, 128]
    need = handle.ssd_chunk_scan_state_passing_bwd_workspace_bytes(1, 1, 2)
    assert need == 1 * 1 * 2 * 8 * 4 and handle.ssd_chunk_scan_state_passing_bwd_workspace_bytes(0, 1, 2) == 0

    def rwalk(dtype=1, chunk=128, states_dtype=1, dA=fake, ddA=fake, ws_bytes=need, dout=seq, hdim=64, dstate=128, out_dtype=1):
        return handle.ssd_chunk_scan_state_passing_bwd(*grp128, *dout, dtype, dA, fake, states_dtype, None, fake, out_dtype,
                                                       ddA, None, fake, ws_bytes, 1, 64, 2, 1, hdim, dstate, chunk, None)
    assert rwalk(dtype=0) == -5 and rwalk(chunk=64) == -5 and rwalk(chunk=160) == -5 and rwalk(states_dtype=0) == -5
    assert rwalk(hdim=128) == -5 and rwalk(out_dtype=7) == -4
    assert rwalk(ddA=None) == -1 and rwalk(dA=fake + 4) == -3 and rwalk(ws_bytes=need - 4) == -2
    assert rwalk(dout=[fake, 64 * 2 * 64, -2 * 64, 64]) == -5  # a reversed view: byte offsets are formed unsigned


def test_error_mapping():
    with pytest.raises(AssertionError):
        _lib.check(-2, "x")
    with pytest.raises(AssertionError):
        _lib.check(-3, "x")
    with pytest.raises(TypeError):
        _lib.check(-4, "x")
    with pytest.raises(NotImplementedError):
        _lib.check(-5, "x")
    with pytest.raises(RuntimeError):
        _lib.check(-6, "x")
    _lib.check(0, "x")


def test_ops_refuse_cpu_tensors():
    import torch

    from kernels.ema_kernels.ema_cumsum import ema_chunk_cumsum_fwd

    with pytest.raises(RuntimeError):
        ema_chunk_cumsum_fwd(torch.zeros(1, 8), 4)
