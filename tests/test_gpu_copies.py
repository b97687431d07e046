"""The copies that bench.py times as ceilings (measurement aids of the library, not part of the
path) must at least be copies: every pattern moves every byte to its place."""
import pytest
import torch

from parity_util import announce

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("slabs,rows,row_bytes", [(3, 256, 1024), (16, 128, 4096), (5, 384, 512)])
@pytest.mark.parametrize("rowmap", [0, 1, 2, 3], ids=["scan_order", "best_order", "exchange", "scan_order_8_waves"])
def test_tile_pattern_copy_copies(rowmap, slabs, rows, row_bytes, device):
    from kernels import _lib

    announce(f"tile pattern copy rowmap {rowmap} slabs {slabs} rows {rows} row bytes {row_bytes}")
    gen = torch.Generator(device=device).manual_seed(rowmap + rows)
    src = torch.randint(0, 256, (slabs, rows, row_bytes), generator=gen, device=device, dtype=torch.uint8)
    dst = torch.zeros_like(src)
    _lib.check(_lib.lib().ema_tile_pattern_copy(src.data_ptr(), None, dst.data_ptr(), slabs, rows, row_bytes, rowmap,
                                                _lib.stream_ptr(device)), "ema_tile_pattern_copy")
    torch.cuda.synchronize()
    assert torch.equal(src, dst)
    if rowmap == 0:  # with a second input: the exclusive or of the two
        other = torch.randint(0, 256, (slabs, rows, row_bytes), generator=gen, device=device, dtype=torch.uint8)
        _lib.check(_lib.lib().ema_tile_pattern_copy(src.data_ptr(), other.data_ptr(), dst.data_ptr(), slabs, rows,
                                                    row_bytes, rowmap, _lib.stream_ptr(device)), "ema_tile_pattern_copy")
        torch.cuda.synchronize()
        assert torch.equal(dst, src ^ other)


def test_tile_pattern_copy_rejects_other_shapes(device):
    from kernels import _lib

    buf = torch.zeros(2 * 128 * 512, device=device, dtype=torch.uint8)
    f = _lib.lib().ema_tile_pattern_copy
    s = _lib.stream_ptr(device)
    assert f(buf.data_ptr(), None, buf.data_ptr(), 2, 100, 512, 0, s) == -2   # rows not a multiple of 128
    assert f(buf.data_ptr(), None, buf.data_ptr(), 2, 128, 500, 2, s) == -2   # row bytes not a multiple of 512
    assert f(None, None, buf.data_ptr(), 2, 128, 512, 1, s) == -1
    assert f(buf.data_ptr(), None, buf.data_ptr(), 2, 128, 512, 9, s) == -5   # no such pattern
    assert f(buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), 2, 128, 512, 1, s) == -5   # two inputs: the kernels' shape only


@pytest.mark.parametrize("two", [False, True], ids=["one_input", "two_inputs"])
def test_stream_copy_copies(two, device):
    from kernels import _lib

    n = 3 * 1024 * 1024 + 4096
    gen = torch.Generator(device=device).manual_seed(7)
    a = torch.randint(0, 256, (n,), generator=gen, device=device, dtype=torch.uint8)
    b = torch.randint(0, 256, (n,), generator=gen, device=device, dtype=torch.uint8) if two else None
    dst = torch.zeros_like(a)
    _lib.check(_lib.lib().ema_stream_copy(a.data_ptr(), None if b is None else b.data_ptr(), dst.data_ptr(), n,
                                          _lib.stream_ptr(device)), "ema_stream_copy")
    torch.cuda.synchronize()
    assert torch.equal(dst, a ^ b if two else a)
