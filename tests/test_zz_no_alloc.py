"""The entry point that allocates nothing (``hgq_quantize_bwd_static``: the bit-width-gradient slices of the per-column
quantizer backward go to a device array inside the library) against the entry point it is a variant of
(``hgq_quantize_bwd_sliced`` with a caller workspace), through the C ABI: two calls in a row, the second with a smaller
input, results bit for bit; a shape whose slices do not fit the array is refused with a message."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, _lib, dev, rows, M, seed, mode, with_di):
    g = torch.Generator().manual_seed(seed)
    n = rows * M
    x = (torch.randn(n, generator=g) * 3).to(dev)
    dy = torch.randn(n, generator=g).to(dev)
    k = torch.randint(0, 2, (M,), generator=g).float().to(dev)
    i = torch.randint(-1, 4, (M,), generator=g).float().to(dev)
    f = torch.randint(0, 7, (M,), generator=g).float().to(dev)
    need = lib.hgq_quantize_bwd_workspace(n, M, 1)
    assert 0 < need <= _lib.STATIC_SCRATCH_FLOATS, (need, rows, M)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for static in (False, True):
        dx = torch.full((n,), float('nan'), device=dev)
        di = torch.full((M,), float('nan'), device=dev)
        df = torch.full((M,), float('nan'), device=dev)
        dip = _p(di) if with_di else ctypes.c_void_p(0)
        if static:
            rc = lib.hgq_quantize_bwd_static(_p(dy), _p(x), _p(k), _p(i), _p(f), _p(dx), dip, _p(df), n, M, 1, mode, stream)
        else:
            ws = torch.full((need,), float('nan'), device=dev)
            rc = lib.hgq_quantize_bwd_sliced(_p(dy), _p(x), _p(k), _p(i), _p(f), _p(dx), dip, _p(df), _p(ws), n, M, 1, mode, stream)
        assert rc == 0, lib.hgq_last_error()
        torch.cuda.synchronize()
        out.append((dx.cpu(), di.cpu() if with_di else None, df.cpu()))
    (dx0, di0, df0), (dx1, di1, df1) = out
    assert not torch.isnan(dx0).any() and not torch.isnan(df0).any()
    assert torch.equal(dx0, dx1), 'dx differs'
    assert torch.equal(df0, df1), 'dfb differs'
    if with_di:
        assert torch.equal(di0, di1), 'di differs'


def test_static_scratch_entry_point_matches_the_workspace_one():
    from hgq2_amd import _lib

    dev = torch.device('cuda:0')
    lib = _lib.load()
    sat = _lib.mode_bits('RND', 'SAT', training=True)
    wrap = _lib.mode_bits('RND', 'WRAP', training=True)
    # a large call, then a smaller one on the same device: the second finds the first call's slices in the array
    _both(lib, _lib, dev, 16384, 64, 1, sat, True)
    _both(lib, _lib, dev, 700, 24, 2, sat, True)
    _both(lib, _lib, dev, 5000, 7, 3, wrap, False)   # odd width: scalar columns, no integer-bit gradient
    _both(lib, _lib, dev, 16384, 64, 4, wrap, True)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from hgq2_amd import _lib

    dev = torch.device('cuda:0')
    lib = _lib.load()
    rows, M = 8192, 4096
    n = rows * M
    need = lib.hgq_quantize_bwd_workspace(n, M, 1)
    assert need > _lib.STATIC_SCRATCH_FLOATS, need
    z = torch.zeros(16, device=dev)  # never read: the size check comes first
    mode = _lib.mode_bits('RND', 'SAT', training=True)
    rc = lib.hgq_quantize_bwd_static(_p(z), _p(z), _p(z), _p(z), _p(z), _p(z), _p(z), _p(z), n, M, 1, mode, ctypes.c_void_p(0))
    assert rc == _lib.ERR_ARG
    assert b'static scratch' in lib.hgq_last_error()
    # a shape the per-column kernels do not take at all is refused as unsupported
    rc = lib.hgq_quantize_bwd_static(_p(z), _p(z), _p(z), _p(z), _p(z), _p(z), _p(z), _p(z), 16, 16, 1, mode, ctypes.c_void_p(0))
    assert rc == _lib.ERR_UNSUPPORTED
