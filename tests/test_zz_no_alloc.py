"""GPU test of kerops_dwconv_wgrad_noalloc_f16, the weight gradient for callers that cannot allocate: called through
the C ABI, compared bit for bit with kerops_dwconv_wgrad_f16 (caller's workspace) on two calls in a row, the second
with a smaller input, so that partials left in the shared device array by the first call cannot leak into the
second result."""
import pytest
import torch

import oracle
from conftest import cpu_gen, rand_cl3d
from kerops_amd import _lib

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def wgrad_workspace(x, g):
    n, c, h, w, d = x.shape
    nbytes = _lib.query('kerops_dwconv_wgrad_workspace_bytes', n, h, w, d, c, 0, 0, 0, 0)
    ws = torch.full((nbytes,), 0x7f, dtype=torch.uint8, device=x.device)  # never zeroed by the library
    gw = torch.empty(3, 3, 3, c, dtype=torch.float32, device=x.device)
    _lib.call('kerops_dwconv_wgrad_f16', x.data_ptr(), g.data_ptr(), gw.data_ptr(), ws.data_ptr(), nbytes, n, h, w, d,
              c, 0, 0, 0, 0, _lib.stream_of(x))
    return gw


def wgrad_noalloc(x, g, gw):
    n, c, h, w, d = x.shape
    _lib.call('kerops_dwconv_wgrad_noalloc_f16', x.data_ptr(), g.data_ptr(), gw.data_ptr(), n, h, w, d, c,
              _lib.stream_of(x))


@pytest.mark.parametrize('c', [64, 8, 128, 32, 16])
def test_noalloc_wgrad_matches_workspace_entry_point_twice(c):
    gen = cpu_gen(1000 + c)
    shapes = [(2, c, 19, 40, 33), (1, c, 5, 9, 12)]  # the second call is the smaller one
    tensors = [(rand_cl3d(gen, *s).to(DEV), rand_cl3d(gen, *s).to(DEV)) for s in shapes]
    outs = [torch.full((3, 3, 3, c), float('nan'), dtype=torch.float32, device=DEV) for _ in shapes]
    refs = [wgrad_workspace(x, g) for x, g in tensors]
    # one call first: the entry point looks up its device array on its first call on a device
    wgrad_noalloc(*tensors[1], outs[1])
    torch.cuda.synchronize()
    outs[1].fill_(float('nan'))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]  # the driver's view: would also see a hipMalloc inside the library
    for (x, g), out in zip(tensors, outs):  # back to back on one stream, no allocation in between
        wgrad_noalloc(x, g, out)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    for (x, g), out, ref in zip(tensors, outs, refs):
        assert torch.equal(out.view(torch.int32), ref.view(torch.int32))  # same kernels, same order: same bits
        gw64 = oracle.dwconv_wgrad(x.cpu(), g.cpu())
        assert ((out.cpu().double() - gw64).norm() / gw64.norm()).item() < 1e-5


def test_noalloc_wgrad_full_shape_then_small():
    """(1,64,350,350,128) needs the largest partial buffer of the built-in shapes; a small call right after it."""
    gen = torch.Generator(DEV).manual_seed(322)
    x = torch.randn(1, 350, 350, 128, 64, device=DEV, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
    g = torch.randn(1, 350, 350, 128, 64, device=DEV, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
    xs = x[:, :, :7, :11, :13].contiguous(memory_format=torch.channels_last_3d)
    gs = g[:, :, :7, :11, :13].contiguous(memory_format=torch.channels_last_3d)
    ref_big, ref_small = wgrad_workspace(x, g), wgrad_workspace(xs, gs)
    big = torch.empty_like(ref_big)
    small = torch.empty_like(ref_small)
    wgrad_noalloc(x, g, big)
    wgrad_noalloc(xs, gs, small)
    torch.cuda.synchronize()
    assert torch.equal(big.view(torch.int32), ref_big.view(torch.int32))
    assert torch.equal(small.view(torch.int32), ref_small.view(torch.int32))


def test_noalloc_wgrad_argument_checks():
    x = torch.zeros(16, dtype=torch.float16, device=DEV)
    gw = torch.zeros(27 * 64, dtype=torch.float32, device=DEV)
    lib = _lib.load()
    s = _lib.stream_of(x)
    assert lib.kerops_dwconv_wgrad_noalloc_f16(None, x.data_ptr(), gw.data_ptr(), 1, 4, 4, 4, 64, s) == \
        _lib.KEROPS_E_BADARG
    assert lib.kerops_dwconv_wgrad_noalloc_f16(x.data_ptr(), x.data_ptr(), gw.data_ptr(), 1, 4, 4, 4, 24, s) == \
        _lib.KEROPS_E_UNSUPPORTED_C
    assert lib.kerops_dwconv_wgrad_noalloc_f16(x.data_ptr(), x.data_ptr(), gw.data_ptr(), 1, 0, 4, 4, 64, s) == \
        _lib.KEROPS_E_BADARG
