"""CPU tests of the C-ABI boundary: the built library loads, exports every symbol the header
declares, validates arguments before touching a device, and the Python ops keep the
reference's host-side contract checks (same exception types, raised before the ABI is
crossed).  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

from kerops_amd import _lib
from kerops_amd.settings import CongiguratorError

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'kerops_hip.h')


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(kerops_[a-z0-9_]+)\s*\(', text)))


def header_version():
    return int(re.search(r'#define\s+KEROPS_HIP_VERSION\s+(\d+)', open(HEADER).read()).group(1))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), f'{name} is declared in include/kerops_hip.h but not exported'
    # and the ctypes table binds exactly the declared set
    assert sorted(_lib.SIGNATURES) == names
    assert lib.kerops_hip_version() == _lib.HEADER_VERSION == header_version()


def test_argument_validation_needs_no_device():
    lib = _lib.load()
    rc = lib.kerops_dwconv_fwd_f16(None, None, None, 1, 4, 4, 4, 8, 0, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_BADARG and 'pointer' in _lib.last_error()
    buf = (ctypes.c_char * 4096)()
    addr = (ctypes.addressof(buf) + 15) & ~15
    rc = lib.kerops_dwconv_fwd_f16(addr, addr, addr, 1, 4, 4, 4, 24, 0, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_UNSUPPORTED_C
    rc = lib.kerops_dwconv_fwd_f16(addr, addr, addr, 1, 4, 4, 4, 64, 5, 7, 0, 2, None)
    assert rc == _lib.KEROPS_E_BADARG and 'no kernel built' in _lib.last_error()
    rc = lib.kerops_dwconv_fwd_f16(addr + 2, addr, addr, 1, 4, 4, 4, 64, 0, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_BADARG
    rc = lib.kerops_dwconv_wgrad_f16(addr, addr, addr, addr, 16, 1, 4, 4, 4, 64, 0, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_WORKSPACE
    # the typed-result variants take fp32 or fp16 only, and check it before anything else
    rc = lib.kerops_dwconv_wgrad_f16_out(addr, addr, addr, 2, addr, 1 << 30, 1, 4, 4, 4, 64, 0, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_BADARG and 'gw_dtype' in _lib.last_error()
    rc = lib.kerops_dwconv_bwd_f16_out(addr, addr, addr, addr, addr, 7, addr, 1 << 30, 1, 4, 4, 4, 64, 0, None)
    assert rc == _lib.KEROPS_E_BADARG and 'gw_dtype' in _lib.last_error()
    rc = lib.kerops_dwconv_wgrad_f16_out(addr, addr, addr, 0, addr, 16, 1, 4, 4, 4, 64, 0, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_WORKSPACE
    rc = lib.kerops_relu_linear_bwd_f16_out(addr, addr, addr, addr, addr, 2, addr, 1 << 30, 64, 32, 32, None)
    assert rc == _lib.KEROPS_E_BADARG and 'dw_dtype' in _lib.last_error()
    rc = lib.kerops_lin_brelu_lin_bwd_f16_out(addr, addr, addr, addr, addr, addr, addr, addr, addr, -1, addr, 1 << 30,
                                              64, 32, None)
    assert rc == _lib.KEROPS_E_BADARG and 'grad_dtype' in _lib.last_error()
    rc = lib.kerops_stats_f16(addr, addr, addr, 64, 1024, addr, 1 << 30, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_UNSUPPORTED_C
    rc = lib.kerops_stats_f16(addr, addr, addr, 64, 12, addr, 1 << 30, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_BADARG
    rc = lib.kerops_quant_u8_window(addr, 7, addr, 16, 1.0, 0, 0, 0, None)
    assert rc == _lib.KEROPS_E_BADARG and 'dtype' in _lib.last_error()
    # launch-shape knobs of the stream kernels: wavefronts per workgroup in {4, 8, 16}, segment in {1, 4, 8}
    for waves, segment, word in [(5, 0, 'waves'), (32, 1, 'waves'), (4, 2, 'segment'), (16, 16, 'segment')]:
        rc = lib.kerops_bnrelu_fwd_f16(addr, addr, addr, addr, 64, 64, 0, waves, segment, None)
        assert rc == _lib.KEROPS_E_BADARG and word in _lib.last_error()
    rc = lib.kerops_stats_f16(addr, addr, addr, 64, 64, addr, 1 << 30, 70000, 0, 0, None)
    assert rc == _lib.KEROPS_E_BADARG and 'blocks' in _lib.last_error()


def test_every_entry_point_rejects_null_pointers_before_touching_the_device():
    # all pointers null, all sizes a plausible 16 / 1.0: every compute entry point must come back with an error
    # code and a message (no launch, no dereference), so that a caller's mistake never reaches the GPU
    lib = _lib.load()
    for name, (res, argtypes) in _lib.SIGNATURES.items():
        if res is not ctypes.c_int or not any(a is ctypes.c_void_p for a in argtypes):
            continue
        args = [None if a is ctypes.c_void_p else (1.0 if a is ctypes.c_float else 16) for a in argtypes]
        rc = getattr(lib, name)(*args)
        assert rc in (_lib.KEROPS_E_BADARG, _lib.KEROPS_E_UNSUPPORTED_C, _lib.KEROPS_E_WORKSPACE), (name, rc)
        assert _lib.last_error(), name


def test_extreme_sizes_never_reach_a_launch():
    # sizes up to INT32_MAX with null pointers, and every workspace query over a grid of extreme extents: the
    # host arithmetic (grid planning, workspace sizes) must neither crash nor report success for a null pointer
    import itertools
    lib = _lib.load()
    for name, (res, argtypes) in _lib.SIGNATURES.items():
        if 'workspace_bytes' in name:
            for vals in itertools.product([1, 8, 64, 350, 2 ** 31 - 1], repeat=min(len(argtypes), 5)):
                n = getattr(lib, name)(*(list(vals) + [0] * (len(argtypes) - len(vals))))
                assert n >= _lib.KEROPS_E_LAUNCH, (name, vals, n)  # a size or one of the error codes
        elif res is ctypes.c_int and any(a is ctypes.c_void_p for a in argtypes):
            for v in (0, 1, 7, 65535, 2 ** 31 - 1):
                args = [None if a is ctypes.c_void_p else (1.0 if a is ctypes.c_float else v) for a in argtypes]
                assert getattr(lib, name)(*args) < 0, (name, v)


def test_workspace_queries():
    lib = _lib.load()
    assert lib.kerops_stats_workspace_bytes(1000, 64, 16) == 16 * 2 * 64 * 4
    assert lib.kerops_stats_workspace_bytes(1000, 64, 0) == 4096 * 2 * 64 * 4  # covers every built-in shape
    assert lib.kerops_stats_workspace_bytes(1000, 24, 16) == _lib.KEROPS_E_BADARG
    n = lib.kerops_dwconv_wgrad_workspace_bytes(1, 350, 350, 128, 64, 0, 0, 0, 0)
    assert n > 0 and n % (27 * 64 * 4) == 0  # one [27][64] fp32 partial per workgroup
    assert lib.kerops_dwconv_wgrad_workspace_bytes(1, 8, 8, 8, 24, 0, 0, 0, 0) == _lib.KEROPS_E_UNSUPPORTED_C
    assert lib.kerops_avgpool_ceil_stats_workspace_bytes(1, 7, 7, 7, 8, 4) == 4 * 2 * 8 * 4
    assert lib.kerops_absmax_workspace_bytes(10) == 40


def test_wgrad_launch_knobs_are_checked_before_any_division():
    # a zero or negative patch extent beside non-zero knobs used to divide by zero on the host
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    addr = (ctypes.addressof(buf) + 15) & ~15
    for tw, td, cl in [(0, 8, 16), (8, 0, 16), (0, 8, 0), (-8, 8, 16), (8, -8, 16), (8, 8, -16), (8, 8, 0),
                       (2 ** 31 - 1, 8, 16)]:
        assert lib.kerops_dwconv_wgrad_workspace_bytes(1, 16, 16, 16, 64, tw, td, 0, cl) == _lib.KEROPS_E_BADARG
        assert 'no kernel built' in _lib.last_error()
        rc = lib.kerops_dwconv_wgrad_f16(addr, addr, addr, addr, 1 << 40, 1, 16, 16, 16, 64, tw, td, 0, cl, None)
        assert rc == _lib.KEROPS_E_BADARG
    # the fused block checks plane and volume limits like the other convolution entry points
    assert lib.kerops_dwsep_block_workspace_bytes(1, 4, 2 ** 20, 2 ** 20, 64, 128) == _lib.KEROPS_E_BADARG
    assert lib.kerops_dwsep_block_workspace_bytes(2 ** 31 - 1, 2 ** 31 - 1, 256, 256, 64, 128) == _lib.KEROPS_E_BADARG


def test_split_of_the_h_march():
    # workgroup counts of the built-in launch shapes, read back from the workspace sizes (one partial per
    # workgroup).  The matrix-core convolution kernels use the balanced split by default: never more workgroups than
    # the GPU holds at once (512 of 512 threads, 1024 of 256), all of them busy at the large shapes.  Uniform chunks
    # on request: patches x chunks.
    lib = _lib.load()

    def wgrad_blocks(n, h, w, d, c, h_chunk=0):
        return lib.kerops_dwconv_wgrad_workspace_bytes(n, h, w, d, c, 0, 0, h_chunk, 0) // (27 * min(c, 64) * 4)

    def bwd_blocks(n, h, w, d, c, h_chunk=0):
        return lib.kerops_dwconv_bwd_workspace_bytes(n, h, w, d, c, h_chunk) // (27 * min(c, 64) * 4)

    def stats_blocks(n, h, w, d, c):
        return lib.kerops_dwconv_stats_workspace_bytes(n, h, w, d, c) // (2 * min(c, 64) * 4)

    for blocks in (wgrad_blocks, bwd_blocks, stats_blocks):
        assert blocks(1, 350, 350, 128, 64) == 512   # 8 groups of 64 (weight gradient: 4 rows of 16 patches)
        assert blocks(1, 350, 350, 128, 128) == 512  # the same patches in 2 slabs
        assert blocks(1, 128, 128, 128, 64) == 512
    assert wgrad_blocks(1, 350, 350, 128, 8) in range(480, 513)  # 512-thread workgroups at every channel count
    assert wgrad_blocks(1, 1, 8, 8, 8) == 1 and stats_blocks(1, 1, 8, 8, 64) == 1 and bwd_blocks(1, 1, 8, 8, 64) == 1
    assert wgrad_blocks(1, 350, 350, 128, 64, 175) == 1408 and bwd_blocks(1, 350, 350, 128, 64, 175) == 1408  # 8x8 patches
    assert wgrad_blocks(1, 350, 350, 128, 64, -32) == 512 and bwd_blocks(1, 350, 350, 128, 64, -32) == 512
    # a group that is not a multiple of the two slabs of 128 channels is refused
    assert lib.kerops_dwconv_wgrad_workspace_bytes(1, 350, 350, 128, 128, 0, 0, -3, 0) == _lib.KEROPS_E_BADARG
    assert lib.kerops_dwconv_bwd_workspace_bytes(1, 350, 350, 128, 128, -3) == _lib.KEROPS_E_BADARG


def cl3d(*shape, dtype=torch.float16):
    return torch.zeros(*shape, dtype=dtype).to(memory_format=torch.channels_last_3d)


def test_ops_keep_reference_contract_checks():
    from kerops_amd.ops.avgpool import AvgPoolCeilStats
    from kerops_amd.ops.bnrelu import ApplyBNReLU, ApplyBNReLUBackward
    from kerops_amd.ops.conv import DWConv, DWConvWGRAD
    from kerops_amd.ops.stats import Stats

    x = cl3d(1, 8, 4, 4, 4)
    w = torch.zeros(3, 3, 3, 8, dtype=torch.float16)
    with pytest.raises(AssertionError):  # not channels_last_3d
        DWConv(torch.zeros(1, 8, 4, 4, 4, dtype=torch.float16), w)
    with pytest.raises(AssertionError):  # dtype
        DWConv(x.float(), w.float())
    with pytest.raises(AssertionError):  # weight layout
        DWConv(x, torch.zeros(8, 1, 3, 3, 3, dtype=torch.float16))
    with pytest.raises(CongiguratorError):  # channel count with no launch table entry
        DWConv(cl3d(1, 4, 4, 4, 4), torch.zeros(3, 3, 3, 4, dtype=torch.float16))
    with pytest.raises(CongiguratorError):
        DWConvWGRAD(cl3d(1, 256, 2, 2, 2), cl3d(1, 256, 2, 2, 2))
    with pytest.raises(KeyError):
        DWConv(x, w, ACCTYPE='bfloat16')
    with pytest.raises(AssertionError):
        DWConvWGRAD(x, cl3d(1, 8, 4, 4, 5))
    with pytest.raises(AssertionError):  # non power of two
        Stats(cl3d(1, 6, 4, 4, 4))
    with pytest.raises(AssertionError):
        ApplyBNReLU(x, torch.zeros(4), torch.zeros(8))
    with pytest.raises(AssertionError):  # fp32 weight / bias required by the backward
        ApplyBNReLUBackward(x, torch.zeros(8, dtype=torch.float64), torch.zeros(8, dtype=torch.float64), x)
    with pytest.raises(AssertionError):  # D*C above the reference's row limit
        AvgPoolCeilStats(cl3d(1, 128, 2, 2, 512))


def test_no_cpu_fallback():
    from kerops_amd.ops.conv import DWConv
    from kerops_amd.ops.quantization import QuantUint8Window
    from kerops_amd.ops.stats import Stats

    x = cl3d(1, 8, 4, 4, 4)
    with pytest.raises(RuntimeError, match='no CPU path'):
        DWConv(x, torch.zeros(3, 3, 3, 8, dtype=torch.float16))
    with pytest.raises(RuntimeError, match='no CPU path'):
        Stats(x)
    with pytest.raises(RuntimeError, match='no CPU path'):
        QuantUint8Window(x, 1.0)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setattr(_lib, 'LIB_PATH', os.path.join(ROOT, 'kerops_amd', '_C', 'does_not_exist.so'))
    with pytest.raises(RuntimeError, match='no fallback'):
        _lib.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, 'kerops_amd')
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(('.py', '.hip', '.hpp', '.h', '.cpp')):
                text = open(os.path.join(dirpath, f)).read()
                assert 'import oracle' not in text and 'from oracle' not in text and 'oracle/' not in text, f
