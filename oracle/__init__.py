"""Python face of the CPU oracle (oracle/kerops_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  Nothing under kerops_amd/ may import it.

Every function takes and returns CPU torch tensors with the same contracts as
the op it checks: activations are (N, C, H, W, D) fp16 in channels_last_3d,
depthwise weights are [3, 3, 3, C] fp16, per-channel vectors are [C].
"""
import ctypes
import os

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, '_build', 'liboracle.so')
_lib = None

_i32 = ctypes.c_int
_i64 = ctypes.c_int64
_f32 = ctypes.c_float
_ptr = ctypes.c_void_p


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from .build_oracle import build

            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_absmax_f16.restype = ctypes.c_float
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads():
    return int(lib().oracle_num_threads())


def _p(t):
    return _ptr(t.data_ptr()) if t is not None else _ptr(0)


def _cl(x):
    """(N,C,H,W,D) tensor -> dense [N,H,W,D,C] tensor sharing or copying memory."""
    assert x.ndim == 5 and x.device.type == 'cpu'
    return x.permute(0, 2, 3, 4, 1).contiguous()


def _from_cl(y):
    """dense [N,H,W,D,C] -> (N,C,H,W,D) view, which is channels_last_3d contiguous."""
    return y.permute(0, 4, 1, 2, 3)


def h2f(x):
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=torch.float32)
    lib().oracle_h2f_array(_p(x), _p(out), _i64(x.numel()))
    return out


def f2h(x):
    x = x.contiguous().float()
    out = torch.empty(x.shape, dtype=torch.float16)
    lib().oracle_f2h_array(_p(x), _p(out), _i64(x.numel()))
    return out


def dwconv_fwd(x, weight, wide=True, return_fp32=False):
    assert x.dtype == weight.dtype == torch.float16
    n, c, h, w, d = x.shape
    assert list(weight.shape) == [3, 3, 3, c]
    xc, wc = _cl(x), weight.contiguous()
    y16 = torch.empty_like(xc)
    y32 = torch.empty(xc.shape, dtype=torch.float32) if return_fp32 else None
    lib().oracle_dwconv_fwd(_p(xc), _p(wc), _p(y32), _p(y16), _i32(n), _i32(h), _i32(w), _i32(d), _i32(c),
                            _i32(1 if wide else 0))
    if return_fp32:
        return _from_cl(y16), _from_cl(y32)
    return _from_cl(y16)


def dwconv_wgrad(x, grad):
    """Returns the fp64 weight gradient, shape [3,3,3,C]."""
    assert x.dtype == grad.dtype == torch.float16 and x.shape == grad.shape
    n, c, h, w, d = x.shape
    xc, gc = _cl(x), _cl(grad)
    gw = torch.empty(3, 3, 3, c, dtype=torch.float64)
    lib().oracle_dwconv_wgrad(_p(xc), _p(gc), _p(gw), _i32(n), _i32(h), _i32(w), _i32(d), _i32(c))
    return gw


def stats(x):
    """Returns (mean, sqmean) in fp64."""
    assert x.dtype == torch.float16
    c = x.shape[1]
    xc = _cl(x)
    mean = torch.empty(c, dtype=torch.float64)
    sq = torch.empty(c, dtype=torch.float64)
    lib().oracle_stats(_p(xc), _p(mean), _p(sq), _i64(xc.numel() // c), _i32(c))
    return mean, sq


def stats_bwd(x, mean_grad, sqmean_grad):
    c = x.shape[1]
    xc = _cl(x)
    dx = torch.empty_like(xc)
    mg, sg = mean_grad.float().contiguous(), sqmean_grad.float().contiguous()
    lib().oracle_stats_bwd(_p(xc), _p(mg), _p(sg), _p(dx), _i64(xc.numel() // c), _i32(c))
    return _from_cl(dx)


def add_stats(x, y):
    c = x.shape[1]
    xc, yc = _cl(x), _cl(y)
    z = torch.empty_like(xc)
    mean = torch.empty(c, dtype=torch.float64)
    sq = torch.empty(c, dtype=torch.float64)
    lib().oracle_add_stats(_p(xc), _p(yc), _p(z), _p(mean), _p(sq), _i64(xc.numel() // c), _i32(c))
    return _from_cl(z), mean, sq


def add_stats_bwd(add_grad, mean_grad, sqmean_grad, add_result):
    c = add_grad.shape[1]
    gc, rc = _cl(add_grad), _cl(add_result)
    out = torch.empty_like(gc)
    mg, sg = mean_grad.float().contiguous(), sqmean_grad.float().contiguous()
    lib().oracle_add_stats_bwd(_p(gc), _p(mg), _p(sg), _p(rc), _p(out), _i64(gc.numel() // c), _i32(c))
    return _from_cl(out)


def bnrelu_fwd(x, weight, bias):
    c = x.shape[1]
    xc = _cl(x)
    y = torch.empty_like(xc)
    wv, bv = weight.float().reshape(-1).contiguous(), bias.float().reshape(-1).contiguous()
    lib().oracle_bnrelu_fwd(_p(xc), _p(wv), _p(bv), _p(y), _i64(xc.numel() // c), _i32(c))
    return _from_cl(y)


def bnrelu_bwd(x, weight, bias, grad):
    """Returns (dx fp16, dW fp64 [C], dB fp64 [C])."""
    c = x.shape[1]
    xc, gc = _cl(x), _cl(grad)
    dx = torch.empty_like(xc)
    wv, bv = weight.float().reshape(-1).contiguous(), bias.float().reshape(-1).contiguous()
    dw = torch.empty(c, dtype=torch.float64)
    db = torch.empty(c, dtype=torch.float64)
    lib().oracle_bnrelu_bwd(_p(xc), _p(wv), _p(bv), _p(gc), _p(dx), _p(dw), _p(db), _i64(xc.numel() // c), _i32(c))
    return _from_cl(dx), dw, db


def avgpool_ceil_stats(x, return_fp32=False):
    """Returns (pooled fp16, mean fp64, sqmean fp64) [+ pooled fp32]."""
    n, c, h, w, d = x.shape
    xc = _cl(x)
    ho, wo, do = (h + 1) // 2, (w + 1) // 2, (d + 1) // 2
    y16 = torch.empty(n, ho, wo, do, c, dtype=torch.float16)
    y32 = torch.empty(n, ho, wo, do, c, dtype=torch.float32)
    mean = torch.empty(c, dtype=torch.float64)
    sq = torch.empty(c, dtype=torch.float64)
    lib().oracle_avgpool_ceil_stats(_p(xc), _p(y32), _p(y16), _p(mean), _p(sq), _i32(n), _i32(h), _i32(w), _i32(d),
                                    _i32(c))
    if return_fp32:
        return _from_cl(y16), mean, sq, _from_cl(y32)
    return _from_cl(y16), mean, sq


def avgpool_ceil_stats_bwd(inpgrad, meangrad, sqmeangrad, output, outgrad_shape):
    n, c, h, w, d = outgrad_shape
    gc, oc = _cl(inpgrad), _cl(output)
    dx = torch.zeros(n, h, w, d, c, dtype=torch.float16)
    mg, sg = meangrad.float().contiguous(), sqmeangrad.float().contiguous()
    lib().oracle_avgpool_ceil_stats_bwd(_p(gc), _p(mg), _p(sg), _p(oc), _p(dx), _i32(n), _i32(h), _i32(w), _i32(d),
                                        _i32(c))
    return _from_cl(dx)


def quant_u8_window(x, window):
    xc = x.contiguous()
    q = torch.empty(xc.shape, dtype=torch.uint8)
    if xc.dtype == torch.float16:
        lib().oracle_quant_u8_window_f16(_p(xc), _p(q), _i64(xc.numel()), _f32(window))
    elif xc.dtype in (torch.float32, torch.bfloat16):
        xc = xc.float()  # bf16 -> fp32 is exact: the same first step as the kernel's
        lib().oracle_quant_u8_window_f32(_p(xc), _p(q), _i64(xc.numel()), _f32(window))
    else:
        raise TypeError(xc.dtype)
    return q


def dequant_u8_window(q, init_dtype, window):
    qc = q.contiguous()
    if init_dtype == torch.bfloat16:  # the fp32 value, rounded once to nearest-even by torch's conversion
        return dequant_u8_window(q, torch.float32, window).to(torch.bfloat16)
    out = torch.empty(qc.shape, dtype=init_dtype)
    if init_dtype == torch.float16:
        lib().oracle_dequant_u8_window_f16(_p(qc), _p(out), _i64(qc.numel()), _f32(window))
    elif init_dtype == torch.float32:
        lib().oracle_dequant_u8_window_f32(_p(qc), _p(out), _i64(qc.numel()), _f32(window))
    else:
        raise TypeError(init_dtype)
    return out


def absmax_f16(y):
    yc = y.contiguous()
    return float(lib().oracle_absmax_f16(_p(yc), _i64(yc.numel())))


def quant_i8_sym(y, absmax):
    yc = y.contiguous()
    q = torch.empty(yc.shape, dtype=torch.int8)
    lib().oracle_quant_i8_sym_f16(_p(yc), _p(q), _i64(yc.numel()), _f32(absmax))
    return q


def pointwise(x, weight, add=None, relu_in=False):
    """x (N,Cin,H,W,D) fp16 cl3d, weight [Cin,Cout] fp16 -> (N,Cout,H,W,D) fp16."""
    n, cin, h, w, d = x.shape
    cout = weight.shape[1]
    xc = _cl(x)
    wc = weight.contiguous()
    ac = _cl(add) if add is not None else None
    out = torch.empty(n, h, w, d, cout, dtype=torch.float16)
    lib().oracle_pointwise(_p(xc), _p(wc), _p(ac), _p(out), _i64(n * h * w * d), _i32(cin), _i32(cout),
                           _i32(1 if relu_in else 0))
    return _from_cl(out)


def relu_linear_bwd(x, grad, weight):
    """x (N,Cin,H,W,D), grad (N,Cout,H,W,D) fp16 cl3d, weight [Cin,Cout] fp16 -> (dx fp16 like x, dW fp64 [Cin,Cout])."""
    n, cin, h, w, d = x.shape
    cout = weight.shape[1]
    xc, gc = _cl(x), _cl(grad)
    dx = torch.empty_like(xc)
    dw = torch.empty(cin, cout, dtype=torch.float64)
    lib().oracle_relu_linear_bwd(_p(xc), _p(gc), _p(weight.contiguous()), _p(dx), _p(dw), _i64(n * h * w * d),
                                 _i32(cin), _i32(cout))
    return _from_cl(dx), dw


def lin_brelu_lin_add(x, weight_up, weight_down, bias, add, return_hidden=False):
    """x, add (N,C,H,W,D) fp16 cl3d; weight_up [C,2C], weight_down [2C,C], bias [2C] fp16 -> (N,C,H,W,D) fp16."""
    n, c, h, w, d = x.shape
    xc, ac = _cl(x), _cl(add)
    out = torch.empty_like(xc)
    hid = torch.empty(n, h, w, d, 2 * c, dtype=torch.float16)
    lib().oracle_lin_brelu_lin_add(_p(xc), _p(weight_up.contiguous()), _p(weight_down.contiguous()),
                                   _p(bias.contiguous()), _p(ac), _p(hid), _p(out), _i64(n * h * w * d), _i32(c))
    if return_hidden:
        return _from_cl(out), _from_cl(hid)
    return _from_cl(out)


def lin_brelu_lin_bwd(x, grad, weight_up, weight_down, bias):
    """-> (dx fp16 like x, dWup fp64 [C,2C], dWdown fp64 [2C,C], dbias fp64 [2C])."""
    n, c, h, w, d = x.shape
    xc, gc = _cl(x), _cl(grad)
    dx = torch.empty_like(xc)
    dup = torch.empty(c, 2 * c, dtype=torch.float64)
    ddn = torch.empty(2 * c, c, dtype=torch.float64)
    db = torch.empty(2 * c, dtype=torch.float64)
    lib().oracle_lin_brelu_lin_bwd(_p(xc), _p(gc), _p(weight_up.contiguous()), _p(weight_down.contiguous()),
                                   _p(bias.contiguous()), _p(dx), _p(dup), _p(ddn), _p(db), _i64(n * h * w * d),
                                   _i32(c))
    return _from_cl(dx), dup, ddn, db


def dwsep_block(x, dw_weight, scale, shift, pw_weight, return_mid=False):
    n, cin, h, w, d = x.shape
    cout = pw_weight.shape[1]
    xc = _cl(x)
    t = torch.empty_like(xc)
    y = torch.empty(n, h, w, d, cout, dtype=torch.float16)
    sc, sh = scale.float().contiguous(), shift.float().contiguous()
    lib().oracle_dwsep_block(_p(xc), _p(dw_weight.contiguous()), _p(sc), _p(sh), _p(pw_weight.contiguous()), _p(t),
                             _p(y), _i32(n), _i32(h), _i32(w), _i32(d), _i32(cin), _i32(cout))
    if return_mid:
        return _from_cl(y), _from_cl(t)
    return _from_cl(y)


def np_quant_u8_window(x_f32, window):
    """Independent numpy restatement of the window quantiser, used to pin the C one."""
    w = np.float32(window)
    t = np.minimum(np.maximum(x_f32.astype(np.float32), -w), w)
    t = (t + w).astype(np.float32)
    t = (t / np.float32(np.float32(2.0) * w)).astype(np.float32)
    t = (t * np.float32(255.0)).astype(np.float32)
    return t.astype(np.uint8)
