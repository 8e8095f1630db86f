"""LinBReLULinBackward: gradients of out = relu(x @ weight_up + bias) @ weight_down.

Host side of kerops_lin_brelu_lin_bwd_f16 (MFMA kernel, one pass over x and grad); same name,
positional arguments, asserts and result tuple as
kerops/ops/linear/linear_bias_relu_linear_backward.py:20-73 of the reference.  The reference stores
fp16 partial gradients and returns their fp16 sums; here the sums are fp32 end to end and are cast once
to `out_dtype` (fp16 by default).
"""
import torch

from ... import _lib
from ...settings import ConfigurableArg, confexc, configure
from .._common import next_power_of_2, require_cuda


@confexc(KeyError)
def dblock(channels):
    # table keys = served channel counts (the reference serves 16 and 32,
    # kerops/ops/linear/linear_bias_relu_linear_backward.py:10-12); the value is the voxel tile of a workgroup
    return {16: 64, 32: 64, 64: 64}[channels]


@configure(num_warps=4, D_block=lambda x: dblock(x.shape[1]), ILP=1, out_dtype=torch.float16)
def LinBReLULinBackward(x, grad, weight_up, weight_down, bias, *, num_warps: ConfigurableArg,
                        D_block: ConfigurableArg, ILP: ConfigurableArg, out_dtype: ConfigurableArg):
    """Returns (x_grad like x, weight_up_grad [C,2C], weight_down_grad [2C,C], bias_grad [2C])."""
    in_channels = x.shape[1]
    hidden_channels = 2 * in_channels

    assert grad.ndim == x.ndim == 5
    assert list(x.shape) == list(grad.shape)
    assert in_channels == next_power_of_2(in_channels)
    assert list(weight_up.shape) == [in_channels, hidden_channels]
    assert list(weight_down.shape) == [hidden_channels, in_channels]
    assert list(bias.shape) == [hidden_channels]
    assert x.dtype == grad.dtype == weight_up.dtype == weight_down.dtype == bias.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert grad.is_contiguous(memory_format=torch.channels_last_3d)
    require_cuda(x, grad, weight_up, weight_down, bias)

    weight_up, weight_down, bias = weight_up.contiguous(), weight_down.contiguous(), bias.contiguous()
    V = grad.numel() // in_channels
    ws_bytes = _lib.query('kerops_lin_brelu_lin_bwd_workspace_bytes', V, in_channels)
    ws = _lib.workspace(ws_bytes, x.device)
    x_grad = torch.empty_like(x)
    # fp32 and fp16 results are written by the library's reduction kernel; any other type is cast from fp32
    direct = out_dtype in _lib.GW_DTYPES
    res = dict(dtype=out_dtype if direct else torch.float32, device=x.device)
    up_grad = torch.empty([in_channels, hidden_channels], **res)
    down_grad = torch.empty([hidden_channels, in_channels], **res)
    bias_grad = torch.empty([hidden_channels], **res)
    _lib.call('kerops_lin_brelu_lin_bwd_f16_out', x.data_ptr(), grad.data_ptr(), weight_up.data_ptr(),
              weight_down.data_ptr(), bias.data_ptr(), x_grad.data_ptr(), up_grad.data_ptr(), down_grad.data_ptr(),
              bias_grad.data_ptr(), _lib.GW_DTYPES[res['dtype']], ws.data_ptr(), ws_bytes, V, in_channels,
              _lib.stream_of(x))
    if not direct:
        up_grad, down_grad, bias_grad = up_grad.to(out_dtype), down_grad.to(out_dtype), bias_grad.to(out_dtype)
    return x_grad, up_grad, down_grad, bias_grad
