"""ReLULinearBackward: gradients of out = relu(x) @ weight with respect to x and weight.

Host side of kerops_relu_linear_bwd_f16 (MFMA kernel, one pass over x and grad); same name,
positional arguments, asserts and result tuple as kerops/ops/linear/relu_linear_backward.py:20-72
of the reference.  The reference stores fp16 partial weight gradients and returns their fp16 sum;
here the sum is fp32 end to end and is cast once to `out_dtype` (fp16 by default).
"""
import torch

from ... import _lib
from ...settings import ConfigurableArg, confexc, configure
from .._common import next_power_of_2, require_cuda

_BUILT = (16, 32, 64, 128)


@confexc(KeyError)
def warps(in_channels):
    # the reference's table keys (kerops/ops/linear/relu_linear_backward.py:10-12) decide which channel
    # counts are served; the gfx950 kernel always runs four wavefronts per workgroup
    return {16: 4, 32: 4, 64: 4, 128: 4}[in_channels]


@confexc(KeyError)
def dblock(in_channels):
    # voxels per tile of the gfx950 kernel
    return {16: 64, 32: 64, 64: 64, 128: 64}[in_channels]


@configure(
    num_warps=lambda x: warps(x.shape[1]),
    D_block=lambda x: dblock(x.shape[1]),
    ILP=1,
    out_dtype=torch.float16,
)
def ReLULinearBackward(
    x,
    grad,
    weight,
    *,
    num_warps: ConfigurableArg,
    D_block: ConfigurableArg,
    ILP: ConfigurableArg,
    out_dtype: ConfigurableArg,
):
    """x (N,Cin,H,W,D), grad (N,Cout,H,W,D), weight [Cin, Cout]; fp16, channels_last_3d.
    Returns (x_grad like x, weight_grad [Cin, Cout])."""
    in_channels = x.shape[1]
    out_channels = grad.shape[1]

    assert grad.ndim == x.ndim == 5
    assert list(grad.shape[2:]) == list(x.shape[2:])
    assert grad.shape[0] == x.shape[0]
    assert in_channels == next_power_of_2(in_channels)
    assert out_channels == next_power_of_2(out_channels)
    assert list(weight.shape) == [in_channels, out_channels]
    assert x.dtype == grad.dtype == weight.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert grad.is_contiguous(memory_format=torch.channels_last_3d)
    assert out_channels in _BUILT, 'the MFMA kernel is built for 16, 32, 64 or 128 output channels'
    # num_warps, D_block and ILP are accepted with any positive value, as in the reference
    # (kerops/ops/linear/relu_linear_backward.py:20-24), and not used: the gfx950 kernel always runs 4
    # wavefronts on tiles of 64 voxels
    assert int(num_warps) > 0 and int(D_block) > 0 and int(ILP) > 0
    require_cuda(x, grad, weight)

    weight = weight.contiguous()
    V = grad.numel() // out_channels
    ws_bytes = _lib.query('kerops_relu_linear_bwd_workspace_bytes', V, in_channels, out_channels)
    ws = _lib.workspace(ws_bytes, x.device)
    x_grad = torch.empty_like(x)
    # fp32 and fp16 results are written by the library's reduction kernel; any other type is cast from fp32
    direct = out_dtype in _lib.GW_DTYPES
    weight_grad = torch.empty([in_channels, out_channels], dtype=out_dtype if direct else torch.float32,
                              device=x.device)
    _lib.call('kerops_relu_linear_bwd_f16_out', x.data_ptr(), grad.data_ptr(), weight.data_ptr(), x_grad.data_ptr(),
              weight_grad.data_ptr(), _lib.GW_DTYPES[weight_grad.dtype], ws.data_ptr(), ws_bytes, V, in_channels,
              out_channels, _lib.stream_of(x))
    return x_grad, (weight_grad if direct else weight_grad.to(out_dtype))
