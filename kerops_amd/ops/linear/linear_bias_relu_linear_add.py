"""LinBReLULinAdd: out = fp16(relu(fp16(x @ weight_up) + bias) @ weight_down) + add_other.

Host side of kerops_lin_brelu_lin_add_f16 (MFMA kernel, the hidden activation stays in registers);
same name, positional arguments, asserts and result as
kerops/ops/linear/linear_bias_relu_linear_add.py:22-73 of the reference.
"""
import torch

from ... import _lib
from ...settings import ConfigurableArg, confexc, configure
from .._common import next_power_of_2, require_cuda


@confexc(KeyError)
def dblock(channels):
    # table keys = served channel counts, like kerops/ops/linear/linear_bias_relu_linear_add.py:10-13
    # (the reference serves 16 and 32); the value is the voxel tile of a wavefront
    return {16: 32, 32: 32, 64: 32}[channels]


@confexc(KeyError)
def ilp(channels):
    return {16: 1, 32: 1, 64: 1}[channels]


@configure(num_warps=4, D_block=lambda x: dblock(x.shape[1]), ILP=lambda x: ilp(x.shape[1]))
def LinBReLULinAdd(x, weight_up, weight_down, bias, add_other, *, num_warps: ConfigurableArg,
                   D_block: ConfigurableArg, ILP: ConfigurableArg):
    """x, add_other (N,C,H,W,D); weight_up [C, 2C]; weight_down [2C, C]; bias [2C]; all fp16."""
    in_channels = x.shape[1]
    hidden_channels = 2 * in_channels

    assert x.ndim == add_other.ndim == 5
    assert list(x.shape) == list(add_other.shape)
    assert in_channels == next_power_of_2(in_channels)
    assert list(weight_up.shape) == [in_channels, hidden_channels]
    assert list(weight_down.shape) == [hidden_channels, in_channels]
    assert list(bias.shape) == [hidden_channels]
    assert x.dtype == weight_up.dtype == weight_down.dtype == bias.dtype == add_other.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert add_other.is_contiguous(memory_format=torch.channels_last_3d)
    require_cuda(x, weight_up, weight_down, bias, add_other)

    weight_up, weight_down, bias = weight_up.contiguous(), weight_down.contiguous(), bias.contiguous()
    output = torch.empty_like(x)
    _lib.call('kerops_lin_brelu_lin_add_f16', x.data_ptr(), weight_up.data_ptr(), weight_down.data_ptr(),
              bias.data_ptr(), add_other.data_ptr(), output.data_ptr(), x.numel() // in_channels, in_channels,
              _lib.stream_of(x))
    return output
