"""ReLULinearAdd: out = fp16(relu(x) @ weight) + add_other, a 1x1x1 convolution with residual.

Host side of kerops_pointwise_f16 (MFMA kernel); same name, positional arguments, asserts and
result as kerops/ops/linear/relu_linear_add.py:20-52 of the reference.
"""
import torch

from ... import _lib
from ...settings import ConfigurableArg, confexc, configure
from .._common import next_power_of_2, require_cuda

_BUILT = (16, 32, 64, 128)


@confexc(KeyError)
def ilp(in_channels):
    # the reference's table keys (kerops/ops/linear/relu_linear_add.py:10-12) decide which channel
    # counts are served; the value (tiles per program there) has no meaning for the MFMA kernel
    return {16: 1, 32: 1, 64: 1, 128: 1}[in_channels]


@configure(num_warps=4, D_block=32, ILP=lambda x: ilp(x.shape[1]))
def ReLULinearAdd(x, weight, add_other, *, num_warps: ConfigurableArg, D_block: ConfigurableArg,
                  ILP: ConfigurableArg):
    """x (N,Cin,H,W,D), weight [Cin, Cout], add_other (N,Cout,H,W,D); all fp16, channels_last_3d."""
    in_channels = x.shape[1]
    out_channels = add_other.shape[1]

    assert x.ndim == add_other.ndim == 5
    assert list(x.shape[2:]) == list(add_other.shape[2:])
    assert x.shape[0] == add_other.shape[0]
    assert in_channels == next_power_of_2(in_channels)
    assert out_channels == next_power_of_2(out_channels)
    assert list(weight.shape) == [in_channels, out_channels]
    assert x.dtype == weight.dtype == add_other.dtype == torch.float16
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert add_other.is_contiguous(memory_format=torch.channels_last_3d)
    assert out_channels in _BUILT, 'the MFMA kernel is built for 16, 32, 64 or 128 output channels'
    require_cuda(x, weight, add_other)

    weight = weight.contiguous()
    output = torch.empty_like(add_other)
    _lib.call('kerops_pointwise_f16', x.data_ptr(), weight.data_ptr(), add_other.data_ptr(), output.data_ptr(),
              x.numel() // in_channels, in_channels, out_channels, 1, _lib.stream_of(x))
    return output


def ApplyBNReLULinearAdd(x, bn_weight, bn_bias, weight, add_other):
    """ReLULinearAdd(ApplyBNReLU(x, bn_weight, bn_bias), weight, add_other) in one pass, bit-identical to that
    composition (kerops/ops/bnrelu.py:11-42 then kerops/ops/linear/relu_linear_add.py:20-52): the normalised
    activation is formed in registers from the loaded x fragments and never written.  An addition to the
    reference's op set; host side of kerops_bnrelu_pointwise_f16."""
    in_channels = x.shape[1]
    out_channels = add_other.shape[1]

    assert x.ndim == add_other.ndim == 5
    assert list(x.shape[2:]) == list(add_other.shape[2:])
    assert x.shape[0] == add_other.shape[0]
    assert list(weight.shape) == [in_channels, out_channels]
    assert x.dtype == weight.dtype == add_other.dtype == torch.float16
    assert bn_weight.numel() == bn_bias.numel() == in_channels
    assert x.is_contiguous(memory_format=torch.channels_last_3d)
    assert add_other.is_contiguous(memory_format=torch.channels_last_3d)
    assert in_channels in _BUILT and out_channels in _BUILT, 'built for 16, 32, 64 or 128 channels on either side'
    require_cuda(x, bn_weight, bn_bias, weight, add_other)

    weight = weight.contiguous()
    scale = bn_weight.to(torch.float32).contiguous()
    shift = bn_bias.to(torch.float32).contiguous()
    output = torch.empty_like(add_other)
    _lib.call('kerops_bnrelu_pointwise_f16', x.data_ptr(), scale.data_ptr(), shift.data_ptr(), weight.data_ptr(),
              add_other.data_ptr(), output.data_ptr(), x.numel() // in_channels, in_channels, out_channels,
              _lib.stream_of(x))
    return output
