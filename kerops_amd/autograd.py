"""torch.autograd.Function wrappers around the forward / backward op pairs.

The reference exposes forward and backward as separate plain functions (`Stats` /
`StatsBackward`, ...) and leaves wiring them into autograd to the user; these classes do that
wiring once.  Each `apply` takes and returns exactly what the forward op does.  `DWConvFn` also
provides the input gradient, which the reference lacks (a TODO at kerops/kernels/dw_conv.py:145):
it is the same depthwise kernel run on the upstream gradient with the weight flipped along the
three spatial axes.  When both gradients are wanted the wrapper calls `ops.conv.DWConvBackward`, which
computes them in one pass over x and the upstream gradient (4-8 % faster than the two kernels, the same input
gradient bit for bit).
"""
import torch

from .ops.addition import AddStats, AddStatsBackward
from .ops.avgpool import AvgPoolCeilStats, AvgPoolCeilStatsBackward
from .ops.bnrelu import ApplyBNReLU, ApplyBNReLUBackward
from .ops.conv import DWConv, DWConvBackward, DWConvStats, DWConvWGRAD
from .ops.linear import (ApplyBNReLULinearAdd, LinBReLULinAdd, LinBReLULinBackward, ReLULinearAdd,
                         ReLULinearBackward)
from .ops.stats import Stats, StatsBackward


def _cl3d(t):
    return t.contiguous(memory_format=torch.channels_last_3d)


def _dwconv_grads(x, weight, grad_out, want_x, want_w):
    """Input and weight gradient of DWConv for the upstream gradient grad_out."""
    if want_x and want_w:
        return DWConvBackward(x, grad_out, weight, out_dtype=weight.dtype)
    grad_x = DWConv(grad_out, torch.flip(weight, dims=(0, 1, 2)).contiguous()) if want_x else None
    grad_w = DWConvWGRAD(x, grad_out, out_dtype=weight.dtype) if want_w else None
    return grad_x, grad_w


class DWConvFn(torch.autograd.Function):
    """y = DWConv(x, weight); weight is [3, 3, 3, C] fp16."""

    @staticmethod
    def forward(ctx, x, weight):
        ctx.save_for_backward(x, weight)
        return DWConv(x, weight)

    @staticmethod
    def backward(ctx, grad_out):
        x, weight = ctx.saved_tensors
        return _dwconv_grads(x, weight, _cl3d(grad_out), ctx.needs_input_grad[0], ctx.needs_input_grad[1])


class StatsFn(torch.autograd.Function):
    """(mean, sqmean) = Stats(x)."""

    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        mean, sqmean = Stats(x)
        return mean, sqmean

    @staticmethod
    def backward(ctx, grad_mean, grad_sqmean):
        (x,) = ctx.saved_tensors
        return StatsBackward(x, grad_mean.contiguous(), grad_sqmean.contiguous())


class AddStatsFn(torch.autograd.Function):
    """(z, mean, sqmean) = AddStats(x, y)."""

    @staticmethod
    def forward(ctx, x, y):
        z, mean, sqmean = AddStats(x, y)
        ctx.save_for_backward(z)
        return z, mean, sqmean

    @staticmethod
    def backward(ctx, grad_z, grad_mean, grad_sqmean):
        (z,) = ctx.saved_tensors
        g = AddStatsBackward(_cl3d(grad_z), grad_mean.contiguous(), grad_sqmean.contiguous(), z)
        return g, g


class ApplyBNReLUFn(torch.autograd.Function):
    """y = relu(x * weight[c] + bias[c]); weight, bias fp32 with C elements."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight, bias)
        return ApplyBNReLU(x, weight, bias)

    @staticmethod
    def backward(ctx, grad_out):
        x, weight, bias = ctx.saved_tensors
        dx, dw, db = ApplyBNReLUBackward(x, weight.float(), bias.float(), _cl3d(grad_out))
        return dx, dw.reshape(weight.shape).to(weight.dtype), db.reshape(bias.shape).to(bias.dtype)


class AvgPoolCeilStatsFn(torch.autograd.Function):
    """(pooled, mean, sqmean) = AvgPoolCeilStats(x)."""

    @staticmethod
    def forward(ctx, x):
        pooled, mean, sqmean = AvgPoolCeilStats(x)
        ctx.save_for_backward(pooled)
        ctx.in_shape = tuple(x.shape)
        return pooled, mean, sqmean

    @staticmethod
    def backward(ctx, grad_pooled, grad_mean, grad_sqmean):
        (pooled,) = ctx.saved_tensors
        return AvgPoolCeilStatsBackward(_cl3d(grad_pooled), grad_mean.float().contiguous(),
                                        grad_sqmean.float().contiguous(), _cl3d(pooled), ctx.in_shape)


class ReLULinearAddFn(torch.autograd.Function):
    """out = fp16(relu(x) @ weight) + add_other; weight is [Cin, Cout] fp16."""

    @staticmethod
    def forward(ctx, x, weight, add_other):
        ctx.save_for_backward(x, weight)
        return ReLULinearAdd(x, weight, add_other)

    @staticmethod
    def backward(ctx, grad_out):
        x, weight = ctx.saved_tensors
        grad_out = _cl3d(grad_out)
        grad_x, grad_w = ReLULinearBackward(x, grad_out, weight, out_dtype=weight.dtype)
        return grad_x, grad_w, grad_out  # the residual passes the gradient through


class LinBReLULinAddFn(torch.autograd.Function):
    """out = fp16(relu(fp16(x @ weight_up) + bias) @ weight_down) + add_other."""

    @staticmethod
    def forward(ctx, x, weight_up, weight_down, bias, add_other):
        ctx.save_for_backward(x, weight_up, weight_down, bias)
        return LinBReLULinAdd(x, weight_up, weight_down, bias, add_other)

    @staticmethod
    def backward(ctx, grad_out):
        x, weight_up, weight_down, bias = ctx.saved_tensors
        grad_out = _cl3d(grad_out)
        grad_x, grad_up, grad_down, grad_bias = LinBReLULinBackward(x, grad_out, weight_up, weight_down, bias,
                                                                    out_dtype=weight_up.dtype)
        return grad_x, grad_up, grad_down, grad_bias, grad_out


class DWConvStatsFn(torch.autograd.Function):
    """(y, mean, sqmean) = DWConvStats(x, weight): DWConvFn followed by StatsFn on y in one forward pass.

    Backward: the gradient that reaches y is the upstream gradient of y plus the statistics' contribution
    (AddStatsBackward on y does exactly that sum), then the two convolution gradients as in DWConvFn."""

    @staticmethod
    def forward(ctx, x, weight):
        y, mean, sqmean = DWConvStats(x, weight)
        ctx.save_for_backward(x, weight, y)
        return y, mean, sqmean

    @staticmethod
    def backward(ctx, grad_y, grad_mean, grad_sqmean):
        x, weight, y = ctx.saved_tensors
        g = AddStatsBackward(_cl3d(grad_y), grad_mean.float().contiguous(), grad_sqmean.float().contiguous(), y)
        return _dwconv_grads(x, weight, g, ctx.needs_input_grad[0], ctx.needs_input_grad[1])


class ApplyBNReLULinearAddFn(torch.autograd.Function):
    """out = ReLULinearAdd(ApplyBNReLU(x, bn_weight, bn_bias), weight, add_other) in one forward pass.

    The normalised activation is not kept: backward recomputes it (one ApplyBNReLU pass, the time the forward
    saved) and then runs the two backward ops of the composition."""

    @staticmethod
    def forward(ctx, x, bn_weight, bn_bias, weight, add_other):
        ctx.save_for_backward(x, bn_weight, bn_bias, weight)
        return ApplyBNReLULinearAdd(x, bn_weight, bn_bias, weight, add_other)

    @staticmethod
    def backward(ctx, grad_out):
        x, bn_weight, bn_bias, weight = ctx.saved_tensors
        grad_out = _cl3d(grad_out)
        z = ApplyBNReLU(x, bn_weight, bn_bias)
        grad_z, grad_w = ReLULinearBackward(z, grad_out, weight, out_dtype=weight.dtype)
        dx, dbw, dbb = ApplyBNReLUBackward(x, bn_weight.float(), bn_bias.float(), grad_z)
        return (dx, dbw.reshape(bn_weight.shape).to(bn_weight.dtype), dbb.reshape(bn_bias.shape).to(bn_bias.dtype),
                grad_w, grad_out)
