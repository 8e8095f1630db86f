"""Pointwise (1x1x1) ops on the matrix cores: the reference's four linear ops plus the one-pass
batch-norm + ReLU + pointwise + residual op."""
from .linear_bias_relu_linear_add import LinBReLULinAdd
from .linear_bias_relu_linear_backward import LinBReLULinBackward
from .relu_linear_add import ApplyBNReLULinearAdd, ReLULinearAdd
from .relu_linear_backward import ReLULinearBackward

__all__ = ['ApplyBNReLULinearAdd', 'LinBReLULinAdd', 'LinBReLULinBackward', 'ReLULinearAdd', 'ReLULinearBackward']
