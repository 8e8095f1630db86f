"""Depthwise 3x3x3 convolution ops: forward, weight gradient, and the one-pass variants (both gradients;
forward with the statistics of its output)."""
from .dwconv import DWConv
from .dwconv_backward import DWConvBackward
from .dwconv_stats import DWConvStats
from .dwconv_wgrad import DWConvWGRAD

__all__ = ['DWConv', 'DWConvBackward', 'DWConvStats', 'DWConvWGRAD']
