from .dwconv import DWConv
from .dwconv_backward import DWConvBackward
from .dwconv_stats import DWConvStats
from .dwconv_wgrad import DWConvWGRAD
