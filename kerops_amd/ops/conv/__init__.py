from .dwconv import DWConv
from .dwconv_wgrad import DWConvWGRAD
