from .relu_linear_add import ReLULinearAdd
from .relu_linear_backward import ReLULinearBackward
