from .relu_linear_add import ReLULinearAdd
