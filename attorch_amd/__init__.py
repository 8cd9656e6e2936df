"""
MI355X-native implementation of attorch's layer-kernel hot path.

The public names match attorch's (Linear, LayerNorm, RMSNorm, Softmax, LogSoftmax, Softmin,
CrossEntropyLoss, NLLLoss, the p-norm losses, GLU, Conv2d, BatchNorm2d, AvgPool, the activation layers
with fused dropout, Dropout, and their autograd Functions), so
`import attorch_amd as attorch` is a drop-in for that path.  All compute happens in
hand-written gfx950 HIP kernels behind the C ABI declared in include/attorch_hip.h.
"""

from .act_layers import (CELU, ELU, GELU, SELU, ActFuncAutoGrad, Dropout, DropoutAutoGrad, Hardshrink,
                         Hardsigmoid, Hardswish, Hardtanh, LeakyReLU, LogSigmoid, Mish, ReLU, ReLU6,
                         Sigmoid, SiLU, Softplus, Softshrink, Softsign, Tanh, Tanhshrink)
from .batch_norm import BatchNorm1d, BatchNorm2d, BatchNormAutoGrad
from .conv import Conv1d, Conv2d, Conv2dAutoGrad
from .cross_entropy import CrossEntropyLoss, CrossEntropyLossAutoGrad
from .glu import GLU, GLUAutoGrad
from .linear import Linear, LinearAutoGrad
from .nll_loss import NLLLoss, NLLLossAutoGrad
from .p_loss import HuberLoss, L1Loss, MSELoss, PLossAutoGrad, SmoothL1Loss
from .pooling import AvgPool1d, AvgPool2d
from .norms import LayerNorm, LayerNormAutoGrad, RMSNorm, RMSNormAutoGrad
from .softmax import LogSoftmax, Softmax, SoftmaxAutoGrad, Softmin
from .utils import get_output_dtype

__all__ = [
    'ActFuncAutoGrad', 'AvgPool1d', 'AvgPool2d', 'BatchNorm1d', 'BatchNorm2d', 'BatchNormAutoGrad',
    'CELU', 'Conv1d', 'Conv2d', 'Conv2dAutoGrad', 'CrossEntropyLoss', 'CrossEntropyLossAutoGrad',
    'Dropout', 'DropoutAutoGrad', 'ELU', 'GELU', 'GLU', 'GLUAutoGrad', 'Hardshrink', 'Hardsigmoid',
    'Hardswish', 'Hardtanh', 'HuberLoss', 'L1Loss', 'LayerNorm', 'LayerNormAutoGrad', 'LeakyReLU',
    'Linear', 'LinearAutoGrad', 'LogSigmoid', 'LogSoftmax', 'MSELoss', 'Mish', 'NLLLoss',
    'NLLLossAutoGrad', 'PLossAutoGrad', 'RMSNorm', 'RMSNormAutoGrad', 'ReLU', 'ReLU6', 'SELU', 'SiLU',
    'Sigmoid', 'SmoothL1Loss', 'Softmax', 'SoftmaxAutoGrad', 'Softmin', 'Softplus', 'Softshrink',
    'Softsign', 'Tanh', 'Tanhshrink', 'get_output_dtype',
]
