"""
MI355X-native implementation of attorch's layer-kernel hot path.

The public names match attorch's (Linear, LayerNorm, RMSNorm, Softmax, LogSoftmax, Softmin,
CrossEntropyLoss, NLLLoss, Conv2d, BatchNorm2d, the activation layers with fused dropout, Dropout, and
their autograd Functions), so
`import attorch_amd as attorch` is a drop-in for that path.  All compute happens in
hand-written gfx950 HIP kernels behind the C ABI declared in include/attorch_hip.h.
"""

from .act_layers import (CELU, ELU, GELU, SELU, ActFuncAutoGrad, Dropout, DropoutAutoGrad, Hardshrink,
                         Hardsigmoid, Hardswish, Hardtanh, LeakyReLU, LogSigmoid, Mish, ReLU, ReLU6,
                         Sigmoid, SiLU, Softplus, Softshrink, Softsign, Tanh, Tanhshrink)
from .batch_norm import BatchNorm1d, BatchNorm2d, BatchNormAutoGrad
from .conv import Conv1d, Conv2d, Conv2dAutoGrad
from .cross_entropy import CrossEntropyLoss, CrossEntropyLossAutoGrad
from .linear import Linear, LinearAutoGrad
from .nll_loss import NLLLoss, NLLLossAutoGrad
from .norms import LayerNorm, LayerNormAutoGrad, RMSNorm, RMSNormAutoGrad
from .softmax import LogSoftmax, Softmax, SoftmaxAutoGrad, Softmin
from .utils import get_output_dtype

__all__ = [
    'ActFuncAutoGrad', 'BatchNorm1d', 'BatchNorm2d', 'BatchNormAutoGrad', 'CELU', 'Conv1d', 'Conv2d',
    'Conv2dAutoGrad', 'CrossEntropyLoss', 'CrossEntropyLossAutoGrad', 'Dropout', 'DropoutAutoGrad', 'ELU',
    'GELU', 'Hardshrink', 'Hardsigmoid', 'Hardswish', 'Hardtanh', 'LayerNorm', 'LayerNormAutoGrad',
    'LeakyReLU', 'Linear', 'LinearAutoGrad', 'LogSigmoid', 'LogSoftmax', 'Mish', 'NLLLoss', 'NLLLossAutoGrad',
    'RMSNorm',
    'RMSNormAutoGrad', 'ReLU', 'ReLU6', 'SELU', 'SiLU', 'Sigmoid', 'Softmax', 'SoftmaxAutoGrad', 'Softmin',
    'Softplus', 'Softshrink', 'Softsign', 'Tanh', 'Tanhshrink', 'get_output_dtype',
]
