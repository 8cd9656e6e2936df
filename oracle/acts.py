"""
Oracle (test infrastructure): the 21 activation functions and their derivatives, restated
from attorch/act_kernels.py:13-628 and the dispatchers at :631-837.
"""

from typing import Optional, Tuple

import torch
from torch import Tensor

ACT_NAMES = ('sigmoid', 'logsigmoid', 'tanh', 'relu', 'gelu', 'geluapprox', 'silu', 'relu6',
             'hardsigmoid', 'hardtanh', 'hardswish', 'selu', 'mish', 'softplus', 'softsign',
             'tanhshrink', 'leaky_relu', 'elu', 'celu', 'hardshrink', 'softshrink')

SELU_SCALE = 1.0507009873554804934193349852946
SELU_ALPHA = 1.6732632423543772848170429916717


def parse_act_func(act_func: Optional[str]) -> Tuple[Optional[str], Optional[float]]:
    """
    Splits 'name_PARAM' into (name, float(PARAM)) as attorch/linear_layer.py:65-69 does:
    any name containing '_' is split at its last underscore.
    """
    param = None
    if act_func is not None and '_' in act_func:
        comps = act_func.split('_')
        act_func = '_'.join(comps[:-1])
        param = float(comps[-1])
    return act_func, param


def _sigmoid(x: Tensor) -> Tensor:
    return 1 / (1 + torch.exp(-x))                      # act_kernels.py:24


def _tanh(x: Tensor) -> Tensor:
    return 2 * _sigmoid(2 * x) - 1                      # act_kernels.py:81


def act_forward(x: Tensor, name: str, param: Optional[float] = None) -> Tensor:
    """
    Applies activation `name` elementwise (attorch/act_kernels.py:631-732).
    The input is used in its own floating dtype (callers pass fp32 or fp64).
    """
    zero = torch.zeros((), dtype=x.dtype)
    if name == 'sigmoid':
        return _sigmoid(x)
    if name == 'logsigmoid':
        return torch.log(_sigmoid(x))                   # :53
    if name == 'tanh':
        return _tanh(x)
    if name == 'relu':
        return torch.maximum(zero, x)                   # :110
    if name == 'gelu':
        return 0.5 * (1 + torch.erf(0.707106781 * x)) * x          # :138-139
    if name == 'geluapprox':
        return 0.5 * (1 + _tanh(0.7978845608 * x * (1 + 0.044715 * x * x))) * x   # :169-170
    if name == 'silu':
        return x * _sigmoid(x)                          # :200
    if name == 'relu6':
        return torch.clamp(x, 0, 6)                     # :229
    if name == 'hardsigmoid':
        return torch.clamp(x / 6 + 0.5, 0, 1)           # :257
    if name == 'hardtanh':
        return torch.clamp(x, -1, 1)                    # :285
    if name == 'hardswish':
        return x * torch.clamp(x + 3, 0, 6) / 6         # :313
    if name == 'selu':
        return SELU_SCALE * (torch.maximum(zero, x) +
                             torch.minimum(zero, SELU_ALPHA * (torch.exp(x) - 1)))   # :341-344
    if name == 'mish':
        return x * _tanh(torch.log(1 + torch.exp(x)))   # :374
    if name == 'softplus':
        return torch.log(1 + torch.exp(x))              # :405
    if name == 'softsign':
        return x / (1 + x.abs())                        # :433
    if name == 'tanhshrink':
        return x - _tanh(x)                             # :462
    if name == 'leaky_relu':
        return torch.maximum(zero, x) + param * torch.minimum(zero, x)     # :491
    if name == 'elu':
        return torch.where(x <= 0, param * (torch.exp(x) - 1), x)          # :521
    if name == 'celu':
        return torch.maximum(zero, x) + torch.minimum(zero, param * (torch.exp(x / param) - 1))  # :551
    if name == 'hardshrink':
        return torch.where(x.abs() <= param, zero, x)   # :582
    if name == 'softshrink':
        return torch.where(x > param, x - param,
                           torch.where(x < -param, x + param, zero))       # :612-613
    raise ValueError(f'unknown activation {name}')


def act_grad(x: Tensor, name: str, param: Optional[float] = None) -> Tensor:
    """
    Derivative of activation `name` at x (attorch/act_kernels.py:735-837); the piecewise
    ones keep the reference's choice of <= / < at the joints.
    """
    one = torch.ones((), dtype=x.dtype)
    zero = torch.zeros((), dtype=x.dtype)
    if name == 'sigmoid':
        s = _sigmoid(x)
        return s * (1 - s)                              # :38-39
    if name == 'logsigmoid':
        return 1 / (1 + torch.exp(x))                   # :67
    if name == 'tanh':
        t = _tanh(x)
        return 1 - t * t                                # :95-96
    if name == 'relu':
        return torch.where(x <= 0, zero, one)           # :124
    if name == 'gelu':
        cdf = 0.5 * (1 + torch.erf(0.707106781 * x))
        return 0.39894228 * torch.exp(-0.5 * x * x) * x + cdf       # :153-155
    if name == 'geluapprox':
        t = _tanh(0.7978845608 * x * (1 + 0.044715 * x * x))
        return 0.5 * (1 + t + x * (1 - t * t) * 0.7978845608 * (1 + 3 * 0.044715 * x * x))  # :184-186
    if name == 'silu':
        s = _sigmoid(x)
        return s * (x * (1 - s) + 1)                    # :214-215
    if name == 'relu6':
        return torch.where((0 < x) & (x < 6), one, zero)            # :243
    if name == 'hardsigmoid':
        return torch.where((-3 < x) & (x < 3), one / 6, zero)       # :271
    if name == 'hardtanh':
        return torch.where((-1 < x) & (x < 1), one, zero)           # :299
    if name == 'hardswish':
        return torch.where(x < -3, zero, torch.where(x <= 3, x / 3 + 0.5, one))   # :327
    if name == 'selu':
        return SELU_SCALE * torch.where(x <= 0, SELU_ALPHA * torch.exp(x), one)   # :358-360
    if name == 'mish':
        e = torch.exp(x)
        delta = e * (e + 2) + 2
        return e * (e * ((4 * x + 6) + e * (e + 4)) + 4 * (x + 1)) / (delta * delta)   # :388-391
    if name == 'softplus':
        return _sigmoid(x)                              # :419
    if name == 'softsign':
        d = 1 + x.abs()
        return 1 / (d * d)                              # :447-448
    if name == 'tanhshrink':
        t = _tanh(x)
        return t * t                                    # :476 (1 - tanh_grad)
    if name == 'leaky_relu':
        return torch.where(x <= 0, param * one, one)    # :506
    if name == 'elu':
        return torch.where(x <= 0, param * torch.exp(x), one)       # :536
    if name == 'celu':
        return torch.where(x <= 0, torch.exp(x / param), one)       # :566
    if name in ('hardshrink', 'softshrink'):
        return torch.where(x.abs() <= param, zero, one)             # :597, :628
    raise ValueError(f'unknown activation {name}')
