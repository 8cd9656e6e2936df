"""
Gated linear unit with an arbitrary activation function and PyTorch autodiff support.

API mirrors attorch/glu_layer.py.  Unlike the reference, the two halves of the gated dimension
are read where they lie and both gradients are written straight into the input gradient, so
no chunk, contiguous or concat copy is made.
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn

from . import _lib
from .act import act_id, parse_act_func


def _gate_geometry(shape: torch.Size, dim: int) -> Tuple[int, int]:
    """
    (outer, half): product of the sizes before `dim`, and half the size of `dim` times the
    product of the sizes after it.
    """
    dim = dim % len(shape)
    outer = 1
    for size in shape[:dim]:
        outer *= size
    inner = 1
    for size in shape[dim + 1:]:
        inner *= size
    return outer, (shape[dim] // 2) * inner


class GLUAutoGrad(torch.autograd.Function):
    """
    Autodiff for gated linear unit (attorch/glu_layer.py:18-116).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        dim: int,
        act_func: str,
        ) -> Tensor:
        """
        Applies the gated linear unit with an arbitrary activation function to the input:
        first half of dimension dim times the activated second half.

        Args:
            input: Input to gate; dimension dim must be even.
            dim: Dimension over which to gate.
            act_func: Activation name: 'sigmoid', 'logsigmoid', 'tanh', 'relu', 'gelu',
                'geluapprox', 'silu', 'relu6', 'hardsigmoid', 'hardtanh', 'hardswish', 'selu',
                'mish', 'softplus', 'softsign', 'tanhshrink', 'leaky_relu_PARAM', 'elu_PARAM',
                'celu_PARAM', 'hardshrink_PARAM', 'softshrink_PARAM'.

        Returns:
            Gated input, dimension dim halved.
        """
        assert input.shape[dim] % 2 == 0, \
            f'Dimension {dim} of the input ({input.shape[dim]}) must be even'
        _lib.require_gpu(input, 'GLU')
        lib = _lib.load()
        name, param = parse_act_func(act_func)
        act = act_id(name, param)

        input_k = input.contiguous()
        outer, half = _gate_geometry(input.shape, dim)
        out_shape = list(input.shape)
        out_shape[dim] //= 2
        output = torch.empty(out_shape, dtype=input.dtype, device=input.device)
        with _lib.device_guard(input):
            _lib.check(lib.at_glu_fwd(_lib.ptr(input_k), _lib.ptr(output), outer, half, act,
                                      0.0 if param is None else param, _lib.dtype_id(input.dtype),
                                      _lib.stream_of(input)), 'at_glu_fwd')

        ctx.act = act
        ctx.param = param
        ctx.geometry = (outer, half)
        if input.requires_grad:
            ctx.save_for_backward(input_k)
        return output

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Input gradient of the gated linear unit, both halves in one tensor.
        """
        lib = _lib.load()
        (input_k,) = ctx.saved_tensors
        _lib.require_same_device('GLU backward', input_k, output_grad)
        outer, half = ctx.geometry
        output_grad = output_grad.contiguous()
        input_grad = torch.empty_like(input_k)
        with _lib.device_guard(input_k):
            _lib.check(lib.at_glu_bwd(_lib.ptr(output_grad), _lib.ptr(input_k), _lib.ptr(input_grad),
                                      outer, half, ctx.act, 0.0 if ctx.param is None else ctx.param,
                                      _lib.dtype_id(input_k.dtype), _lib.stream_of(input_k)), 'at_glu_bwd')
        # One gradient (or None) per forward argument.
        return input_grad, None, None


class GLU(nn.GLU):
    """
    Applies the gated linear unit with an arbitrary activation function to the input.
    See also base class.

    Args:
        dim: Dimension over which to gate.
        act_func: Name of the activation applied to the second half (see GLUAutoGrad).
    """
    def __init__(self, dim: int = -1, act_func: str = 'sigmoid') -> None:
        super().__init__(dim)
        self.act_func = act_func

    def forward(self, input: Tensor) -> Tensor:
        return GLUAutoGrad.apply(input, self.dim, self.act_func)
