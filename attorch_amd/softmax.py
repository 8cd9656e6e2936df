"""
Softmax, LogSoftmax and Softmin over the last dimension with PyTorch autodiff support.

API mirrors attorch/softmax_layers.py: one autograd Function parametrized by the `neg`
(softmin) and `log` (log-softmax) flags, and three nn.Module subclasses that reject any
dimension but the last.
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn

from . import _lib
from .utils import get_output_dtype


class SoftmaxAutoGrad(torch.autograd.Function):
    """
    Autodiff for the softmax family (attorch/softmax_layers.py:18-94).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        neg: bool,
        log: bool,
        ) -> Tensor:
        """
        Normalizes the input over its last dimension using softmax.

        Args:
            input: Input of shape [..., feat_dim] (a 1D input is one row).
            neg: Negates the input first (softmin).
            log: Returns the logarithm of the result (log-softmax).

        Returns:
            Normalized input, float32 under autocast and the input dtype otherwise.
        """
        _lib.require_gpu(input, 'Softmax')
        lib = _lib.load()
        flattened_input = _lib.rows(input)
        batch_dim, feat_dim = flattened_input.shape

        output_dtype = get_output_dtype(input.dtype, autocast='fp32')
        output = torch.empty((batch_dim, feat_dim), device=input.device, dtype=output_dtype)

        with _lib.device_guard(input):
            _lib.check(lib.at_softmax_fwd(
                _lib.ptr(flattened_input), _lib.ptr(output), batch_dim, feat_dim,
                _lib.row_stride(flattened_input), _lib.row_stride(output), int(neg), int(log),
                _lib.dtype_id(input.dtype), _lib.dtype_id(output_dtype),
                _lib.stream_of(input)), 'at_softmax_fwd')

        ctx.neg = neg
        ctx.log = log
        if input.requires_grad:
            ctx.save_for_backward(output)

        return output.view_as(input)

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Input gradient of the softmax family, computed from the saved output.
        """
        lib = _lib.load()
        (output,) = ctx.saved_tensors
        _lib.require_same_device('Softmax backward', output, output_grad)
        flattened_output_grad = _lib.rows(output_grad.reshape(output.shape).to(output.dtype))
        batch_dim, feat_dim = output.shape
        input_grad = torch.empty_like(output)

        with _lib.device_guard(output):
            _lib.check(lib.at_softmax_bwd(
                _lib.ptr(flattened_output_grad), _lib.ptr(output), _lib.ptr(input_grad),
                batch_dim, feat_dim, _lib.row_stride(flattened_output_grad), _lib.row_stride(output),
                _lib.row_stride(input_grad), int(ctx.neg), int(ctx.log),
                _lib.dtype_id(flattened_output_grad.dtype), _lib.dtype_id(output.dtype),
                _lib.dtype_id(input_grad.dtype), _lib.stream_of(output)), 'at_softmax_bwd')

        return input_grad.view_as(output_grad), None, None


class Softmax(nn.Softmax):
    """
    Normalizes the input using softmax. See also base class.

    Args:
        dim: Dimension along which softmax is computed; only the last one is supported.
    """
    def forward(self, input: Tensor) -> Tensor:
        if self.dim != -1 and self.dim != input.ndim - 1:
            raise RuntimeError('Only softmax along the last dimension is supported.')

        return SoftmaxAutoGrad.apply(input, False, False)


class LogSoftmax(nn.LogSoftmax):
    """
    Normalizes the input using softmax and takes its log. See also base class.

    Args:
        dim: Dimension along which softmax is computed; only the last one is supported.
    """
    def forward(self, input: Tensor) -> Tensor:
        if self.dim != -1 and self.dim != input.ndim - 1:
            raise RuntimeError('Only softmax along the last dimension is supported.')

        return SoftmaxAutoGrad.apply(input, False, True)


class Softmin(nn.Softmin):
    """
    Normalizes the input using softmin. See also base class.

    Args:
        dim: Dimension along which softmin is computed; only the last one is supported.
    """
    def forward(self, input: Tensor) -> Tensor:
        if self.dim != -1 and self.dim != input.ndim - 1:
            raise RuntimeError('Only softmin along the last dimension is supported.')

        return SoftmaxAutoGrad.apply(input, True, False)
