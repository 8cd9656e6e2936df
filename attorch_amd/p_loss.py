"""
L1, squared L2 (MSE), smooth L1 and Huber losses with PyTorch autodiff support.

API mirrors attorch/p_loss_layers.py: reductions 'none' / 'mean' / 'sum', gradients for both
the input and the target.
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn

from . import _lib
from .nll_loss import REDUCTIONS
from .utils import get_output_dtype


class PLossAutoGrad(torch.autograd.Function):
    """
    Autodiff for the p-norm-induced losses (attorch/p_loss_layers.py:18-107).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        target: Tensor,
        p_loss: int,
        reduction: str,
        param: float = 1.0,
        ) -> Tensor:
        """
        Measures the smooth L1, L1, squared L2, or Huber loss of the difference
        between the input and target.

        Args:
            input: Input of arbitrary shape.
            target: Target of the same shape.
            p_loss: 0 for smooth L1, 1 for L1, 2 for squared L2, 3 for Huber loss.
            reduction: 'none', 'mean' or 'sum'.
            param: Beta (smooth L1) or delta (Huber).

        Returns:
            Error, float32 under autocast and the input dtype otherwise.
        """
        assert input.shape == target.shape, \
            f'Input shape {input.shape} and target shape {target.shape} not equal'
        assert reduction in REDUCTIONS, f'Reduction must be one of {tuple(REDUCTIONS)}, received {reduction}'
        _lib.require_same_device('p-norm loss', input, target)
        lib = _lib.load()
        output_dtype = get_output_dtype(input.dtype, autocast='fp32')
        device = input.device

        input_k = input.contiguous()
        target_k = target.to(input.dtype).contiguous()
        size = input_k.numel()
        output = torch.empty(input.shape if reduction == 'none' else (), dtype=output_dtype, device=device)
        if size == 0:
            if reduction != 'none':
                output.fill_(float('nan') if reduction == 'mean' else 0.0)
        else:
            workspace = workspace_bytes = None
            if reduction != 'none':
                workspace_bytes = lib.at_p_loss_workspace_bytes(size)
                workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device)
            with _lib.device_guard(input):
                _lib.check(lib.at_p_loss_fwd(
                    _lib.ptr(input_k), _lib.ptr(target_k), _lib.ptr(output), _lib.ptr(workspace),
                    workspace_bytes or 0, size, p_loss, REDUCTIONS[reduction], param,
                    _lib.dtype_id(input.dtype), _lib.dtype_id(output_dtype), _lib.stream_of(input)),
                    'at_p_loss_fwd')

        ctx.p_loss = p_loss
        ctx.reduction = reduction
        ctx.param = param
        ctx.output_dtype = output_dtype
        ctx.needs = (input.requires_grad, target.requires_grad)
        if input.requires_grad or target.requires_grad:
            ctx.save_for_backward(input_k, target_k)
        return output

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Gradients of the error with respect to the input and the target (its negative).
        """
        lib = _lib.load()
        input_k, target_k = ctx.saved_tensors
        _lib.require_same_device('p-norm loss backward', input_k, output_grad)
        needs_input, needs_target = ctx.needs
        size = input_k.numel()
        input_grad = torch.empty_like(input_k, dtype=ctx.output_dtype) if needs_input else None
        target_grad = torch.empty_like(target_k, dtype=ctx.output_dtype) if needs_target else None
        if size > 0:
            output_grad = output_grad.contiguous()
            with _lib.device_guard(input_k):
                _lib.check(lib.at_p_loss_bwd(
                    _lib.ptr(output_grad), _lib.ptr(input_k), _lib.ptr(target_k), _lib.ptr(input_grad),
                    _lib.ptr(target_grad), size, ctx.p_loss, REDUCTIONS[ctx.reduction], ctx.param,
                    _lib.dtype_id(input_k.dtype), _lib.dtype_id(output_grad.dtype),
                    _lib.dtype_id(ctx.output_dtype), _lib.stream_of(input_k)), 'at_p_loss_bwd')
        # One gradient (or None) per forward argument.
        return input_grad, target_grad, None, None, None


class L1Loss(nn.L1Loss):
    """
    Measures the L1 error (mean absolute error) between the input and target.
    See also base class.
    """
    def forward(self, input: Tensor, target: Tensor) -> Tensor:
        return PLossAutoGrad.apply(input, target, 1, self.reduction)


class MSELoss(nn.MSELoss):
    """
    Measures the squared L2 error (mean squared error) between the input and target.
    See also base class.
    """
    def forward(self, input: Tensor, target: Tensor) -> Tensor:
        return PLossAutoGrad.apply(input, target, 2, self.reduction)


class SmoothL1Loss(nn.SmoothL1Loss):
    """
    Measures the smooth L1 error between the input and target; beta is the softening threshold.
    See also base class.
    """
    def forward(self, input: Tensor, target: Tensor) -> Tensor:
        return PLossAutoGrad.apply(input, target, 0, self.reduction, self.beta)


class HuberLoss(nn.HuberLoss):
    """
    Measures the Huber loss between the input and target; delta is the softening threshold.
    See also base class.
    """
    def forward(self, input: Tensor, target: Tensor) -> Tensor:
        return PLossAutoGrad.apply(input, target, 3, self.reduction, self.delta)
