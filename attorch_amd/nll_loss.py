"""
Negative log likelihood loss with PyTorch autodiff support, running on the gfx950 kernels.

API mirrors attorch/nll_loss_layer.py: inputs of shape [batch, feat, ...] holding
log-probabilities, targets of shape [batch, ...], reductions 'none' / 'mean' / 'sum',
optional class weights, no ignore_index.  Together with LogSoftmax it is the reference's
flexible alternative to CrossEntropyLoss (attorch/cross_entropy_loss_layer.py:130-133).
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn

from . import _lib
from .utils import get_output_dtype


REDUCTIONS = {'none': 0, 'mean': 1, 'sum': 2}


class NLLLossAutoGrad(torch.autograd.Function):
    """
    Autodiff for negative log likelihood loss (attorch/nll_loss_layer.py:20-141).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        target: Tensor,
        reduction: str,
        weight: Optional[Tensor] = None,
        ) -> Tensor:
        """
        Measures the negative log likelihood loss between the input and target,
        with optional reweighing of each class.

        Args:
            input: Log-probabilities of shape [batch_dim, feat_dim, ...].
            target: Class indices of shape [batch_dim, ...] (same trailing dimensions).
            reduction: 'none' for a loss per entry, 'mean' for the (weighted) average,
                'sum' for the total.
            weight: Optional class weights of shape [feat_dim].

        Returns:
            Loss of shape [batch_dim, ...] for 'none' and a scalar otherwise, float32
            under autocast and the input dtype otherwise.
        """
        assert len(input) == len(target) and input.shape[2:] == target.shape[1:], \
            f'Incompatible input shape ({input.shape}) and target shape ({target.shape})'
        assert weight is None or len(weight) == input.shape[1], \
            f'Dimensionality of weight vector ({len(weight)}) and input features ({input.shape[1]}) not equal'
        assert reduction in REDUCTIONS, f'Reduction must be one of {tuple(REDUCTIONS)}, received {reduction}'

        _lib.require_same_device('NLLLoss', input, target, weight)
        lib = _lib.load()
        batch_dim, feat_dim = input.shape[:2]
        spatial_dim = 1
        for size in target.shape[1:]:
            spatial_dim *= size
        output_dtype = get_output_dtype(input.dtype, autocast='fp32')
        device = input.device

        input_k = input.contiguous()
        target_k = target.to(torch.int64).contiguous()
        weight_k = None if weight is None else weight.contiguous()
        output = torch.empty(target.shape if reduction == 'none' else (), dtype=output_dtype, device=device)
        sum_weights = (torch.empty(1, dtype=torch.float32, device=device)
                       if reduction == 'mean' and weight is not None else None)

        if batch_dim * spatial_dim == 0:
            # nothing to gather; the mean of no entries is nan, as with torch.nn.NLLLoss
            if reduction != 'none':
                output.fill_(float('nan') if reduction == 'mean' else 0.0)
        else:
            workspace = workspace_bytes = None
            if reduction != 'none':
                workspace_bytes = lib.at_nll_loss_workspace_bytes(batch_dim, spatial_dim)
                workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device)
            with _lib.device_guard(input):
                _lib.check(lib.at_nll_loss_fwd(
                    _lib.ptr(input_k), _lib.ptr(target_k), _lib.ptr(weight_k), _lib.ptr(output),
                    _lib.ptr(sum_weights), _lib.ptr(workspace), workspace_bytes or 0, batch_dim,
                    feat_dim, spatial_dim, REDUCTIONS[reduction], _lib.dtype_id(input.dtype),
                    _lib.dtype_id(weight_k.dtype) if weight_k is not None else 0,
                    _lib.dtype_id(output_dtype), _lib.stream_of(input)), 'at_nll_loss_fwd')

        ctx.reduction = reduction
        ctx.output_dtype = output_dtype
        ctx.input_shape = input.shape
        ctx.spatial_dim = spatial_dim
        if input.requires_grad:
            ctx.save_for_backward(target_k, weight_k, sum_weights)

        return output

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Input gradient of the loss: non-zero only at each entry's target class.
        """
        lib = _lib.load()
        target_k, weight_k, sum_weights = ctx.saved_tensors
        _lib.require_same_device('NLLLoss backward', target_k, output_grad)
        batch_dim, feat_dim = ctx.input_shape[:2]
        input_grad = torch.empty(ctx.input_shape, dtype=ctx.output_dtype, device=target_k.device)
        if input_grad.numel() > 0:
            output_grad = output_grad.contiguous()
            with _lib.device_guard(target_k):
                _lib.check(lib.at_nll_loss_bwd(
                    _lib.ptr(output_grad), _lib.ptr(target_k), _lib.ptr(weight_k), _lib.ptr(sum_weights),
                    _lib.ptr(input_grad), batch_dim, feat_dim, ctx.spatial_dim,
                    REDUCTIONS[ctx.reduction], _lib.dtype_id(output_grad.dtype),
                    _lib.dtype_id(weight_k.dtype) if weight_k is not None else 0,
                    _lib.dtype_id(ctx.output_dtype), _lib.stream_of(target_k)), 'at_nll_loss_bwd')

        # One gradient (or None) per forward argument.
        return input_grad, None, None, None


class NLLLoss(nn.NLLLoss):
    """
    Measures the negative log likelihood loss between the input and target,
    with optional reweighing of each class.
    See also base class.

    Args:
        reduction: 'none', 'mean' or 'sum'; size_average and reduce override it.
        size_average: Flag for averaging instead of summing the loss entries
            when reduce is True.
        reduce: Flag for averaging or summing all the loss entries instead of
            returning a loss per element.
        weight: Optional class weight vector of shape [feat_dim].
        ignore_index: Not supported, as in the reference (attorch/nll_loss_layer.py:162).
    """
    def forward(self, input: Tensor, target: Tensor) -> Tensor:
        return NLLLossAutoGrad.apply(input, target, self.reduction, self.weight)
