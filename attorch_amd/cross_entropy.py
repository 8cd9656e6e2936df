"""
Cross entropy loss with PyTorch autodiff support, running on the fused gfx950 kernel.

API mirrors attorch/cross_entropy_loss_layer.py (mean reduction only, no label smoothing,
optional class weights) and adds what the reference lacks: ignore_index.  The forward pass
reads the logits once and produces both the loss and, when the logits require a gradient,
the gradient for an upstream gradient of one; backward hands that gradient out when the
upstream gradient is one and recomputes it from the logits otherwise.
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn

from . import _lib
from .utils import get_output_dtype


class CrossEntropyLossAutoGrad(torch.autograd.Function):
    """
    Autodiff for cross entropy loss (attorch/cross_entropy_loss_layer.py:20-121).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        target: Tensor,
        weight: Optional[Tensor] = None,
        ignore_index: int = -100,
        ) -> Tensor:
        """
        Mean cross entropy of the logits against class indices.

        Args:
            input: Logits of shape [batch_dim, feat_dim].
            target: Class indices of shape [batch_dim] (int64).
            weight: Optional class weights of shape [feat_dim]; the mean is then weighted.
            ignore_index: Rows with this target contribute neither loss nor gradient.

        Returns:
            Scalar loss, float32 under autocast and the input dtype otherwise.
        """
        assert input.ndim == 2, f'Inputs of rank other than 2 not valid'
        assert len(input) == len(target), \
            f'Incompatible input shape ({input.shape}) and target shape ({target.shape})'
        assert weight is None or len(weight) == input.shape[1], \
            f'Dimensionality of weight vector ({len(weight)}) and input features ({input.shape[1]}) not equal'

        _lib.require_same_device('CrossEntropyLoss', input, target, weight)
        lib = _lib.load()
        batch_dim, feat_dim = input.shape
        output_dtype = get_output_dtype(input.dtype, autocast='fp32')

        if batch_dim == 0:
            # mean over no rows, as torch: nan loss, empty gradient; nothing is launched
            ctx.empty = True
            ctx.grad_shape_dtype = (input.shape, input.dtype, input.device)
            return torch.full((), float('nan'), dtype=output_dtype, device=input.device)

        logits = input if input.stride(1) == 1 and input.stride(0) >= feat_dim else input.contiguous()
        target_k = target.to(torch.int64).contiguous()
        weight_k = None if weight is None else weight.contiguous()
        output = torch.empty((), dtype=output_dtype, device=input.device)
        # The gradient is computed in float32 and rounded once, straight to the dtype of the
        # logits: under autocast the reference produces a float32 gradient that autograd then
        # casts to that dtype (attorch/cross_entropy_loss_layer.py:24, custom_fwd with
        # cast_inputs), which is the same single rounding after a float32 round trip
        # through memory.
        input_grad = (torch.empty((batch_dim, feat_dim), dtype=input.dtype, device=input.device)
                      if input.requires_grad else None)
        workspace_bytes = lib.at_cross_entropy_workspace_bytes(batch_dim)
        workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=input.device)

        with _lib.device_guard(input):
            _lib.check(lib.at_cross_entropy_fwd_bwd(
                _lib.ptr(logits), _lib.ptr(target_k), _lib.ptr(weight_k), _lib.ptr(output),
                _lib.ptr(input_grad), _lib.ptr(workspace), workspace_bytes, batch_dim, feat_dim,
                _lib.row_stride(logits), feat_dim, ignore_index, _lib.dtype_id(logits.dtype),
                _lib.dtype_id(weight_k.dtype) if weight_k is not None else 0,
                _lib.dtype_id(input.dtype), _lib.dtype_id(output_dtype), _lib.stream_of(input)),
                'at_cross_entropy_fwd_bwd')

        ctx.empty = False
        ctx.output_dtype = output_dtype
        ctx.ignore_index = ignore_index
        ctx.has_weight = weight_k is not None
        # the gradient computed above may be handed to autograd once; see backward
        ctx.unit_grad_available = input.requires_grad
        if input.requires_grad:
            saved = [logits, target_k, workspace, input_grad]
            if weight_k is not None:
                saved.append(weight_k)
            ctx.save_for_backward(*saved)

        return output

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Gradient of the logits, output_grad * (softmax - onehot) * weight[target] / divisor
        (attorch/cross_entropy_loss_layer.py:85-121).  The first call returns the buffer the
        forward pass filled for an upstream gradient of one: the kernel leaves it as it is when
        the upstream value (read on the device) is exactly one and recomputes it from the
        logits otherwise, the upstream value multiplied in before the one rounding.  That
        buffer then belongs to autograd, so any later call (retain_graph) computes into a
        fresh one.
        """
        if ctx.empty:
            shape, dtype, device = ctx.grad_shape_dtype
            return torch.empty(shape, dtype=dtype, device=device), None, None, None

        lib = _lib.load()
        logits, target_k, workspace, unit_grad = ctx.saved_tensors[:4]
        weight_k = ctx.saved_tensors[4] if ctx.has_weight else None
        batch_dim, feat_dim = logits.shape
        _lib.require_same_device('CrossEntropyLoss backward', logits, output_grad)
        output_grad = output_grad.contiguous()
        if output_grad.dtype not in _lib.DTYPE_IDS:
            output_grad = output_grad.float()

        if ctx.unit_grad_available:
            input_grad, holds_unit_grad = unit_grad, 1
            ctx.unit_grad_available = False
        else:
            input_grad, holds_unit_grad = torch.empty_like(unit_grad), 0

        with _lib.device_guard(logits):
            _lib.check(lib.at_cross_entropy_bwd(
                _lib.ptr(logits), _lib.ptr(target_k), _lib.ptr(weight_k), _lib.ptr(output_grad),
                _lib.ptr(workspace), _lib.ptr(input_grad), batch_dim, feat_dim,
                _lib.row_stride(logits), feat_dim, ctx.ignore_index, holds_unit_grad,
                _lib.dtype_id(logits.dtype),
                _lib.dtype_id(weight_k.dtype) if weight_k is not None else 0,
                _lib.dtype_id(output_grad.dtype), _lib.dtype_id(input_grad.dtype),
                _lib.stream_of(logits)), 'at_cross_entropy_bwd')

        return input_grad, None, None, None


class CrossEntropyLoss(nn.CrossEntropyLoss):
    """
    Mean cross entropy between logits and class indices, optionally weighted per class.
    See also base class; mirrors attorch/cross_entropy_loss_layer.py:124-170 and
    additionally honours ignore_index.

    Args:
        reduction: Only 'mean' is supported.
        size_average: Deprecated torch argument, forwarded to the base class.
        reduce: Deprecated torch argument, forwarded to the base class.
        weight: Optional class weights of shape [feat_dim].
        ignore_index: Target value whose rows are ignored.
        label_smoothing: Must be 0.
    """
    def __init__(
        self,
        reduction: str = 'mean',
        size_average: Optional[bool] = None,
        reduce: Optional[bool] = None,
        weight: Optional[Tensor] = None,
        ignore_index: int = -100,
        label_smoothing: float = 0.0,
        ) -> None:
        super().__init__(weight, size_average, ignore_index, reduce,
                         reduction, label_smoothing)

        if self.reduction != 'mean':
            raise RuntimeError('Cross entropy only supports averaging the loss.')

        if label_smoothing > 0.0:
            raise RuntimeError('Cross entropy does not support label smoothing.')

    def forward(self, input: Tensor, target: Tensor) -> Tensor:
        return CrossEntropyLossAutoGrad.apply(input, target, self.weight, self.ignore_index)
