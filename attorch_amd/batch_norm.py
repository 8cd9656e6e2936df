"""
Batch normalization with fused residual addition and activation with PyTorch autodiff
support, running on the gfx950 split-reduction kernels.

API mirrors attorch/batch_norm_layer.py: BatchNormAutoGrad.apply(input, training, weight,
bias, running_mean, running_var, momentum, eps, track_running_stats, pre_act_add, act_func)
and BatchNorm1d / BatchNorm2d modules whose forward takes an optional residual.  Inputs are
used in their native NC / NCL / NCHW layout.
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn
from torch.amp import custom_fwd

from . import _lib
from .utils import custom_bwd
from .act import act_id, parse_act_func


def _dims(input: Tensor) -> Tuple[int, int, int]:
    """
    (batch, feat, spatial) of a 2D, 3D or 4D batch-norm input.
    """
    spatial = 1
    for size in input.shape[2:]:
        spatial *= size
    return input.shape[0], input.shape[1], spatial


class BatchNormAutoGrad(torch.autograd.Function):
    """
    Autodiff for batch normalization (attorch/batch_norm_layer.py:39-245).
    """
    @staticmethod
    @custom_fwd(device_type='cuda')
    def forward(
        ctx: Any,
        input: Tensor,
        training: bool,
        weight: Optional[Tensor] = None,
        bias: Optional[Tensor] = None,
        running_mean: Optional[Tensor] = None,
        running_var: Optional[Tensor] = None,
        momentum: float = 0.1,
        eps: float = 1e-5,
        track_running_stats: bool = True,
        pre_act_add: Optional[Tensor] = None,
        act_func: Optional[str] = None,
        ) -> Tensor:
        """
        Batch-normalizes the input, optionally adding a residual and
        fusing an activation function.

        Args:
            input: Input of shape [batch_dim, feat_dim], [batch_dim, feat_dim, feat_len] or
                [batch_dim, feat_dim, height, width].
            training: Uses batch statistics and updates the running ones when True.
            weight: Optional scale [feat_dim]; affine only when bias is given too.
            bias: Optional shift [feat_dim].
            running_mean: Optional running mean [feat_dim], updated in place when training.
            running_var: Optional running variance [feat_dim], updated in place when training.
            momentum: Momentum of the running statistics.
            eps: Epsilon added under the square root.
            track_running_stats: Without it the batch statistics are always used.
            pre_act_add: Optional residual of the input's shape, added before the activation.
            act_func: Activation name (see attorch_amd.LinearAutoGrad), None for identity.

        Returns:
            Normalized (+ residual, activated) input, same shape and dtype as input.
        """
        _lib.require_same_device('BatchNorm', input, weight, bias, running_mean, running_var, pre_act_add)
        lib = _lib.load()
        act_func, param = parse_act_func(act_func)
        act = act_id(act_func, param)
        ctx.param = param
        ctx.act_func = act_func
        ctx.act = act

        add_pre_act = pre_act_add is not None
        affine = weight is not None and bias is not None
        requires_grad = (input.requires_grad or
                         (add_pre_act and pre_act_add.requires_grad) or
                         (affine and weight.requires_grad) or
                         (affine and bias.requires_grad))
        # relu, relu6 and hardtanh have the same derivative at the output as at the
        # pre-activation (the flat pieces map to their end points), so the output serves in
        # backward and the pre-activation is neither written nor kept
        ctx.output_as_pre_act = act_func in ('relu', 'relu6', 'hardtanh')
        save_pre_act = requires_grad and (act_func is not None) and not ctx.output_as_pre_act

        batch_dim, feat_dim, spatial_dim = _dims(input)
        # Channels-last 4D tensors (torch.channels_last) are processed and returned in that layout.
        layout = torch.contiguous_format
        if (input.dim() == 4 and not input.is_contiguous()
                and input.is_contiguous(memory_format=torch.channels_last)
                and lib.at_batch_norm_nhwc_supported(feat_dim, _lib.dtype_id(input.dtype))):
            layout = torch.channels_last
        ctx.layout = layout
        # Without spatial extent ([batch, feat] inputs) the contiguous tensor already is a matrix
        # of rows of features: the same kernels as for channels-last tensors apply, and read it
        # along its rows instead of one feature at a time.
        ctx.rows_of_features = layout is torch.channels_last or (
            spatial_dim == 1 and bool(lib.at_batch_norm_nhwc_supported(feat_dim, _lib.dtype_id(input.dtype))))
        forward_entry = (lib.at_batch_norm_fwd_nhwc if ctx.rows_of_features
                         else lib.at_batch_norm_fwd)
        input_k = input.contiguous(memory_format=layout)
        residual_k = (_lib.in_memory_format(pre_act_add.to(input.dtype), layout)
                      if add_pre_act else None)
        output = torch.empty_like(input_k)
        pre_act = torch.empty_like(input_k) if save_pre_act else None
        if requires_grad:
            mean = torch.empty(feat_dim, device=input.device, dtype=torch.float32)
            inv_std = torch.empty(feat_dim, device=input.device, dtype=torch.float32)
        else:
            mean = inv_std = None

        weight_k = weight.contiguous() if affine else None
        bias_k = bias.to(weight.dtype).contiguous() if affine else None
        use_running = running_mean is not None and running_var is not None
        workspace_bytes = lib.at_batch_norm_workspace_bytes(feat_dim)
        workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=input.device)

        with _lib.device_guard(input):
            _lib.check(forward_entry(
                _lib.ptr(input_k), _lib.ptr(weight_k), _lib.ptr(bias_k), _lib.ptr(mean),
                _lib.ptr(inv_std), _lib.ptr(residual_k), _lib.ptr(pre_act), _lib.ptr(output),
                _lib.ptr(running_mean) if use_running else None,
                _lib.ptr(running_var) if use_running else None,
                _lib.ptr(workspace), workspace_bytes, batch_dim, feat_dim, spatial_dim,
                momentum, eps, act, 0.0 if param is None else param,
                int(track_running_stats and use_running), int(training),
                _lib.dtype_id(input.dtype), _lib.dtype_id(weight_k.dtype) if affine else 0,
                _lib.dtype_id(running_mean.dtype) if use_running else 0,
                _lib.stream_of(input)), 'at_batch_norm_fwd')

        ctx.affine = affine
        ctx.add_pre_act = add_pre_act
        if requires_grad:
            ctx.save_for_backward(input_k, mean, inv_std, weight_k,
                                  pre_act if save_pre_act else (output if ctx.output_as_pre_act else None))

        return output.view_as(input)

    @staticmethod
    @custom_bwd
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Gradients with respect to input, weight, bias and the residual.
        """
        lib = _lib.load()
        (input, mean, inv_std, weight, pre_act) = ctx.saved_tensors
        _lib.require_same_device('BatchNorm backward', input, output_grad)
        batch_dim, feat_dim, spatial_dim = _dims(input)
        device = input.device

        output_grad_k = _lib.in_memory_format(output_grad.to(input.dtype), ctx.layout)
        backward_entry = (lib.at_batch_norm_bwd_nhwc if ctx.rows_of_features
                          else lib.at_batch_norm_bwd)
        input_grad = torch.empty_like(input)
        pre_act_grad = torch.empty_like(input) if ctx.act_func is not None else None
        if ctx.affine:
            weight_grad = torch.empty(feat_dim, device=device, dtype=torch.float32)
            bias_grad = torch.empty(feat_dim, device=device, dtype=torch.float32)
        else:
            weight_grad = bias_grad = None
        workspace_bytes = lib.at_batch_norm_workspace_bytes(feat_dim)
        workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device)

        with _lib.device_guard(input):
            _lib.check(backward_entry(
                _lib.ptr(output_grad_k), _lib.ptr(pre_act), _lib.ptr(input), _lib.ptr(mean),
                _lib.ptr(inv_std), _lib.ptr(weight), _lib.ptr(input_grad), _lib.ptr(pre_act_grad),
                _lib.ptr(weight_grad), _lib.ptr(bias_grad), _lib.ptr(workspace), workspace_bytes,
                batch_dim, feat_dim, spatial_dim, ctx.act, 0.0 if ctx.param is None else ctx.param,
                _lib.dtype_id(input.dtype), _lib.dtype_id(weight.dtype) if ctx.affine else 0,
                _lib.stream_of(input)), 'at_batch_norm_bwd')

        residual_grad = None
        if ctx.add_pre_act:
            residual_grad = pre_act_grad if pre_act_grad is not None else output_grad_k

        # One gradient (or None) per forward argument.
        return (input_grad, None,
                weight_grad, bias_grad,
                None, None, None, None, None,
                residual_grad,
                None)


class BatchNorm1d(nn.BatchNorm1d):
    """
    Batch-normalizes the 2D or 3D input, optionally fusing an activation function
    and adding a residual to the pre-activation result.
    See also base class; mirrors attorch/batch_norm_layer.py:248-300.

    Args:
        num_features: Number of features.
        eps: Epsilon added under the square root.
        momentum: Momentum of the running statistics.
        affine: Flag for learnable scale and shift.
        track_running_stats: Flag for tracking running statistics.
        act_func: Activation name (see attorch_amd.LinearAutoGrad), None for identity.
        device: Device to use.
        dtype: Dtype of layer.
    """
    def __init__(
        self,
        num_features: int,
        eps: float = 1e-5,
        momentum: float = 0.1,
        affine: bool = True,
        track_running_stats: bool = True,
        act_func: Optional[str] = None,
        device: Any = 'cuda',
        dtype: torch.dtype = torch.float32,
        ) -> None:
        super().__init__(num_features, eps, momentum, affine,
                         track_running_stats, device, dtype)
        self.act_func = act_func

    def forward(
        self,
        input: Tensor,
        pre_act_add: Optional[Tensor] = None,
        ) -> Tensor:
        self._check_input_dim(input)

        return BatchNormAutoGrad.apply(input, self.training,
                                       self.weight, self.bias,
                                       self.running_mean, self.running_var,
                                       self.momentum, self.eps,
                                       self.track_running_stats,
                                       pre_act_add, self.act_func)


class BatchNorm2d(nn.BatchNorm2d):
    """
    Batch-normalizes the 4D input, optionally fusing an activation function
    and adding a residual to the pre-activation result.
    See also base class; mirrors attorch/batch_norm_layer.py:303-355.

    Args:
        num_features: Number of features.
        eps: Epsilon added under the square root.
        momentum: Momentum of the running statistics.
        affine: Flag for learnable scale and shift.
        track_running_stats: Flag for tracking running statistics.
        act_func: Activation name (see attorch_amd.LinearAutoGrad), None for identity.
        device: Device to use.
        dtype: Dtype of layer.
    """
    def __init__(
        self,
        num_features: int,
        eps: float = 1e-5,
        momentum: float = 0.1,
        affine: bool = True,
        track_running_stats: bool = True,
        act_func: Optional[str] = None,
        device: Any = 'cuda',
        dtype: torch.dtype = torch.float32,
        ) -> None:
        super().__init__(num_features, eps, momentum, affine,
                         track_running_stats, device, dtype)
        self.act_func = act_func

    def forward(
        self,
        input: Tensor,
        pre_act_add: Optional[Tensor] = None,
        ) -> Tensor:
        self._check_input_dim(input)

        return BatchNormAutoGrad.apply(input, self.training,
                                       self.weight, self.bias,
                                       self.running_mean, self.running_var,
                                       self.momentum, self.eps,
                                       self.track_running_stats,
                                       pre_act_add, self.act_func)
