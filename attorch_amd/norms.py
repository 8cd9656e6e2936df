"""
LayerNorm and RMSNorm with PyTorch autodiff support, running on the gfx950 row kernels.

API mirrors attorch/layer_norm_layer.py and attorch/rms_norm_layer.py: same autograd
Function signatures, same module constructors, same saved statistics (fp32 mean / inverse
standard deviation / inverse RMS per row) and the same mixed-precision behaviour.
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn
from torch.amp import custom_fwd

from . import _lib
from .utils import custom_bwd, get_output_dtype


def _param_for_kernel(param: Optional[Tensor], input: Tensor) -> Optional[Tensor]:
    """
    Parameters reach the kernels stored like the input or in fp32; any other pairing
    (e.g. a 16-bit parameter beside an fp32 input) is widened to fp32 first.
    """
    if param is None:
        return None
    if param.dtype not in (input.dtype, torch.float32):
        param = param.float()
    return param.contiguous()


class LayerNormAutoGrad(torch.autograd.Function):
    """
    Autodiff for layer normalization (attorch/layer_norm_layer.py:19-157).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        weight: Optional[Tensor] = None,
        bias: Optional[Tensor] = None,
        eps: float = 1e-5,
        autocast_to_fp32: bool = True,
        ) -> Tensor:
        """
        Layer-normalizes the input over its last dimension.

        Args:
            input: Input of shape [..., feat_dim] (a 1D input is one row).
            weight: Optional scale of shape [feat_dim].
            bias: Optional shift of shape [feat_dim]; ignored when weight is None.
            eps: Epsilon added under the square root.
            autocast_to_fp32: Returns float32 under autocast when True.

        Returns:
            Normalized input, same shape as input.
        """
        _lib.require_same_device('LayerNorm', input, weight, bias)
        lib = _lib.load()
        flattened_input = _lib.rows(input)
        batch_dim, feat_dim = flattened_input.shape

        output_dtype = get_output_dtype(input.dtype,
                                        autocast='fp32' if autocast_to_fp32 else None)
        output = torch.empty((batch_dim, feat_dim), device=input.device, dtype=output_dtype)

        scale_by_weight = weight is not None
        add_bias = scale_by_weight and bias is not None
        requires_grad = (input.requires_grad or
                         (scale_by_weight and weight.requires_grad) or
                         (add_bias and bias.requires_grad))
        if requires_grad:
            mean = torch.empty(batch_dim, device=input.device, dtype=torch.float32)
            inv_std = torch.empty(batch_dim, device=input.device, dtype=torch.float32)
        else:
            mean = inv_std = None

        weight_k = _param_for_kernel(weight, flattened_input) if scale_by_weight else None
        bias_k = _param_for_kernel(bias, flattened_input) if add_bias else None
        if add_bias and bias_k.dtype != weight_k.dtype:
            bias_k = bias_k.to(weight_k.dtype)

        with _lib.device_guard(input):
            _lib.check(lib.at_layer_norm_fwd(
                _lib.ptr(flattened_input), _lib.ptr(weight_k), _lib.ptr(bias_k),
                _lib.ptr(mean), _lib.ptr(inv_std), _lib.ptr(output),
                batch_dim, feat_dim, _lib.row_stride(flattened_input), _lib.row_stride(output), eps,
                _lib.dtype_id(input.dtype),
                _lib.dtype_id(weight_k.dtype) if scale_by_weight else 0,
                _lib.dtype_id(output_dtype), _lib.stream_of(input)), 'at_layer_norm_fwd')

        ctx.scale_by_weight = scale_by_weight
        ctx.add_bias = add_bias
        ctx.output_dtype = output_dtype
        if requires_grad:
            ctx.save_for_backward(flattened_input, mean, inv_std, weight)

        return output.view_as(input)

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Input, weight and bias gradients of layer normalization.
        The parameter gradients come back in float32, as in the reference
        (attorch/layer_norm_layer.py:124-128); autograd casts them.
        """
        lib = _lib.load()
        scale_by_weight, add_bias = ctx.scale_by_weight, ctx.add_bias
        (flattened_input, mean, inv_std, weight) = ctx.saved_tensors
        _lib.require_same_device('LayerNorm backward', flattened_input, output_grad)
        flattened_output_grad = _lib.rows(output_grad.reshape(flattened_input.shape)
                                          .to(ctx.output_dtype))
        batch_dim, feat_dim = flattened_output_grad.shape
        device = flattened_input.device

        input_grad = torch.empty((batch_dim, feat_dim), device=device, dtype=ctx.output_dtype)
        weight_grad = bias_grad = workspace = None
        workspace_bytes = 0
        if scale_by_weight:
            weight_grad = torch.empty(feat_dim, device=device, dtype=torch.float32)
            if add_bias:
                bias_grad = torch.empty(feat_dim, device=device, dtype=torch.float32)
            workspace_bytes = lib.at_norm_bwd_workspace_bytes(batch_dim, feat_dim,
                                                              2 if add_bias else 1)
            workspace = torch.empty(workspace_bytes, device=device, dtype=torch.uint8)
        weight_k = _param_for_kernel(weight, flattened_input) if scale_by_weight else None

        with _lib.device_guard(flattened_input):
            _lib.check(lib.at_layer_norm_bwd(
                _lib.ptr(flattened_output_grad), _lib.ptr(flattened_input),
                _lib.ptr(mean), _lib.ptr(inv_std), _lib.ptr(weight_k),
                _lib.ptr(input_grad), _lib.ptr(weight_grad), _lib.ptr(bias_grad),
                _lib.ptr(workspace), workspace_bytes, batch_dim, feat_dim,
                _lib.row_stride(flattened_output_grad), _lib.row_stride(flattened_input),
                _lib.row_stride(input_grad),
                _lib.dtype_id(flattened_output_grad.dtype), _lib.dtype_id(flattened_input.dtype),
                _lib.dtype_id(weight_k.dtype) if scale_by_weight else 0,
                _lib.dtype_id(input_grad.dtype), _lib.stream_of(flattened_input)),
                'at_layer_norm_bwd')

        # One gradient (or None) per forward argument.
        return input_grad.view_as(output_grad), weight_grad, bias_grad, None, None


class LayerNorm(nn.LayerNorm):
    """
    Layer-normalizes the input over its last dimension.
    See also base class; mirrors attorch/layer_norm_layer.py:160-206.

    Args:
        normalized_shape: Size of the last dimension (an integer).
        eps: Epsilon added under the square root.
        elementwise_affine: Flag for a learnable scale.
        bias: Flag for a learnable shift (only with elementwise_affine).
        autocast_to_fp32: Returns float32 under autocast when True.
        device: Device to use.
        dtype: Dtype of layer.
    """
    def __init__(
        self,
        normalized_shape: int,
        eps: float = 1e-5,
        elementwise_affine: bool = True,
        bias: bool = True,
        autocast_to_fp32: bool = True,
        device: Any = 'cuda',
        dtype: torch.dtype = torch.float32,
        ) -> None:
        if not isinstance(normalized_shape, int):
            raise RuntimeError('Normalized shape must be an integer.')

        super().__init__(normalized_shape, eps, elementwise_affine, bias,
                         device, dtype)
        self.autocast_to_fp32 = autocast_to_fp32

    def forward(self, input: Tensor) -> Tensor:
        return LayerNormAutoGrad.apply(input, self.weight, self.bias, self.eps,
                                       self.autocast_to_fp32)


class RMSNormAutoGrad(torch.autograd.Function):
    """
    Autodiff for root mean square normalization (attorch/rms_norm_layer.py:19-134).
    """
    @staticmethod
    @custom_fwd(device_type='cuda')
    def forward(
        ctx: Any,
        input: Tensor,
        weight: Optional[Tensor] = None,
        eps: Optional[float] = None,
        ) -> Tensor:
        """
        Root-mean-square-normalizes the input over its last dimension.

        Args:
            input: Input of shape [..., feat_dim] (a 1D input is one row).
            weight: Optional scale of shape [feat_dim].
            eps: Epsilon added under the square root; None selects
                torch.finfo(input.dtype).eps.

        Returns:
            Normalized input, same shape and dtype as input.
        """
        _lib.require_same_device('RMSNorm', input, weight)
        lib = _lib.load()
        flattened_input = _lib.rows(input)
        batch_dim, feat_dim = flattened_input.shape
        eps = torch.finfo(input.dtype).eps if eps is None else eps

        output = torch.empty((batch_dim, feat_dim), device=input.device, dtype=input.dtype)
        scale_by_weight = weight is not None
        requires_grad = (input.requires_grad or
                         (scale_by_weight and weight.requires_grad))
        inv_rms = (torch.empty(batch_dim, device=input.device, dtype=torch.float32)
                   if requires_grad else None)
        weight_k = _param_for_kernel(weight, flattened_input)

        with _lib.device_guard(input):
            _lib.check(lib.at_rms_norm_fwd(
                _lib.ptr(flattened_input), _lib.ptr(weight_k), _lib.ptr(inv_rms), _lib.ptr(output),
                batch_dim, feat_dim, _lib.row_stride(flattened_input), _lib.row_stride(output), eps,
                _lib.dtype_id(input.dtype),
                _lib.dtype_id(weight_k.dtype) if scale_by_weight else 0,
                _lib.dtype_id(output.dtype), _lib.stream_of(input)), 'at_rms_norm_fwd')

        ctx.scale_by_weight = scale_by_weight
        if requires_grad:
            ctx.save_for_backward(flattened_input, inv_rms, weight)

        return output.view_as(input)

    @staticmethod
    @custom_bwd
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Input and weight gradients of root mean square normalization.
        """
        lib = _lib.load()
        scale_by_weight = ctx.scale_by_weight
        (flattened_input, inv_rms, weight) = ctx.saved_tensors
        _lib.require_same_device('RMSNorm backward', flattened_input, output_grad)
        flattened_output_grad = _lib.rows(output_grad.reshape(flattened_input.shape)
                                          .to(flattened_input.dtype))
        batch_dim, feat_dim = flattened_output_grad.shape
        device = flattened_input.device

        input_grad = torch.empty((batch_dim, feat_dim), device=device,
                                 dtype=flattened_output_grad.dtype)
        weight_grad = workspace = None
        workspace_bytes = 0
        if scale_by_weight:
            weight_grad = torch.empty(feat_dim, device=device, dtype=torch.float32)
            workspace_bytes = lib.at_norm_bwd_workspace_bytes(batch_dim, feat_dim, 1)
            workspace = torch.empty(workspace_bytes, device=device, dtype=torch.uint8)
        weight_k = _param_for_kernel(weight, flattened_input)

        with _lib.device_guard(flattened_input):
            _lib.check(lib.at_rms_norm_bwd(
                _lib.ptr(flattened_output_grad), _lib.ptr(flattened_input), _lib.ptr(inv_rms),
                _lib.ptr(weight_k), _lib.ptr(input_grad), _lib.ptr(weight_grad),
                _lib.ptr(workspace), workspace_bytes, batch_dim, feat_dim,
                _lib.row_stride(flattened_output_grad), _lib.row_stride(flattened_input),
                _lib.row_stride(input_grad),
                _lib.dtype_id(flattened_output_grad.dtype), _lib.dtype_id(flattened_input.dtype),
                _lib.dtype_id(weight_k.dtype) if scale_by_weight else 0,
                _lib.dtype_id(input_grad.dtype), _lib.stream_of(flattened_input)),
                'at_rms_norm_bwd')

        return input_grad.view_as(output_grad), weight_grad, None


class RMSNorm(nn.RMSNorm):
    """
    Root-mean-square-normalizes the input over its last dimension.
    See also base class; mirrors attorch/rms_norm_layer.py:137-168.

    Args:
        normalized_shape: Size of the last dimension (an integer).
        eps: Epsilon added under the square root; None selects
            torch.finfo(input.dtype).eps.
        elementwise_affine: Flag for a learnable scale.
        device: Device to use.
        dtype: Dtype of layer.
    """
    def __init__(
        self,
        normalized_shape: int,
        eps: Optional[float] = None,
        elementwise_affine: bool = True,
        device: Any = 'cuda',
        dtype: torch.dtype = torch.float32,
        ) -> None:
        if not isinstance(normalized_shape, int):
            raise RuntimeError('Normalized shape must be an integer.')

        super().__init__(normalized_shape, eps, elementwise_affine, device, dtype)

    def forward(self, input: Tensor) -> Tensor:
        return RMSNormAutoGrad.apply(input, self.weight, self.eps)
