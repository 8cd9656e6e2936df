"""
2D (and 1D) convolution with PyTorch autodiff support, running on the gfx950 implicit-GEMM
kernels.

API mirrors attorch/conv_layer.py: Conv2dAutoGrad.apply(input, weight, bias, stride_height,
stride_width, padding_height, padding_width, groups) and Conv1d / Conv2d modules (zero
padding, no dilation).  Unlike the reference, the backward pass (input gradient, weight
gradient, bias gradient) also runs on this library's kernels instead of torch.nn.grad.
"""

from typing import Any, Optional, Tuple, Union

import torch
from torch import Tensor
from torch import nn

from . import _lib
from .utils import get_output_dtype


def conv2d_output_size(
    in_size: int,
    kernel_size: int,
    stride: int,
    padding: int,
    ) -> int:
    """
    Output size of a convolution along one dimension (attorch/conv_layer.py:18-36).

    Args:
        in_size: Input size.
        kernel_size: Kernel size.
        stride: Stride.
        padding: Padding on each side.

    Returns:
        Output size.
    """
    return (in_size + 2 * padding - kernel_size) // stride + 1


def _workspace(n_bytes: int, device: torch.device) -> Tuple[Optional[Tensor], int]:
    """
    Scratch buffer of the size a kernel asked for (None when it asked for nothing).
    """
    if n_bytes <= 0:
        return None, 0
    return torch.empty(n_bytes, dtype=torch.uint8, device=device), n_bytes


class Conv2dAutoGrad(torch.autograd.Function):
    """
    Autodiff for 2D convolutional layer (attorch/conv_layer.py:39-164).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        weight: Tensor,
        bias: Optional[Tensor] = None,
        stride_height: int = 1,
        stride_width: int = 1,
        padding_height: int = 1,
        padding_width: int = 1,
        groups: int = 1,
        ) -> Tensor:
        """
        2D-convolves over the input using weights, optionally adding bias.

        Args:
            input: Input of shape [batch_dim, in_feat_dim, in_height, in_width].
            weight: Weights of shape [out_feat_dim, in_feat_dim / groups, kernel_height, kernel_width].
            bias: Optional bias of shape [out_feat_dim].
            stride_height: Stride over the height.
            stride_width: Stride over the width.
            padding_height: Zero padding on each side of the height.
            padding_width: Zero padding on each side of the width.
            groups: Number of groups.

        Returns:
            Output of shape [batch_dim, out_feat_dim, out_height, out_width].
        """
        assert weight.ndim == 4, \
            f'Weights must be 4D, received shape {weight.shape}'
        assert bias is None or bias.ndim == 1, \
            f'Bias must be 1D, received shape {bias.shape}'

        assert input.shape[1] == groups * weight.shape[1], \
            f'Incompatible input ({input.shape}) and weights ({weight.shape}) shape with {groups} groups'
        assert bias is None or weight.shape[0] == bias.shape[0], \
            f'Incompatible weights ({weight.shape}) and bias ({bias.shape}) shape'

        _lib.require_same_device('Conv2d', input, weight, bias)
        lib = _lib.load()
        batch_dim, in_feat_dim, in_height, in_width = input.shape
        out_feat_dim, _, kernel_height, kernel_width = weight.shape
        out_height = conv2d_output_size(in_height, kernel_height,
                                        stride_height, padding_height)
        out_width = conv2d_output_size(in_width, kernel_width,
                                       stride_width, padding_width)

        output_dtype = get_output_dtype(input.dtype, autocast='fp16')
        # Under autocast the operands are rounded to the low-precision dtype first
        # (conv_kernels.py:191-193).
        weight_k = weight.to(output_dtype).contiguous()
        bias_k = None if bias is None else bias.to(output_dtype).contiguous()
        dims = (batch_dim, in_feat_dim, in_height, in_width, out_feat_dim, out_height, out_width,
                kernel_height, kernel_width, stride_height, stride_width,
                padding_height, padding_width, groups)

        dtype = _lib.dtype_id(output_dtype)
        requires_grad = (input.requires_grad or
                         weight.requires_grad or
                         (bias is not None and bias.requires_grad))
        ctx.dims = dims
        ctx.bias_requires_grad = False if bias is None else bias.requires_grad
        ctx.output_dtype = output_dtype
        ctx.input_nhwc = None

        # Tensors that are channels-last in memory (torch.channels_last) are what the matrix-core
        # kernels read and write: no layout copies, and the output is channels-last too.
        ctx.channels_last = (input.dtype is output_dtype and not input.is_contiguous()
                             and input.is_contiguous(memory_format=torch.channels_last)
                             and lib.at_conv2d_nhwc_workspace_bytes(0, *dims, dtype) > 0)
        if ctx.channels_last:
            output = torch.empty((batch_dim, out_feat_dim, out_height, out_width), device=input.device,
                                 dtype=output_dtype, memory_format=torch.channels_last)
            with _lib.device_guard(input):
                workspace, workspace_bytes = _workspace(
                    lib.at_conv2d_nhwc_workspace_bytes(0, *dims, dtype), input.device)
                _lib.check(lib.at_conv2d_fwd_nhwc(
                    _lib.ptr(input), _lib.ptr(weight_k), _lib.ptr(bias_k), _lib.ptr(output),
                    _lib.ptr(workspace), workspace_bytes, *dims, dtype, dtype,
                    _lib.stream_of(input)), 'at_conv2d_fwd_nhwc')
            if requires_grad:
                ctx.save_for_backward(input, weight)
            return output

        input_k = input.to(output_dtype).contiguous()
        output = torch.empty((batch_dim, out_feat_dim, out_height, out_width),
                             device=input.device, dtype=output_dtype)
        with _lib.device_guard(input):
            workspace, workspace_bytes = _workspace(
                lib.at_conv2d_fwd_workspace_bytes(*dims, dtype, dtype), input.device)
            _lib.check(lib.at_conv2d_fwd(
                _lib.ptr(input_k), _lib.ptr(weight_k), _lib.ptr(bias_k), _lib.ptr(output),
                _lib.ptr(workspace), workspace_bytes, *dims, dtype, dtype, dtype,
                _lib.stream_of(input)), 'at_conv2d_fwd')

        # The matrix-core path leaves a channels-last copy of the input at the start of its
        # workspace (unless it had to pad the channels); the weight gradient reuses it instead of
        # transposing the input again.
        keep = (requires_grad and weight.requires_grad and workspace is not None
                and lib.at_conv2d_fwd_leaves_nhwc(*dims, dtype, dtype) == 1)
        ctx.input_nhwc = workspace if keep else None
        if requires_grad:
            # under autocast the weight gradient reads the low-precision copy made above
            # (conv_layer.py:150-151 casts the saved input again): keep that copy
            ctx.save_for_backward(input_k if input_k.dtype is not input.dtype else input, weight)

        return output

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Gradients of the convolution with respect to input, weight and bias, all in the
        output dtype (attorch/conv_layer.py:147-162).
        """
        lib = _lib.load()
        input, weight = ctx.saved_tensors
        _lib.require_same_device('Conv2d backward', input, output_grad)
        output_dtype = ctx.output_dtype
        device = input.device
        dims = ctx.dims
        (batch_dim, in_feat_dim, _, _, out_feat_dim, out_height, out_width,
         kernel_height, kernel_width, _, _, _, _, groups) = dims
        stream = _lib.stream_of(input)
        dtype = _lib.dtype_id(output_dtype)

        input_grad = weight_grad = bias_grad = None
        if ctx.channels_last:
            # channels-last gradients in and out; a product this path does not cover is left to
            # the channels-first code below
            grad_last = _lib.in_memory_format(output_grad.to(output_dtype), torch.channels_last)
            need_input = ctx.needs_input_grad[0]
            need_weight = ctx.needs_input_grad[1]
            with _lib.device_guard(input):
                n_bytes = lib.at_conv2d_nhwc_workspace_bytes(1, *dims, dtype) if need_input else 0
                if n_bytes > 0:
                    weight_k = weight.to(output_dtype).contiguous()
                    input_grad = torch.empty(input.shape, dtype=output_dtype, device=device,
                                             memory_format=torch.channels_last)
                    workspace, workspace_bytes = _workspace(n_bytes, device)
                    _lib.check(lib.at_conv2d_bwd_input_nhwc(
                        _lib.ptr(grad_last), _lib.ptr(weight_k), _lib.ptr(input_grad),
                        _lib.ptr(workspace), workspace_bytes, *dims, dtype, stream),
                        'at_conv2d_bwd_input_nhwc')
                    need_input = False
                n_bytes = lib.at_conv2d_nhwc_workspace_bytes(2, *dims, dtype) if need_weight else 0
                if n_bytes > 0:
                    weight_grad = torch.empty(weight.shape, dtype=output_dtype, device=device)
                    workspace, workspace_bytes = _workspace(n_bytes, device)
                    _lib.check(lib.at_conv2d_bwd_weight_nhwc(
                        _lib.ptr(grad_last), _lib.ptr(input), _lib.ptr(weight_grad),
                        _lib.ptr(workspace), workspace_bytes, *dims, dtype, stream),
                        'at_conv2d_bwd_weight_nhwc')
                    need_weight = False
                if ctx.bias_requires_grad:
                    # the bias gradient: column sums of the [batch * height * width, out_feat] matrix
                    rows = batch_dim * out_height * out_width
                    bias_grad = torch.empty(out_feat_dim, dtype=output_dtype, device=device)
                    workspace, workspace_bytes = _workspace(
                        lib.at_colsum_workspace_bytes(rows, out_feat_dim), device)
                    _lib.check(lib.at_colsum(
                        _lib.ptr(grad_last), _lib.ptr(bias_grad), _lib.ptr(workspace), workspace_bytes,
                        rows, out_feat_dim, out_feat_dim, dtype, dtype, stream), 'at_colsum')
            if not (need_input or need_weight):
                return input_grad, weight_grad, bias_grad, None, None, None, None, None
            rest = Conv2dAutoGrad._backward_channels_first(
                ctx, input, weight, output_grad, need_input, need_weight, False)
            return (input_grad if input_grad is not None else rest[0],
                    weight_grad if weight_grad is not None else rest[1], bias_grad,
                    None, None, None, None, None)
        return Conv2dAutoGrad._backward_channels_first(
            ctx, input, weight, output_grad, ctx.needs_input_grad[0], ctx.needs_input_grad[1],
            ctx.bias_requires_grad)

    @staticmethod
    def _backward_channels_first(
        ctx: Any,
        input: Tensor,
        weight: Tensor,
        output_grad: Tensor,
        need_input: bool,
        need_weight: bool,
        need_bias: bool,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        The three gradients from contiguous [batch, feat, height, width] tensors.
        """
        lib = _lib.load()
        output_dtype = ctx.output_dtype
        device = input.device
        dims = ctx.dims
        (batch_dim, in_feat_dim, _, _, out_feat_dim, out_height, out_width,
         kernel_height, kernel_width, _, _, _, _, groups) = dims
        output_grad = output_grad.to(output_dtype).contiguous()
        stream = _lib.stream_of(input)
        dtype = _lib.dtype_id(output_dtype)

        input_grad = weight_grad = bias_grad = None
        with _lib.device_guard(input):
            input_workspace_bytes = (lib.at_conv2d_bwd_input_workspace_bytes(*dims, dtype)
                                     if need_input else 0)
            # one channels-last copy of the output gradient serves both products
            output_grad_nhwc = None
            if input_workspace_bytes > 0 and need_weight:
                output_grad_nhwc = torch.empty_like(output_grad)
                _lib.check(lib.at_nchw_to_nhwc(
                    _lib.ptr(output_grad), _lib.ptr(output_grad_nhwc), batch_dim, out_feat_dim,
                    out_height * out_width, dtype, stream), 'at_nchw_to_nhwc')
            if need_input:
                weight_k = weight.to(output_dtype).contiguous()
                input_grad = torch.empty(input.shape, dtype=output_dtype, device=device)
                workspace, workspace_bytes = _workspace(input_workspace_bytes, device)
                _lib.check(lib.at_conv2d_bwd_input(
                    _lib.ptr(output_grad), _lib.ptr(output_grad_nhwc), _lib.ptr(weight_k),
                    _lib.ptr(input_grad), _lib.ptr(workspace), workspace_bytes, *dims, dtype,
                    stream), 'at_conv2d_bwd_input')
            if need_weight:
                input_k = input.to(output_dtype).contiguous()
                weight_grad = torch.empty(weight.shape, dtype=output_dtype, device=device)
                workspace, workspace_bytes = _workspace(
                    lib.at_conv2d_bwd_weight_workspace_bytes(*dims, dtype), device)
                _lib.check(lib.at_conv2d_bwd_weight(
                    _lib.ptr(output_grad), _lib.ptr(output_grad_nhwc), _lib.ptr(input_k),
                    _lib.ptr(ctx.input_nhwc), _lib.ptr(weight_grad),
                    _lib.ptr(workspace), workspace_bytes, *dims, dtype, stream),
                    'at_conv2d_bwd_weight')
            if need_bias:
                bias_grad = torch.empty(out_feat_dim, dtype=output_dtype, device=device)
                if output_grad_nhwc is not None:
                    # the channels-last copy is a [batch * height * width, out_feat] matrix:
                    # its column sums use the whole GPU whatever the channel count
                    rows = batch_dim * out_height * out_width
                    workspace, workspace_bytes = _workspace(
                        lib.at_colsum_workspace_bytes(rows, out_feat_dim), device)
                    _lib.check(lib.at_colsum(
                        _lib.ptr(output_grad_nhwc), _lib.ptr(bias_grad), _lib.ptr(workspace),
                        workspace_bytes, rows, out_feat_dim, out_feat_dim, dtype, dtype,
                        stream), 'at_colsum')
                else:
                    _lib.check(lib.at_channel_sum(
                        _lib.ptr(output_grad), _lib.ptr(bias_grad), batch_dim, out_feat_dim,
                        out_height * out_width, dtype, dtype, stream), 'at_channel_sum')

        return input_grad, weight_grad, bias_grad, None, None, None, None, None


class Conv1d(nn.Conv1d):
    """
    1D-convolves over the input using weights, optionally adding bias.
    See also base class; mirrors attorch/conv_layer.py:167-220.

    Args:
        in_channels: Number of input channels.
        out_channels: Number of output channels.
        kernel_size: Kernel size.
        stride: Stride of kernel.
        padding: Padding applied to the input.
        dilation: Dilation of kernel. Only 1 is supported.
        groups: Number of groups for the convolution.
        bias: Flag for additive bias.
        padding_mode: Padding mode. Only 'zeros' is supported.
        device: Device to use.
        dtype: Dtype of layer.
    """
    def __init__(
        self,
        in_channels: int,
        out_channels: int,
        kernel_size: int,
        stride: int = 1,
        padding: int = 0,
        dilation: int = 1,
        groups: int = 1,
        bias: bool = True,
        padding_mode: str = 'zeros',
        device: Any = 'cuda',
        dtype: torch.dtype = torch.float32,
        ) -> None:
        super().__init__(in_channels, out_channels, kernel_size, stride, padding,
                         dilation, groups, bias, padding_mode, device, dtype)

        if self.dilation != (1,):
            raise RuntimeError('Convolutional layer only supports dilation of 1.')

        if self.padding_mode != 'zeros':
            raise RuntimeError("Convolutional layer only support 'zeros' padding mode.")

    def forward(self, input: Tensor) -> Tensor:
        return Conv2dAutoGrad.apply(input.unsqueeze(-1), self.weight.unsqueeze(-1),
                                    self.bias,
                                    *self.stride, 1, *self.padding, 0,
                                    self.groups).squeeze(-1)


class Conv2d(nn.Conv2d):
    """
    2D-convolves over the input using weights, optionally adding bias.
    See also base class; mirrors attorch/conv_layer.py:223-278.

    Args:
        in_channels: Number of input channels.
        out_channels: Number of output channels.
        kernel_size: Kernel size.
        stride: Stride of kernel.
        padding: Padding applied to the input.
        dilation: Dilation of kernel. Only 1 and (1, 1) are supported.
        groups: Number of groups for the convolution.
        bias: Flag for additive bias.
        padding_mode: Padding mode. Only 'zeros' is supported.
        device: Device to use.
        dtype: Dtype of layer.
    """
    def __init__(
        self,
        in_channels: int,
        out_channels: int,
        kernel_size: Union[int, Tuple[int, int]],
        stride: Union[int, Tuple[int, int]] = 1,
        padding: Union[int, Tuple[int, int]] = 0,
        dilation: Union[int, Tuple[int, int]] = 1,
        groups: int = 1,
        bias: bool = True,
        padding_mode: str = 'zeros',
        device: Any = 'cuda',
        dtype: torch.dtype = torch.float32,
        ) -> None:
        super().__init__(in_channels, out_channels, kernel_size, stride, padding,
                         dilation, groups, bias, padding_mode, device, dtype)

        if self.dilation != (1, 1):
            raise RuntimeError('Convolutional layer only supports dilation of 1 and (1, 1).')

        if self.padding_mode != 'zeros':
            raise RuntimeError("Convolutional layer only support 'zeros' padding mode.")

    def forward(self, input: Tensor) -> Tensor:
        return Conv2dAutoGrad.apply(input, self.weight, self.bias,
                                    *self.stride, *self.padding,
                                    self.groups)
