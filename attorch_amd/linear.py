"""
Linear layer with fused bias and activation with PyTorch autodiff support, running on the
gfx950 MFMA GEMM kernels.

API mirrors attorch/linear_layer.py: the weight is stored [in_features, out_features], the
forward pass fuses bias + activation (saving the pre-activation only when a gradient is
needed), and backward returns gradients for (input, weight, bias, act_func).  Unlike the
reference, the two backward matrix products and the bias column sum also run on this
library's kernels instead of torch's.
"""

from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn
from torch.nn import functional as F

from . import _lib
from .act import act_id, parse_act_func
from .utils import get_output_dtype


def _matrix(tensor: Tensor) -> Tensor:
    """
    2D view with unit inner stride (copies only when the layout requires it).
    """
    if tensor.stride(-1) != 1 or (tensor.shape[0] > 1 and tensor.stride(0) < tensor.shape[1]):
        tensor = tensor.contiguous()
    return tensor


def _round_up8(size: int) -> int:
    return (size + 7) // 8 * 8


def _pad_features(batch_dim: int, in_feat_dim: int, out_feat_dim: int, dtype: torch.dtype) -> bool:
    """
    Whether the 16-bit operands get zero-padded copies with feature strides in multiples of 8.

    The tiled matrix-core kernels read 16 bytes at a time and need 16-byte aligned rows; other
    shapes run on the generic kernel, which is several times slower on large problems (a
    vocabulary of 50257 columns, say).  Copying the operands costs one pass over each, far
    less than the difference, once the problem is large enough for those kernels at all.
    """
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    if in_feat_dim % 8 == 0 and out_feat_dim % 8 == 0:
        return False
    return (min(batch_dim, in_feat_dim, out_feat_dim) >= 64 and
            batch_dim * min(in_feat_dim, out_feat_dim) >= 32768)


def _zero_pad(matrix: Tensor, rows: int, cols: int) -> Tensor:
    """
    Copy of a 2D tensor extended with zeros to [rows, cols] (the tensor itself if it fits already).
    """
    if matrix.shape == (rows, cols):
        return matrix
    return F.pad(matrix, (0, cols - matrix.shape[1], 0, rows - matrix.shape[0]))


class LinearAutoGrad(torch.autograd.Function):
    """
    Autodiff for linear layer (attorch/linear_layer.py:19-161).
    """
    @staticmethod
    def forward(
        ctx: Any,
        input: Tensor,
        weight: Tensor,
        bias: Optional[Tensor] = None,
        act_func: Optional[str] = None,
        ) -> Tensor:
        """
        Linearly transforms the input using weights, optionally adding bias
        and fusing an activation function.

        Args:
            input: Input of shape [..., in_feat_dim].
            weight: Weights of shape [in_feat_dim, out_feat_dim].
            bias: Optional bias of shape [out_feat_dim].
            act_func: Activation name, None for identity: 'sigmoid', 'logsigmoid', 'tanh',
                'relu', 'gelu', 'geluapprox', 'silu', 'relu6', 'hardsigmoid', 'hardtanh',
                'hardswish', 'selu', 'mish', 'softplus', 'softsign', 'tanhshrink',
                'leaky_relu_PARAM', 'elu_PARAM', 'celu_PARAM', 'hardshrink_PARAM',
                'softshrink_PARAM'.

        Returns:
            Transformed input of shape [..., out_feat_dim].
        """
        assert weight.ndim == 2, \
            f'Weights must be 2D, received shape {weight.shape}'
        assert bias is None or bias.ndim == 1, \
            f'Bias must be 1D, received shape {bias.shape}'

        assert input.shape[-1] == weight.shape[0], \
            f'Incompatible input ({input.shape}) and weights ({weight.shape}) shape'
        assert bias is None or weight.shape[1] == bias.shape[0], \
            f'Incompatible weights ({weight.shape}) and bias ({bias.shape}) shape'

        _lib.require_same_device('Linear', input, weight, bias)
        lib = _lib.load()
        act_func, param = parse_act_func(act_func)
        act = act_id(act_func, param)

        flattened_input = input.flatten(0, -2)
        batch_dim, in_feat_dim = flattened_input.shape
        _, out_feat_dim = weight.shape

        requires_grad = (input.requires_grad or
                         weight.requires_grad or
                         (bias is not None and bias.requires_grad))
        save_pre_act = requires_grad and (act_func is not None)

        output_dtype = get_output_dtype(input.dtype, autocast='fp16')
        # Under autocast the operands are rounded to the low-precision dtype before the
        # product (linear_kernels.py:161-163); otherwise input and weight share a dtype.
        compute_dtype = output_dtype if output_dtype != input.dtype else input.dtype
        input_k = _matrix(flattened_input.to(compute_dtype))
        weight_k = _matrix(weight.to(compute_dtype))
        bias_k = None if bias is None else bias.contiguous()
        if bias_k is not None and output_dtype != input.dtype:
            bias_k = bias_k.to(output_dtype)
        contract_dim = in_feat_dim
        padded_weight = None
        if _pad_features(batch_dim, in_feat_dim, out_feat_dim, compute_dtype):
            # zeros along the contraction add nothing; padded output columns are never stored
            contract_dim = _round_up8(in_feat_dim)
            input_k = _zero_pad(input_k, batch_dim, contract_dim)
            weight_k = _zero_pad(weight_k, contract_dim, _round_up8(out_feat_dim))
            if input.requires_grad:
                # the input gradient multiplies by the same padded copy: keep it instead of
                # padding the weight a second time (one more weight-sized buffer alive between
                # forward and backward; it travels with the saved tensors, so hooks see it)
                padded_weight = weight_k

        output = torch.empty((batch_dim, out_feat_dim), device=input.device, dtype=output_dtype)
        if save_pre_act and padded_weight is not None and out_feat_dim % 8:
            # the saved pre-activation gets rows that start on 16-byte boundaries (row stride
            # rounded up, the spare columns zero): the kernels then write and later read it in
            # whole vectors
            padded = torch.empty((batch_dim, _round_up8(out_feat_dim)), device=input.device, dtype=output_dtype)
            padded[:, out_feat_dim:].zero_()
            pre_act = padded[:, :out_feat_dim]
        else:
            pre_act = torch.empty_like(output) if save_pre_act else output

        with _lib.device_guard(input):
            _lib.check(lib.at_linear_fwd(
                _lib.ptr(input_k), _lib.ptr(weight_k), _lib.ptr(bias_k), _lib.ptr(pre_act),
                _lib.ptr(output), batch_dim, contract_dim, out_feat_dim, _lib.row_stride(input_k),
                _lib.row_stride(weight_k), _lib.row_stride(pre_act), _lib.row_stride(output), act,
                0.0 if param is None else param, _lib.dtype_id(compute_dtype),
                _lib.dtype_id(bias_k.dtype) if bias_k is not None else 0,
                _lib.dtype_id(output_dtype), _lib.stream_of(input)), 'at_linear_fwd')

        ctx.param = param
        ctx.act_func = act_func
        ctx.act = act
        ctx.bias_requires_grad = False if bias is None else bias.requires_grad
        ctx.output_dtype = output_dtype
        ctx.input_shape = input.shape
        ctx.leaf_dtypes = (input.dtype, weight.dtype)
        if requires_grad:
            # Under autocast the low-precision copies made for the forward product are what the
            # backward products read (linear_layer.py:152-155 casts them again there): keeping
            # them costs one cast per operand and step instead of two.  Copies that were
            # zero-padded are not kept (the padded weight aside): backward pads afresh.
            cast = compute_dtype != input.dtype or compute_dtype != weight.dtype
            keep_input = (input_k if cast and input_k.shape[1] == in_feat_dim and weight.requires_grad
                          else flattened_input)
            keep_weight = (weight_k if cast and weight_k.shape == weight.shape and input.requires_grad
                           else weight)
            ctx.save_for_backward(keep_input, pre_act if save_pre_act else None, keep_weight, padded_weight)

        return output.view(*input.shape[:-1], out_feat_dim)

    @staticmethod
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Gradients of the linear layer with respect to input, weight and bias.
        """
        lib = _lib.load()
        flattened_input, pre_act, weight, padded_weight = ctx.saved_tensors
        _lib.require_same_device('Linear backward', flattened_input, output_grad)
        output_dtype = ctx.output_dtype
        device = flattened_input.device
        input_needs_grad, weight_needs_grad = ctx.needs_input_grad[0], ctx.needs_input_grad[1]

        output_grad = _matrix(output_grad.flatten(0, -2))
        batch_dim, in_feat_dim = flattened_input.shape
        _, out_feat_dim = weight.shape
        stream = _lib.stream_of(flattened_input)

        if (weight_needs_grad and output_dtype is torch.float32
                and output_grad.dtype is torch.float32 and flattened_input.dtype is torch.float32
                and weight.dtype is torch.float32 and (pre_act is None or pre_act.dtype is torch.float32)
                and lib.at_linear_bwd_small_supported(batch_dim, in_feat_dim, out_feat_dim,
                                                      _lib.dtype_id(torch.float32))):
            # small fp32 layer: activation gradient, both products and the bias sum in one launch.
            # The kernel always forms the weight gradient (a workgroup's tile of it is what its
            # waves share), so a frozen weight takes the separate launches below instead.
            input_mm, weight_mm = _matrix(flattened_input), _matrix(weight)
            pre_act_mm = None if ctx.act_func is None else _matrix(pre_act)
            operands = [output_grad, input_mm, weight_mm] + ([] if pre_act_mm is None else [pre_act_mm])
            if all(t.data_ptr() % 16 == 0 and _lib.row_stride(t) % 4 == 0 for t in operands):
                input_grad = (torch.empty((batch_dim, in_feat_dim), dtype=output_dtype, device=device)
                              if input_needs_grad else None)
                weight_grad = torch.empty((in_feat_dim, out_feat_dim), dtype=output_dtype, device=device)
                bias_grad = (torch.empty(out_feat_dim, dtype=output_dtype, device=device)
                             if ctx.bias_requires_grad else None)
                with _lib.device_guard(flattened_input):
                    _lib.check(lib.at_linear_bwd_small(
                        _lib.ptr(output_grad), _lib.ptr(pre_act_mm), _lib.ptr(input_mm), _lib.ptr(weight_mm),
                        _lib.ptr(input_grad), _lib.ptr(weight_grad), _lib.ptr(bias_grad), batch_dim,
                        in_feat_dim, out_feat_dim, _lib.row_stride(output_grad),
                        0 if pre_act_mm is None else _lib.row_stride(pre_act_mm), _lib.row_stride(input_mm),
                        _lib.row_stride(weight_mm), in_feat_dim, out_feat_dim,
                        ctx.act if ctx.act_func is not None else 0,
                        0.0 if ctx.param is None else ctx.param, _lib.dtype_id(torch.float32), stream),
                        'at_linear_bwd_small')
                if input_grad is not None:
                    input_grad = input_grad.view(ctx.input_shape)
                return input_grad, weight_grad, bias_grad, None

        with _lib.device_guard(flattened_input):
            bias_grad = None
            padded_cols = _round_up8(out_feat_dim)
            # set only where this function itself allocates a gradient buffer whose rows are
            # zero-padded to whole vectors; never inferred from a tensor's strides
            padded_grad = None
            if ctx.act_func is None:
                pre_act_grad = output_grad
            elif (pre_act.stride(0) == padded_cols and padded_cols != out_feat_dim
                  and output_grad.dtype is pre_act.dtype):
                # rows of the saved pre-activation are padded to whole vectors (see forward): one
                # zero-padded copy of the output gradient lets the activation gradient run on whole
                # vectors too, and its result is the padded operand both products need
                output_grad_p = _zero_pad(output_grad, batch_dim, padded_cols)
                pre_act_grad_p = torch.empty((batch_dim, padded_cols), dtype=pre_act.dtype, device=device)
                bias_grad_p = workspace = None
                workspace_bytes = 0
                if ctx.bias_requires_grad:
                    bias_grad_p = torch.empty(padded_cols, dtype=pre_act.dtype, device=device)
                    workspace_bytes = lib.at_act_bwd_workspace_bytes(batch_dim, padded_cols)
                    workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device)
                _lib.check(lib.at_act_bwd(
                    _lib.ptr(output_grad_p), _lib.ptr(pre_act), _lib.ptr(pre_act_grad_p),
                    _lib.ptr(bias_grad_p), _lib.ptr(workspace), workspace_bytes,
                    batch_dim, padded_cols, padded_cols, padded_cols, padded_cols, ctx.act,
                    0.0 if ctx.param is None else ctx.param, _lib.dtype_id(pre_act.dtype),
                    _lib.dtype_id(pre_act.dtype), _lib.dtype_id(pre_act.dtype), stream), 'at_act_bwd')
                pre_act_grad = pre_act_grad_p[:, :out_feat_dim]
                padded_grad = pre_act_grad_p
                if bias_grad_p is not None:
                    bias_grad = bias_grad_p[:out_feat_dim].clone()
            else:
                pre_act_grad = torch.empty((batch_dim, out_feat_dim), dtype=pre_act.dtype,
                                           device=device)
                # the bias gradient (column sums of pre_act_grad) comes out of the same pass
                fuse_bias = ctx.bias_requires_grad and batch_dim > 0
                workspace = workspace_bytes = None
                if fuse_bias:
                    bias_grad = torch.empty(out_feat_dim, dtype=pre_act.dtype, device=device)
                    workspace_bytes = lib.at_act_bwd_workspace_bytes(batch_dim, out_feat_dim)
                    workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device)
                _lib.check(lib.at_act_bwd(
                    _lib.ptr(output_grad), _lib.ptr(pre_act), _lib.ptr(pre_act_grad),
                    _lib.ptr(bias_grad), _lib.ptr(workspace), workspace_bytes or 0,
                    batch_dim, out_feat_dim, _lib.row_stride(output_grad), _lib.row_stride(pre_act),
                    _lib.row_stride(pre_act_grad), ctx.act, 0.0 if ctx.param is None else ctx.param,
                    _lib.dtype_id(output_grad.dtype), _lib.dtype_id(pre_act.dtype),
                    _lib.dtype_id(pre_act.dtype), stream), 'at_act_bwd')

            # The products run in the output dtype, as under the reference's
            # torch.autocast(dtype=output_dtype) block (linear_layer.py:152-155).
            grad_mm = _matrix(pre_act_grad.to(output_dtype))
            pad = _pad_features(batch_dim, in_feat_dim, out_feat_dim, output_dtype)
            contract_dim = out_feat_dim
            if pad:
                contract_dim = _round_up8(out_feat_dim)
                if padded_grad is not None and padded_grad.dtype is output_dtype:
                    grad_mm = padded_grad
                else:
                    grad_mm = _zero_pad(grad_mm, batch_dim, contract_dim)
            # Gradients of float32 tensors that took part in 16-bit products (autocast): the
            # kernels write the 16-bit result widened to float32 themselves, which spares
            # autograd's cast pass over each gradient.
            wide = (not pad and output_dtype is not torch.float32 and batch_dim > 0
                    and bool(lib.at_linear_bwd_wide_output_supported(batch_dim, in_feat_dim, out_feat_dim,
                                                                     _lib.dtype_id(output_dtype))))
            input_grad_dtype = torch.float32 if wide and ctx.leaf_dtypes[0] is torch.float32 else output_dtype
            weight_grad_dtype = torch.float32 if wide and ctx.leaf_dtypes[1] is torch.float32 else output_dtype
            input_grad = weight_grad = None
            if input_needs_grad:
                if pad and padded_weight is not None and padded_weight.dtype is output_dtype:
                    weight_mm = padded_weight
                else:
                    weight_mm = _matrix(weight.to(output_dtype))
                    if pad:
                        weight_mm = _zero_pad(weight_mm, in_feat_dim, contract_dim)
                input_grad = torch.empty((batch_dim, in_feat_dim), dtype=input_grad_dtype, device=device)
                _lib.check(lib.at_linear_bwd_input(
                    _lib.ptr(grad_mm), _lib.ptr(weight_mm), _lib.ptr(input_grad), batch_dim,
                    in_feat_dim, contract_dim, _lib.row_stride(grad_mm), _lib.row_stride(weight_mm),
                    _lib.row_stride(input_grad), _lib.dtype_id(output_dtype),
                    _lib.dtype_id(input_grad_dtype), stream), 'at_linear_bwd_input')
                input_grad = input_grad.view(ctx.input_shape)
            if weight_needs_grad:
                input_mm = _matrix(flattened_input.to(output_dtype))
                if pad:
                    input_mm = _zero_pad(input_mm, batch_dim, _round_up8(in_feat_dim))
                weight_grad = torch.empty((in_feat_dim, out_feat_dim), dtype=weight_grad_dtype,
                                          device=device)
                if batch_dim == 0:
                    weight_grad.zero_()
                else:
                    workspace_bytes = lib.at_linear_bwd_weight_workspace_bytes(
                        batch_dim, in_feat_dim, out_feat_dim, _lib.dtype_id(output_dtype))
                    workspace = (torch.empty(workspace_bytes, dtype=torch.uint8, device=device)
                                 if workspace_bytes else None)
                    _lib.check(lib.at_linear_bwd_weight(
                        _lib.ptr(input_mm), _lib.ptr(grad_mm), _lib.ptr(weight_grad),
                        _lib.ptr(workspace), workspace_bytes, batch_dim,
                        in_feat_dim, out_feat_dim, _lib.row_stride(input_mm), _lib.row_stride(grad_mm),
                        _lib.row_stride(weight_grad), _lib.dtype_id(output_dtype),
                        _lib.dtype_id(weight_grad_dtype), stream), 'at_linear_bwd_weight')
            if ctx.bias_requires_grad and bias_grad is None:
                bias_grad = torch.empty(out_feat_dim, dtype=pre_act_grad.dtype, device=device)
                if batch_dim == 0:
                    bias_grad.zero_()
                else:
                    workspace_bytes = lib.at_colsum_workspace_bytes(batch_dim, out_feat_dim)
                    workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device)
                    _lib.check(lib.at_colsum(
                        _lib.ptr(pre_act_grad), _lib.ptr(bias_grad), _lib.ptr(workspace),
                        workspace_bytes, batch_dim, out_feat_dim, _lib.row_stride(pre_act_grad),
                        _lib.dtype_id(pre_act_grad.dtype), _lib.dtype_id(bias_grad.dtype), stream),
                        'at_colsum')

        # One gradient (or None) per forward argument.
        return input_grad, weight_grad, bias_grad, None


class Linear(nn.Linear):
    """
    Linearly transforms the input using weights, optionally adding bias
    and fusing an activation function.
    See also base class; mirrors attorch/linear_layer.py:164-205.

    Note: the weight matrix of this module has shape [in_features, out_features], not
    torch's [out_features, in_features].

    Args:
        in_features: Number of input features.
        out_features: Number of output features.
        bias: Flag for additive bias.
        act_func: Name of activation function to apply, with None for identity
            (see LinearAutoGrad.forward for the options).
        device: Device to use.
        dtype: Dtype of layer.
    """
    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = True,
        act_func: Optional[str] = None,
        device: Any = 'cuda',
        dtype: torch.dtype = torch.float32,
        ) -> None:
        super().__init__(in_features, out_features, bias, device, dtype)
        self.weight = nn.Parameter(self.weight.T.contiguous())
        self.act_func = act_func

    def forward(self, input: Tensor) -> Tensor:
        return LinearAutoGrad.apply(input, self.weight, self.bias,
                                    self.act_func)
