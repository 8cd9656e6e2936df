"""
Activation function layers with fused dropout, and the Dropout layer, with PyTorch autodiff
support, running on the gfx950 elementwise kernels of libattorch_hip.so.

API mirrors attorch/act_layers.py and attorch/dropout_layer.py: ActFuncAutoGrad.apply(input,
act_func, drop_p, training), DropoutAutoGrad.apply(input, drop_p, training), and one
nn.Module subclass per activation taking `drop_p` (plus the dummy `inplace` arguments).
"""

import warnings
from random import randint
from typing import Any, Optional, Tuple

import torch
from torch import Tensor
from torch import nn
from torch.amp import custom_fwd

from . import _lib
from .utils import custom_bwd
from .act import act_id, parse_act_func


def _launch_forward(input: Tensor, act: int, param: float, drop_p: float, seed: int) -> Tensor:
    flattened_input = input.contiguous().view(-1)
    output = torch.empty_like(flattened_input)
    with _lib.device_guard(input):
        _lib.check(_lib.load().at_act_dropout_fwd(
            _lib.ptr(flattened_input), _lib.ptr(output), flattened_input.numel(), act, param,
            drop_p, seed, _lib.dtype_id(input.dtype), _lib.stream_of(input)),
            'at_act_dropout_fwd')
    return output.view(input.shape)


def _launch_backward(output_grad: Tensor, input: Optional[Tensor], act: int, param: float,
                     drop_p: float, seed: int) -> Tensor:
    reference = output_grad if input is None else input
    _lib.require_same_device('activation / dropout backward', output_grad, input)
    flattened_grad = output_grad.to(reference.dtype).contiguous().view(-1)
    flattened_input = None if input is None else input.contiguous().view(-1)
    input_grad = torch.empty_like(flattened_grad)
    with _lib.device_guard(output_grad):
        _lib.check(_lib.load().at_act_dropout_bwd(
            _lib.ptr(flattened_grad), _lib.ptr(flattened_input), _lib.ptr(input_grad),
            flattened_grad.numel(), act, param, drop_p, seed, _lib.dtype_id(reference.dtype),
            _lib.stream_of(output_grad)), 'at_act_dropout_bwd')
    return input_grad.view(reference.shape)


class ActFuncAutoGrad(torch.autograd.Function):
    """
    Autodiff for activation functions (attorch/act_layers.py:20-117).
    """
    @staticmethod
    @custom_fwd(device_type='cuda')
    def forward(
        ctx: Any,
        input: Tensor,
        act_func: str,
        drop_p: float,
        training: bool,
        ) -> Tensor:
        """
        Applies an activation function to the input, optionally fusing dropout.

        Args:
            ctx: Context for variable storage.
            input: Input to transform.
                Can have arbitrary shape.
            act_func: Name of activation function to apply.
                Options are 'sigmoid', 'logsigmoid', 'tanh', 'relu', 'gelu', 'geluapprox',
                'silu', 'relu6', 'hardsigmoid', 'hardtanh', 'hardswish', 'selu', 'mish',
                'softplus', 'softsign', 'tanhshrink', 'leaky_relu_PARAM', 'elu_PARAM',
                'celu_PARAM', 'hardshrink_PARAM' and 'softshrink_PARAM'.
            drop_p: Probability of dropping an element for dropout.
            training: Flag indicating if the model is in training mode,
                only applicable if drop_p is greater than 0.

        Returns:
            Input transformed by the desired activation function,
            potentially with fused dropout.
        """
        _lib.require_gpu(input, 'activation layer')
        name, param = parse_act_func(act_func)
        ctx.act = act_id(name, param)
        ctx.param = 0.0 if param is None else param
        dropout = drop_p > 0 and training
        ctx.drop_p = float(drop_p) if dropout else 0.0
        # same seed range as the reference (act_layers.py:66)
        ctx.seed = randint(0, 65535) if dropout else 0
        if input.requires_grad:
            ctx.save_for_backward(input)
        return _launch_forward(input, ctx.act, ctx.param, ctx.drop_p, ctx.seed)

    @staticmethod
    @custom_bwd
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Calculates the input gradient of the activation function.

        Args:
            ctx: Context containing stored variables.
            output_grad: Output gradients.
                Must be the same shape as the output.

        Returns:
            Input gradient of the activation function.
        """
        (input,) = ctx.saved_tensors
        input_grad = _launch_backward(output_grad, input, ctx.act, ctx.param, ctx.drop_p, ctx.seed)
        return input_grad, None, None, None


class DropoutAutoGrad(torch.autograd.Function):
    """
    Autodiff for dropout (attorch/dropout_layer.py:19-96).
    """
    @staticmethod
    @custom_fwd(device_type='cuda')
    def forward(
        ctx: Any,
        input: Tensor,
        drop_p: float,
        training: bool,
        ) -> Tensor:
        """
        Randomly zeroes elements in the input.

        Args:
            ctx: Context for variable storage.
            input: Input to perform dropout on.
                Can have arbitrary shape.
            drop_p: Probability of dropping an element.
            training: Flag indicating if the model is in training mode.
                If False, no dropout is applied.

        Returns:
            Input with some elements zeroed out.
        """
        ctx.do_dropout = True
        if not training or drop_p == 0:
            ctx.do_dropout = False
            return input

        ctx.drop_all = False
        if drop_p == 1:
            ctx.drop_all = True
            return torch.zeros_like(input)

        _lib.require_gpu(input, 'Dropout')
        ctx.seed = randint(0, 65535)
        ctx.drop_p = float(drop_p)
        return _launch_forward(input, 0, 0.0, ctx.drop_p, ctx.seed)

    @staticmethod
    @custom_bwd
    def backward(
        ctx: Any,
        output_grad: Tensor,
        ) -> Tuple[Optional[Tensor], ...]:
        """
        Calculates the input gradient of dropout.

        Args:
            ctx: Context containing stored variables.
            output_grad: Output gradients.
                Must be the same shape as the output.

        Returns:
            Input gradient of dropout.
        """
        if not ctx.do_dropout:
            return output_grad, None, None
        if ctx.drop_all:
            return torch.zeros_like(output_grad), None, None
        return _launch_backward(output_grad, None, 0, 0.0, ctx.drop_p, ctx.seed), None, None


class Dropout(nn.Dropout):
    """
    Randomly zeroes elements in the input during training.
    See also base class.

    Args:
        p: Probability of dropping an element.
        inplace: This is a dummy argument and has no effects,
            as in-place is currently not supported.
    """
    def __init__(self, p: float = 0.5, inplace: bool = False) -> None:
        super().__init__(p=p, inplace=False)
        if inplace is True:
            warnings.warn('In-place dropout currently not supported; '
                          'falling back to out-of-place.')

    def forward(self, input: Tensor) -> Tensor:
        return DropoutAutoGrad.apply(input, self.p, self.training)


def _warn_inplace(inplace: bool, name: str) -> None:
    if inplace is True:
        warnings.warn(f'In-place {name} currently not supported; falling back to out-of-place.')


def _plain_layer(base: type, act_func: str, label: str, takes_inplace: bool) -> type:
    """
    Builds the layer class of a parameter-free activation: a subclass of the torch module
    `base` whose constructor takes `drop_p` (after the dummy `inplace` where torch's has one,
    as in attorch/act_layers.py:120-433) and whose forward runs ActFuncAutoGrad.
    """
    if takes_inplace:
        def __init__(self, inplace: bool = False, drop_p: float = 0.0) -> None:
            base.__init__(self, inplace=False)
            self.drop_p = drop_p
            _warn_inplace(inplace, label)
    else:
        def __init__(self, drop_p: float = 0.0) -> None:
            base.__init__(self)
            self.drop_p = drop_p

    def forward(self, input: Tensor) -> Tensor:
        return ActFuncAutoGrad.apply(input, act_func, self.drop_p, self.training)

    doc = (f'Applies {label} to the input, optionally fusing dropout.\n\n'
           f'Args:\n'
           + ('    inplace: Dummy argument; in-place is not supported.\n' if takes_inplace else '')
           + '    drop_p: Probability of dropping an element for dropout.\n')
    return type(base.__name__, (base,), {'__init__': __init__, 'forward': forward, '__doc__': doc,
                                         '__module__': __name__})


Sigmoid = _plain_layer(nn.Sigmoid, 'sigmoid', 'sigmoid', False)
LogSigmoid = _plain_layer(nn.LogSigmoid, 'logsigmoid', 'the log of sigmoid', False)
Tanh = _plain_layer(nn.Tanh, 'tanh', 'tanh', False)
ReLU = _plain_layer(nn.ReLU, 'relu', 'ReLU', True)
SiLU = _plain_layer(nn.SiLU, 'silu', 'SiLU', True)
ReLU6 = _plain_layer(nn.ReLU6, 'relu6', 'ReLU6', True)
Hardsigmoid = _plain_layer(nn.Hardsigmoid, 'hardsigmoid', 'hard sigmoid', True)
Hardswish = _plain_layer(nn.Hardswish, 'hardswish', 'hard Swish', True)
SELU = _plain_layer(nn.SELU, 'selu', 'SELU', True)
Mish = _plain_layer(nn.Mish, 'mish', 'Mish', True)
Softplus = _plain_layer(nn.Softplus, 'softplus', 'softplus', False)
Softsign = _plain_layer(nn.Softsign, 'softsign', 'softsign', False)
Tanhshrink = _plain_layer(nn.Tanhshrink, 'tanhshrink', 'tanh shrink', False)


class GELU(nn.GELU):
    """
    Applies GELU to the input, optionally fusing dropout (attorch/act_layers.py:190-213).

    Args:
        approximate: GELU approximation algorithm to use.
            Options are 'none' and 'tanh'.
        drop_p: Probability of dropping an element for dropout.

    Raises:
        RuntimeError: Approximation algorithm is invalid.
    """
    def __init__(self, approximate: str = 'none', drop_p: float = 0.0) -> None:
        if approximate not in ['none', 'tanh']:
            raise RuntimeError(f'Approximation algorithm {approximate} invalid.')
        super().__init__(approximate=approximate)
        self.drop_p = drop_p

    def forward(self, input: Tensor) -> Tensor:
        name = 'gelu' if self.approximate == 'none' else 'geluapprox'
        return ActFuncAutoGrad.apply(input, name, self.drop_p, self.training)


class Hardtanh(nn.Hardtanh):
    """
    Applies hard tanh to the input, optionally fusing dropout (attorch/act_layers.py:282-319).

    Args:
        min_val: Only -1 is supported.
        max_val: Only 1 is supported.
        inplace: Dummy argument; in-place is not supported.
        drop_p: Probability of dropping an element for dropout.

    Raises:
        RuntimeError: The minimum is not -1 or the maximum is not 1.
    """
    def __init__(self, min_val: float = -1.0, max_val: float = 1.0, inplace: bool = False,
                 drop_p: float = 0.0) -> None:
        if min_val != -1.0:
            raise RuntimeError('Hard tanh only supports a minimum value of -1.')
        if max_val != 1.0:
            raise RuntimeError('Hard tanh only supports a maximum value of 1.')
        super().__init__(inplace=False)
        self.drop_p = drop_p
        _warn_inplace(inplace, 'hard tanh')

    def forward(self, input: Tensor) -> Tensor:
        return ActFuncAutoGrad.apply(input, 'hardtanh', self.drop_p, self.training)


class _ParamLayer:
    """
    Shared forward of the parametrized activations: the parameter travels inside the
    activation string ('leaky_relu_0.01'), as in attorch/act_layers.py:436-570.
    """
    _act_func = ''
    _param_attr = ''

    def forward(self, input: Tensor) -> Tensor:
        act_func = f'{self._act_func}_{getattr(self, self._param_attr)}'
        return ActFuncAutoGrad.apply(input, act_func, self.drop_p, self.training)


class LeakyReLU(_ParamLayer, nn.LeakyReLU):
    """
    Applies leaky ReLU to the input, optionally fusing dropout.

    Args:
        inplace: Dummy argument; in-place is not supported.
        negative_slope: Slope of the negative component.
        drop_p: Probability of dropping an element for dropout.
    """
    _act_func, _param_attr = 'leaky_relu', 'negative_slope'

    def __init__(self, inplace: bool = False, negative_slope: float = 1e-2, drop_p: float = 0.0) -> None:
        nn.LeakyReLU.__init__(self, negative_slope=negative_slope, inplace=False)
        self.drop_p = drop_p
        _warn_inplace(inplace, 'leaky ReLU')


class ELU(_ParamLayer, nn.ELU):
    """
    Applies ELU to the input, optionally fusing dropout.

    Args:
        inplace: Dummy argument; in-place is not supported.
        alpha: Alpha value.
        drop_p: Probability of dropping an element for dropout.
    """
    _act_func, _param_attr = 'elu', 'alpha'

    def __init__(self, inplace: bool = False, alpha: float = 1.0, drop_p: float = 0.0) -> None:
        nn.ELU.__init__(self, alpha, inplace=False)
        self.drop_p = drop_p
        _warn_inplace(inplace, 'ELU')


class CELU(_ParamLayer, nn.CELU):
    """
    Applies CELU to the input, optionally fusing dropout.

    Args:
        inplace: Dummy argument; in-place is not supported.
        alpha: Alpha value.
        drop_p: Probability of dropping an element for dropout.
    """
    _act_func, _param_attr = 'celu', 'alpha'

    def __init__(self, inplace: bool = False, alpha: float = 1.0, drop_p: float = 0.0) -> None:
        nn.CELU.__init__(self, alpha, inplace=False)
        self.drop_p = drop_p
        _warn_inplace(inplace, 'CELU')


class Hardshrink(_ParamLayer, nn.Hardshrink):
    """
    Applies hard shrink to the input, optionally fusing dropout.

    Args:
        lambd: Lambda value.
        drop_p: Probability of dropping an element for dropout.
    """
    _act_func, _param_attr = 'hardshrink', 'lambd'

    def __init__(self, lambd: float = 0.5, drop_p: float = 0.0) -> None:
        nn.Hardshrink.__init__(self, lambd)
        self.drop_p = drop_p


class Softshrink(_ParamLayer, nn.Softshrink):
    """
    Applies soft shrink to the input, optionally fusing dropout.

    Args:
        lambd: Lambda value.
        drop_p: Probability of dropping an element for dropout.
    """
    _act_func, _param_attr = 'softshrink', 'lambd'

    def __init__(self, lambd: float = 0.5, drop_p: float = 0.0) -> None:
        nn.Softshrink.__init__(self, lambd)
        self.drop_p = drop_p
