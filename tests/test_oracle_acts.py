"""
Pins oracle.acts against independent implementations: torch.nn.functional (values and
autograd derivatives, float64) and the known-answer boundary points of the reference's
tests/test_act_layers.py:55-61.
"""

import pytest
import torch
from torch.nn import functional as F

from oracle import ACT_NAMES, act_forward, act_grad, parse_act_func

TORCH_ACTS = {
    'sigmoid': torch.sigmoid, 'logsigmoid': F.logsigmoid, 'tanh': torch.tanh, 'relu': F.relu,
    'gelu': F.gelu, 'geluapprox': lambda x: F.gelu(x, approximate='tanh'), 'silu': F.silu,
    'relu6': F.relu6, 'hardsigmoid': F.hardsigmoid, 'hardtanh': F.hardtanh,
    'hardswish': F.hardswish, 'selu': F.selu, 'mish': F.mish, 'softplus': F.softplus,
    'softsign': F.softsign, 'tanhshrink': F.tanhshrink,
    'leaky_relu': lambda x: F.leaky_relu(x, 0.01), 'elu': lambda x: F.elu(x, 1.0),
    'celu': lambda x: F.celu(x, 1.5), 'hardshrink': lambda x: F.hardshrink(x, 0.5),
    'softshrink': lambda x: F.softshrink(x, 0.5),
}
PARAMS = {'leaky_relu': 0.01, 'elu': 1.0, 'celu': 1.5, 'hardshrink': 0.5, 'softshrink': 0.5}


def test_all_names_covered() -> None:
    assert set(TORCH_ACTS) == set(ACT_NAMES) and len(ACT_NAMES) == 21


@pytest.mark.parametrize('name', ACT_NAMES)
def test_act_values_and_derivatives_match_torch(name: str) -> None:
    torch.manual_seed(0)
    x = (3 * torch.randn(4096, dtype=torch.float64)).requires_grad_(True)
    expected = TORCH_ACTS[name](x)
    (expected_grad,) = torch.autograd.grad(expected.sum(), x)
    got = act_forward(x.detach(), name, PARAMS.get(name))
    got_grad = act_grad(x.detach(), name, PARAMS.get(name))
    # The reference truncates constants to ~9 digits (e.g. 0.707106781), hence 1e-7.
    torch.testing.assert_close(got, expected.detach(), rtol=1e-7, atol=1e-7)
    torch.testing.assert_close(got_grad, expected_grad, rtol=1e-7, atol=1e-7)


@pytest.mark.parametrize('name, torch_fn, param, boundaries',
                         [('hardshrink', lambda x: F.hardshrink(x, 0.5), 0.5, [-0.5, 0.5]),
                          ('softshrink', lambda x: F.softshrink(x, 0.5), 0.5, [-0.5, 0.5]),
                          ('hardswish', F.hardswish, None, [-3.0, 3.0]),
                          ('hardsigmoid', F.hardsigmoid, None, [-3.0, 3.0]),
                          ('hardtanh', F.hardtanh, None, [-1.0, 1.0]),
                          ('relu6', F.relu6, None, [0.0, 6.0])])
def test_piece_boundaries(name, torch_fn, param, boundaries) -> None:
    x = torch.tensor(boundaries, dtype=torch.float32, requires_grad=True)
    expected = torch_fn(x)
    (expected_grad,) = torch.autograd.grad(expected.sum(), x)
    torch.testing.assert_close(act_forward(x.detach(), name, param), expected.detach())
    if name == 'hardswish':
        # torch's CPU kernel returns 0 and 1 at the joints while its device kernel (the one the
        # reference test runs against) and the reference formula return x/3 + 0.5 there.
        expected_grad = torch.tensor([-0.5, 1.5])
    torch.testing.assert_close(act_grad(x.detach(), name, param), expected_grad)


def test_relu_derivative_at_zero_is_zero() -> None:
    assert act_grad(torch.zeros(1), 'relu').item() == 0.0


def test_parse_act_func() -> None:
    assert parse_act_func(None) == (None, None)
    assert parse_act_func('relu') == ('relu', None)
    assert parse_act_func('leaky_relu_0.01') == ('leaky_relu', 0.01)
    assert parse_act_func('elu_1') == ('elu', 1.0)
    # a parameterless name with '_' is split at its last underscore, as in the reference
    with pytest.raises(ValueError):
        parse_act_func('leaky_relu')
