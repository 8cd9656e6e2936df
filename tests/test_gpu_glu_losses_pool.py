"""
GPU parity tests of GLU, the p-norm losses and average pooling against the CPU oracle
(torch's avg_pool for pooling); shapes follow the reference's tests/test_glu_layer.py,
tests/test_p_loss_layers.py and tests/test_pooling_layer.py.
"""

import pytest
import torch

import attorch_amd
import oracle
from .helpers import ACT_FUNCS, DTYPES, assert_close, compute_dtype, randn

pytestmark = pytest.mark.gpu

GLU_CASES = [((1, 8000), -1), ((4, 2000), -1), ((8, 1024), 1), ((2048, 768), -1), ((6144, 256), 0),
             ((8096, 32), 0), ((12288, 2), 1), ((1, 1024, 3072), 2), ((8, 960, 196), 1), ((64, 64, 56, 56), 1),
             ((5, 6, 7), 1), ((3, 10, 9), -2), ((6, 3, 5), 0)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape, dim', GLU_CASES)
@pytest.mark.parametrize('act_func', ['sigmoid', 'geluapprox', 'leaky_relu_0.01'])
def test_glu(shape, dim, act_func, dtype) -> None:
    x = randn(shape, 1, dtype)
    name, param = oracle.parse_act_func(act_func)
    cd = compute_dtype(dtype)
    y_ref = oracle.glu_forward(x, dim, name, param, dtype, compute=cd)
    dy = randn(y_ref.shape, 2, dtype)
    dx_ref = oracle.glu_backward(dy, x, dim, name, param, dtype, compute=cd)
    xd = x.cuda().requires_grad_(True)
    y = attorch_amd.GLU(dim, act_func)(xd)
    y.backward(dy.cuda())
    assert y.dtype is dtype and y.shape == y_ref.shape
    assert_close(y, y_ref, dtype, 'output')
    assert_close(xd.grad, dx_ref, dtype, 'input_grad')


@pytest.mark.parametrize('act_func', [a for a in ACT_FUNCS if a is not None])
def test_glu_every_activation(act_func) -> None:
    x = randn((96, 200), 3)
    name, param = oracle.parse_act_func(act_func)
    # keep the gate away from the joints of the piecewise activations (their derivative jumps there)
    gate = x[:, 100:]
    for joint in (-3.0, -1.0, -0.5, 0.0, 0.5, 1.0, 3.0, 6.0):
        gate[(gate - joint).abs() < 1e-3] += 0.01
    y_ref = oracle.glu_forward(x, -1, name, param, torch.float32, compute=torch.float64)
    dy = randn(y_ref.shape, 4)
    dx_ref = oracle.glu_backward(dy, x, -1, name, param, torch.float32, compute=torch.float64)
    xd = x.cuda().requires_grad_(True)
    y = attorch_amd.GLUAutoGrad.apply(xd, -1, act_func)
    y.backward(dy.cuda())
    assert_close(y, y_ref, torch.float32, 'output')
    assert_close(xd.grad, dx_ref, torch.float32, 'input_grad')


def test_glu_matches_torch_module_and_strided_input() -> None:
    x = randn((7, 12, 10), 5).cuda()
    torch.testing.assert_close(attorch_amd.GLU(1)(x), torch.nn.GLU(1)(x), rtol=1e-4, atol=1e-5)
    view = x.transpose(0, 2)                         # not contiguous
    torch.testing.assert_close(attorch_amd.GLU(0)(view), torch.nn.GLU(0)(view), rtol=1e-4, atol=1e-5)
    with pytest.raises(AssertionError):
        attorch_amd.GLU(-1)(randn((4, 7), 6).cuda())
    with pytest.raises(RuntimeError):
        attorch_amd.GLU(-1, 'nope')(x)


LOSSES = [(0, 'SmoothL1Loss', {'beta': 0.7}, 0.7), (1, 'L1Loss', {}, 1.0), (2, 'MSELoss', {}, 1.0),
          (3, 'HuberLoss', {'delta': 0.6}, 0.6)]
LOSS_SHAPES = [(1, 8000), (8, 1024), (2048, 768), (8096, 32), (12288, 1), (8, 960, 196), (64, 64, 56, 56), (5, 7),
               (1000003,)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', LOSS_SHAPES)
@pytest.mark.parametrize('p_loss, cls, kwargs, param', LOSSES)
@pytest.mark.parametrize('reduction', ['none', 'mean', 'sum'])
def test_p_loss(shape, dtype, p_loss, cls, kwargs, param, reduction) -> None:
    x, t = randn(shape, 1, dtype), randn(shape, 2, dtype)
    cd = compute_dtype(dtype)
    loss_ref = oracle.p_loss_forward(x, t, p_loss, reduction, param, dtype, compute=cd)
    upstream = randn(loss_ref.shape, 3, dtype) if reduction == 'none' else torch.tensor(0.37, dtype=dtype)
    dx_ref, dt_ref = oracle.p_loss_backward(upstream, x, t, p_loss, reduction, param, dtype, compute=cd)
    xd, td = x.cuda().requires_grad_(True), t.cuda().requires_grad_(True)
    loss = getattr(attorch_amd, cls)(reduction=reduction, **kwargs)(xd, td)
    loss.backward(upstream.cuda())
    assert loss.dtype is dtype and loss.shape == loss_ref.shape
    if not (reduction == 'sum' and dtype is torch.float16 and not torch.isfinite(loss_ref)):
        assert_close(loss, loss_ref, dtype, 'loss')
    scale = x.numel() if reduction == 'mean' else 1.0
    assert_close(xd.grad * scale, dx_ref.to(cd) * scale, dtype, 'input_grad')
    assert_close(td.grad * scale, dt_ref.to(cd) * scale, dtype, 'target_grad')


def test_p_loss_modules_match_torch_and_autocast() -> None:
    x, t = randn((33, 65), 1).cuda().requires_grad_(True), randn((33, 65), 2).cuda()
    for ours, theirs in ((attorch_amd.L1Loss(), torch.nn.L1Loss()), (attorch_amd.MSELoss(), torch.nn.MSELoss()),
                         (attorch_amd.SmoothL1Loss(beta=0.3), torch.nn.SmoothL1Loss(beta=0.3)),
                         (attorch_amd.HuberLoss(delta=1.5), torch.nn.HuberLoss(delta=1.5))):
        a, b = ours(x, t), theirs(x, t)
        torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-5)
        (ga,), (gb,) = torch.autograd.grad(a, x), torch.autograd.grad(b, x)
        torch.testing.assert_close(ga * x.numel(), gb * x.numel(), rtol=1e-4, atol=1e-5)
    with torch.autocast('cuda', dtype=torch.bfloat16):
        loss = attorch_amd.MSELoss()(x.bfloat16(), t.bfloat16())
    assert loss.dtype is torch.float32                                   # 'fp32' autocast policy
    # only the target needs a gradient
    t2 = t.clone().requires_grad_(True)
    attorch_amd.L1Loss(reduction='sum')(x.detach(), t2).backward()
    torch.testing.assert_close(t2.grad, -torch.where(x.detach() - t >= 0, 1.0, -1.0))
    empty = torch.empty((0, 4), device='cuda')
    assert attorch_amd.MSELoss(reduction='sum')(empty, empty).item() == 0.0


POOL_CASES = [((4, 8, 32, 32), (2, 2), None, (0, 0)), ((2, 16, 28, 28), (3, 3), (2, 2), (1, 1)),
              ((3, 5, 17, 19), (3, 2), (1, 2), (1, 0)), ((1, 64, 56, 56), (7, 7), (7, 7), (0, 0))]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape, kernel, stride, padding', POOL_CASES)
def test_avg_pool2d(shape, kernel, stride, padding, dtype) -> None:
    x = randn(shape, 1, dtype)
    cd = compute_dtype(dtype)
    xr = x.to(cd).requires_grad_(True)
    y_ref = torch.nn.functional.avg_pool2d(xr, kernel, stride, padding)
    dy = randn(y_ref.shape, 2, dtype)
    (dx_ref,) = torch.autograd.grad(y_ref, xr, dy.to(cd))
    xd = x.cuda().requires_grad_(True)
    y = attorch_amd.AvgPool2d(kernel, stride, padding)(xd)
    y.backward(dy.cuda())
    assert y.dtype is dtype
    assert_close(y, y_ref.detach().to(dtype), dtype, 'output')
    assert_close(xd.grad, dx_ref.to(dtype), dtype, 'input_grad')


def test_avg_pool1d_and_argument_errors() -> None:
    x = randn((3, 6, 50), 1).cuda().requires_grad_(True)
    y = attorch_amd.AvgPool1d(4, 2, 1)(x)
    torch.testing.assert_close(y, torch.nn.functional.avg_pool1d(x, 4, 2, 1), rtol=1e-4, atol=1e-5)
    y.sum().backward()
    assert x.grad.shape == x.shape
    with pytest.raises(RuntimeError):
        attorch_amd.AvgPool1d(2, ceil_mode=True)
    with pytest.raises(RuntimeError):
        attorch_amd.AvgPool2d(2, count_include_pad=False)
    with pytest.raises(RuntimeError):
        attorch_amd.AvgPool2d(2, divisor_override=3)
    import attorch_amd.nn as ann
    assert ann.AvgPool2d is torch.nn.AvgPool2d and ann.GLU is attorch_amd.GLU and ann.MSELoss is attorch_amd.MSELoss
