"""
The example blocks (MLP classifier, ResNet basic block, GPT block) on the attorch_amd layers
against the same blocks on torch.nn with the same parameters: loss / output and every parameter
gradient, forward + backward, fp32 and bf16.  This is the hot path as its callers use it (fused
activations, residual into BatchNorm, cross entropy on the head), end to end through autograd.
"""

import pytest
import torch

import attorch_amd.nn as fused_nn
from examples.blocks import BasicBlock, MLPClassifier, TinyGPT

pytestmark = pytest.mark.gpu


def _pair(cls, dtype, *args, **kwargs):
    torch.manual_seed(0)
    ours = cls(fused_nn, *args, **kwargs).to('cuda', dtype)
    theirs = cls(torch.nn, *args, **kwargs).to('cuda', dtype)
    theirs.load_from(ours)
    return ours, theirs


def _assert_mostly_close(actual, expected, rtol, atol, what, outliers=2e-3) -> None:
    """
    Elementwise comparison after scaling by max(1, max|expected|).  Through a ReLU the two
    implementations may round a pre-activation next to zero to opposite sides, which flips that
    element's gradient mask: a fraction `outliers` of the elements may therefore miss the tolerance
    (exactly none in float32, where the comparison stays strict).
    """
    a, e = actual.float(), expected.float()
    scale = max(1.0, e.abs().max().item())
    bad = ((a - e).abs() / scale > atol + rtol * e.abs() / scale).float().mean().item()
    limit = 0.0 if actual.dtype is torch.float32 else outliers
    assert bad <= limit, f'{what}: {bad:.5f} of the elements differ by more than the tolerance'


def _compare_grads(ours, theirs, rtol, atol) -> None:
    mine = dict(ours.named_parameters())
    for name, param in theirs.named_parameters():
        grad = mine[name].grad
        expected = param.grad
        if name.endswith('linear.weight'):          # Linear weights are [in, out] on our side
            expected = expected.T
        _assert_mostly_close(grad, expected, rtol, atol, name)


def test_nn_namespace_falls_back_to_torch() -> None:
    import attorch_amd
    assert fused_nn.Linear is attorch_amd.Linear and fused_nn.Conv2d is attorch_amd.Conv2d
    assert fused_nn.GELU is attorch_amd.GELU and fused_nn.Dropout is attorch_amd.Dropout
    assert fused_nn.Embedding is torch.nn.Embedding and fused_nn.AvgPool2d is torch.nn.AvgPool2d
    assert fused_nn.Sequential is torch.nn.Sequential


@pytest.mark.parametrize('dtype, rtol, atol', [(torch.float32, 1e-3, 1e-4), (torch.bfloat16, 5e-2, 5e-2)])
def test_mlp_classifier(dtype, rtol, atol) -> None:
    ours, theirs = _pair(MLPClassifier, dtype, 784, 256, 2, 10)
    x = torch.randn(512, 1, 28, 28, device='cuda', dtype=dtype)
    target = torch.randint(0, 10, (512,), device='cuda')
    loss, ref = ours(x, target), theirs(x, target)
    torch.testing.assert_close(loss.float(), ref.float(), rtol=rtol, atol=atol)
    loss.backward()
    ref.backward()
    _compare_grads(ours, theirs, rtol, atol)


@pytest.mark.parametrize('dtype, rtol, atol', [(torch.float32, 1e-3, 1e-3), (torch.bfloat16, 5e-2, 5e-2)])
@pytest.mark.parametrize('in_dim, out_dim, stride', [(64, 64, 1), (64, 128, 2)])
def test_basic_block(dtype, rtol, atol, in_dim, out_dim, stride) -> None:
    ours, theirs = _pair(BasicBlock, dtype, in_dim, out_dim, stride)
    x = torch.randn(8, in_dim, 16, 16, device='cuda', dtype=dtype)
    xo, xt = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    out, ref = ours(xo), theirs(xt)
    torch.testing.assert_close(out.float(), ref.float(), rtol=rtol, atol=atol)
    dy = torch.randn_like(out)
    out.backward(dy)
    ref.backward(dy)
    _assert_mostly_close(xo.grad, xt.grad, rtol, atol, 'input_grad')
    _compare_grads(ours, theirs, rtol, atol)
    # running statistics were updated alike
    torch.testing.assert_close(ours.first.bn.running_var.float(), theirs.first.bn.running_var.float(),
                               rtol=rtol, atol=atol)


@pytest.mark.parametrize('dtype, rtol, atol', [(torch.float32, 2e-3, 2e-3), (torch.bfloat16, 6e-2, 6e-2)])
def test_tiny_gpt(dtype, rtol, atol) -> None:
    ours, theirs = _pair(TinyGPT, dtype, 1000, 2, 128, 4, 64)
    tokens = torch.randint(0, 1000, (4, 64), device='cuda')
    torch.testing.assert_close(ours(tokens).float(), theirs(tokens).float(), rtol=rtol, atol=atol)
    loss, ref = ours(tokens, return_loss=True), theirs(tokens, return_loss=True)
    torch.testing.assert_close(loss.float(), ref.float(), rtol=rtol, atol=atol)
    loss.backward()
    ref.backward()
    _compare_grads(ours, theirs, rtol, atol)
