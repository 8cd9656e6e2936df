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


def _assert_mostly_close(actual, expected, rtol, atol, what, outliers=2e-3, low_precision=None) -> None:
    """
    Elementwise comparison after scaling by max(1, max|expected|).  Through a ReLU the two
    implementations may round a pre-activation next to zero to opposite sides, which flips that
    element's gradient mask: a fraction `outliers` of the elements may therefore miss the tolerance
    (exactly none in float32, where the comparison stays strict).  low_precision=True says that
    float32 tensors were computed from 16-bit intermediates (autocast) and may have such outliers too.
    """
    a, e = actual.float(), expected.float()
    scale = max(1.0, e.abs().max().item())
    bad = ((a - e).abs() / scale > atol + rtol * e.abs() / scale).float().mean().item()
    if low_precision is None:
        low_precision = actual.dtype is not torch.float32
    # small tensors: one element may miss whatever the fraction says
    limit = max(outliers, 1.5 / max(1, a.numel())) if low_precision else 0.0
    assert bad <= limit, f'{what}: {bad:.5f} of the elements differ by more than the tolerance'


def _compare_grads(ours, theirs, rtol, atol, low_precision=None) -> None:
    mine = dict(ours.named_parameters())
    for name, param in theirs.named_parameters():
        grad = mine[name].grad
        expected = param.grad
        if name.endswith('linear.weight'):          # Linear weights are [in, out] on our side
            expected = expected.T
        _assert_mostly_close(grad, expected, rtol, atol, name, low_precision=low_precision)


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


# The reference's examples run their models with float32 parameters under torch.autocast
# (examples/utils.py:13-36, amp=True).  Both backends then round the matrix operands to the
# autocast dtype, so the comparison is at 16-bit tolerance; the parameter gradients arrive in
# float32 on both sides.
AMP_CASES = [(torch.float16, 5e-2, 5e-2), (torch.bfloat16, 6e-2, 6e-2)]


def _assert_fp32_grads(model) -> None:
    for name, param in model.named_parameters():
        assert param.grad is not None and param.grad.dtype is torch.float32, name


@pytest.mark.parametrize('amp_dtype, rtol, atol', AMP_CASES)
def test_mlp_classifier_under_autocast(amp_dtype, rtol, atol) -> None:
    ours, theirs = _pair(MLPClassifier, torch.float32, 784, 256, 2, 10)
    x = torch.randn(512, 1, 28, 28, device='cuda')
    target = torch.randint(0, 10, (512,), device='cuda')
    with torch.autocast('cuda', dtype=amp_dtype):
        loss, ref = ours(x, target), theirs(x, target)
    assert loss.dtype is torch.float32          # the loss follows the 'fp32' autocast policy
    torch.testing.assert_close(loss, ref.float(), rtol=rtol, atol=atol)
    loss.backward()
    ref.backward()
    _assert_fp32_grads(ours)
    _compare_grads(ours, theirs, rtol, atol, low_precision=True)


@pytest.mark.parametrize('amp_dtype, rtol, atol', AMP_CASES)
@pytest.mark.parametrize('in_dim, out_dim, stride', [(64, 64, 1), (64, 128, 2)])
def test_basic_block_under_autocast(amp_dtype, rtol, atol, in_dim, out_dim, stride) -> None:
    ours, theirs = _pair(BasicBlock, torch.float32, in_dim, out_dim, stride)
    x = torch.randn(8, in_dim, 16, 16, device='cuda')
    xo, xt = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    with torch.autocast('cuda', dtype=amp_dtype):
        out, ref = ours(xo), theirs(xt)
    assert out.dtype is amp_dtype               # conv under the 'fp16' policy, BatchNorm keeps its input's dtype
    torch.testing.assert_close(out.float(), ref.float(), rtol=rtol, atol=atol)
    dy = torch.randn_like(out)
    out.backward(dy)
    ref.backward(dy.to(ref.dtype))
    assert xo.grad.dtype is torch.float32
    _assert_mostly_close(xo.grad, xt.grad, rtol, atol, 'input_grad', outliers=5e-3, low_precision=True)
    _assert_fp32_grads(ours)
    mine = dict(ours.named_parameters())
    for name, param in theirs.named_parameters():
        _assert_mostly_close(mine[name].grad, param.grad, rtol, atol, name, outliers=5e-3, low_precision=True)


@pytest.mark.parametrize('amp_dtype, rtol, atol', AMP_CASES)
def test_tiny_gpt_under_autocast(amp_dtype, rtol, atol) -> None:
    ours, theirs = _pair(TinyGPT, torch.float32, 1000, 2, 128, 4, 64)
    tokens = torch.randint(0, 1000, (4, 64), device='cuda')
    with torch.autocast('cuda', dtype=amp_dtype):
        loss, ref = ours(tokens, return_loss=True), theirs(tokens, return_loss=True)
    torch.testing.assert_close(loss.float(), ref.float(), rtol=rtol, atol=atol)
    loss.backward()
    ref.backward()
    _assert_fp32_grads(ours)
    _compare_grads(ours, theirs, rtol, atol, low_precision=True)


def test_harness_reports_forward_backward_and_step_times() -> None:
    """
    examples.run_blocks.benchmark_fw_and_bw: forward, backward through one retained graph and
    the whole step, with and without automatic mixed precision.
    """
    from examples.run_blocks import benchmark_fw_and_bw
    model = MLPClassifier(fused_nn, 64, 128, 1, 10).to('cuda')
    x = torch.randn(256, 64, device='cuda')
    target = torch.randint(0, 10, (256,), device='cuda')
    for amp in (False, True):
        fw, bw, both = benchmark_fw_and_bw(model, lambda m: m(x, target), amp, torch.float16, 3)
        assert fw > 0 and bw > 0 and both > 0
