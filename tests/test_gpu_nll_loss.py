"""
GPU parity tests of NLLLoss (reductions, class weights, spatial dimensions) against the CPU
oracle; shapes follow the reference's tests/test_nll_loss_layer.py plus vocabulary-sized and
unaligned rows, and the LogSoftmax + NLLLoss pair against CrossEntropyLoss.
"""

import pytest
import torch

import attorch_amd
import oracle
from .helpers import DTYPES, assert_close, compute_dtype, randn

pytestmark = pytest.mark.gpu

SHAPES = [(1, 8000), (4, 2000), (8, 1024), (32, 1024), (2048, 768), (6144, 256), (8096, 32), (12288, 1),
          (5, 7), (48, 50257), (9, 12345),
          (4, 16, 96), (16, 10, 33), (3, 5, 7, 9), (128, 4, 14, 14), (2, 3, 4, 5, 6)]


def log_probs(shape, seed, dtype):
    return torch.log_softmax(randn(shape, seed, torch.float32, 2.0), dim=1).to(dtype)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('weighted', [False, True])
@pytest.mark.parametrize('reduction', ['none', 'mean', 'sum'])
def test_nll_loss(shape, dtype, weighted, reduction) -> None:
    feat = shape[1]
    x = log_probs(shape, 1, dtype)
    gen = torch.Generator().manual_seed(2)
    target = torch.randint(0, feat, (shape[0], *shape[2:]), generator=gen)
    weight = 0.5 + torch.rand(feat, generator=gen) if weighted else None
    cd = compute_dtype(dtype)
    loss_ref, _ = oracle.nll_loss_forward(x, target, weight, reduction, dtype, compute=cd)
    upstream = randn(loss_ref.shape, 4, dtype) if reduction == 'none' else torch.tensor(0.37, dtype=dtype)
    grad_ref = oracle.nll_loss_backward(upstream, x.shape, target, weight, reduction, dtype, compute=cd)

    xd = x.cuda().requires_grad_(True)
    loss = attorch_amd.NLLLossAutoGrad.apply(xd, target.cuda(), reduction,
                                             None if weight is None else weight.cuda())
    loss.backward(upstream.cuda())
    assert loss.dtype is dtype and loss.shape == loss_ref.shape
    # a sum over many entries grows with their number: compare on the scale of the result
    assert_close(loss, loss_ref, dtype, 'loss')
    entries = target.numel()
    scale = entries if reduction == 'mean' else 1.0
    assert xd.grad.shape == x.shape and xd.grad.dtype is dtype
    assert_close(xd.grad * scale, grad_ref.to(cd) * scale, dtype, 'input_grad')
    # exactly one non-zero per (batch, spatial) entry at most, all others exact zeros
    assert int((xd.grad != 0).sum()) <= entries


def test_module_matches_torch_and_cross_entropy() -> None:
    logits = randn((64, 1000), 1, torch.float32, 2.0).cuda().requires_grad_(True)
    target = torch.randint(0, 1000, (64,), generator=torch.Generator().manual_seed(5)).cuda()
    weight = (0.5 + torch.rand(1000, generator=torch.Generator().manual_seed(6))).cuda()
    for w in (None, weight):
        for reduction in ('mean', 'sum', 'none'):
            ours = attorch_amd.NLLLoss(weight=w, reduction=reduction)(attorch_amd.LogSoftmax(dim=-1)(logits), target)
            theirs = torch.nn.NLLLoss(weight=w, reduction=reduction)(torch.log_softmax(logits, dim=-1), target)
            torch.testing.assert_close(ours, theirs, rtol=1e-4, atol=1e-5)
    # LogSoftmax + NLLLoss is CrossEntropyLoss (attorch/cross_entropy_loss_layer.py:130-133), gradients included
    loss_pair = attorch_amd.NLLLoss(weight=weight)(attorch_amd.LogSoftmax(dim=-1)(logits), target)
    (grad_pair,) = torch.autograd.grad(loss_pair, logits)
    loss_fused = attorch_amd.CrossEntropyLoss(weight=weight)(logits, target)
    (grad_fused,) = torch.autograd.grad(loss_fused, logits)
    torch.testing.assert_close(loss_pair, loss_fused, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(grad_pair * 64, grad_fused * 64, rtol=1e-4, atol=1e-5)


def test_autocast_and_layouts() -> None:
    x = torch.log_softmax(randn((6, 5, 4, 3), 1).cuda(), dim=1)
    target = torch.randint(0, 5, (6, 4, 3), generator=torch.Generator().manual_seed(2)).cuda()
    expected = torch.nn.functional.nll_loss(x, target)
    with torch.autocast('cuda', dtype=torch.float16):
        loss = attorch_amd.NLLLoss()(x.half(), target)
    assert loss.dtype is torch.float32                                   # 'fp32' autocast policy
    torch.testing.assert_close(loss, expected, rtol=2e-3, atol=2e-3)
    # non-contiguous input (channels-last view) and int32 targets
    permuted = x.permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)
    assert not permuted.is_contiguous()
    torch.testing.assert_close(attorch_amd.NLLLoss()(permuted, target.int()), expected, rtol=1e-4, atol=1e-5)
    # out-of-range targets contribute nothing (the reference reads out of bounds there)
    bad = target.clone()
    bad[0, 0, 0] = 17
    kept = torch.ones_like(target, dtype=torch.bool)
    kept[0, 0, 0] = False
    xg = x.clone().requires_grad_(True)
    loss = attorch_amd.NLLLoss(reduction='sum')(xg, bad)
    loss.backward()
    torch.testing.assert_close(loss, -(x.gather(1, target[:, None])[:, 0][kept]).sum(), rtol=1e-4, atol=1e-5)
    assert torch.all(xg.grad[0, :, 0, 0] == 0)


def test_empty_batch() -> None:
    x = torch.empty((0, 5), device='cuda', requires_grad=True)
    target = torch.empty((0,), dtype=torch.int64, device='cuda')
    loss = attorch_amd.NLLLoss(reduction='sum')(x, target)
    assert loss.item() == 0.0
    loss.backward()
    assert x.grad.shape == (0, 5)
    assert attorch_amd.NLLLoss(reduction='none')(x, target).shape == (0,)
    assert torch.isnan(attorch_amd.NLLLoss(reduction='mean')(x, target))
    spatial = torch.empty((0, 5, 3), device='cuda')
    assert attorch_amd.NLLLoss(reduction='none')(spatial, torch.empty((0, 3), dtype=torch.int64, device='cuda')).shape == (0, 3)
