"""
GPU parity tests of CrossEntropyLoss (fused loss + gradient, class weights, ignore_index)
against the CPU oracle; shapes follow the reference's tests/test_cross_entropy_loss_layer.py
plus vocabulary-sized and unaligned rows.
"""

import math

import pytest
import torch

import attorch_amd
import oracle
from .helpers import DTYPES, assert_close, compute_dtype, randn

pytestmark = pytest.mark.gpu

SHAPES = [(1, 8000), (4, 2000), (8, 1024), (32, 1024), (2048, 768), (6144, 256), (8096, 32), (12288, 1),
          (5, 7), (48, 50257), (9, 12345), (4, 131075)]


def make_targets(batch, feat, seed, ignore_fraction):
    gen = torch.Generator().manual_seed(seed)
    target = torch.randint(0, feat, (batch,), generator=gen)
    if ignore_fraction:
        target[torch.rand(batch, generator=gen) < ignore_fraction] = -100
    return target


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('weighted', [False, True])
@pytest.mark.parametrize('ignore_fraction, upstream', [(0.0, 1.0), (0.3, 1.0), (0.05, 0.37)])
def test_cross_entropy(shape, dtype, weighted, ignore_fraction, upstream) -> None:
    batch, feat = shape
    x = randn(shape, 1, dtype, 2.0)
    target = make_targets(batch, feat, 2, ignore_fraction)
    gen = torch.Generator().manual_seed(3)
    weight = 0.5 + torch.rand(feat, generator=gen) if weighted else None
    cd = compute_dtype(dtype)
    loss_ref, denom = oracle.cross_entropy_forward(x, target, weight, -100, dtype, compute=cd)
    grad_ref = oracle.cross_entropy_backward(torch.tensor(upstream), x, target, weight, -100, dtype, compute=cd)

    xd = x.cuda().requires_grad_(True)
    loss = attorch_amd.CrossEntropyLossAutoGrad.apply(xd, target.cuda(),
                                                      None if weight is None else weight.cuda(), -100)
    (loss * upstream).backward()
    assert loss.dtype is dtype and loss.ndim == 0
    assert_close(loss, loss_ref, dtype, 'loss')
    # gradients are O(1 / kept rows); compare them on the scale of one row
    kept = max(1.0, float((target != -100).sum()))
    assert_close(xd.grad * kept, grad_ref.to(cd) * kept, dtype, 'input_grad')
    ignored = (target == -100).cuda()
    assert torch.all(xd.grad[ignored] == 0), 'ignored rows must get exactly zero gradient'
    if dtype is torch.float32:
        # rows of softmax - onehot sum to zero
        assert (xd.grad.sum(dim=1) * kept).abs().max().item() < 1e-3


def test_special_cases() -> None:
    ce = attorch_amd.CrossEntropyLoss()
    target = torch.tensor([0, 3, 2, 1], device='cuda')
    loss = ce(torch.zeros(4, 5, device='cuda'), target)
    assert math.isclose(loss.item(), math.log(5), rel_tol=1e-6)           # uniform logits -> log V
    all_ignored = ce(torch.zeros(4, 5, device='cuda'), torch.full((4,), -100, device='cuda'))
    assert math.isnan(all_ignored.item())                                  # 0 / 0, as torch
    x = randn((4, 5), 1).cuda().requires_grad_(True)
    ce(x, target).backward()
    sm = torch.softmax(x.detach(), dim=1)
    assert math.isclose(x.grad[1, 3].item(), (sm[1, 3].item() - 1) / 4, rel_tol=1e-4)
    torch.testing.assert_close(x.grad.sum(dim=1), torch.zeros(4, device='cuda'), atol=1e-6, rtol=0)


def test_custom_ignore_index_and_module_weight() -> None:
    x = randn((64, 33), 1)
    target = make_targets(64, 33, 2, 0.0)
    target[::5] = 7                                                        # ignore class 7 instead
    weight = 0.5 + torch.rand(33, generator=torch.Generator().manual_seed(4))
    ce = attorch_amd.CrossEntropyLoss(weight=weight.cuda(), ignore_index=7)
    xd = x.cuda().requires_grad_(True)
    loss = ce(xd, target.cuda())
    loss.backward()
    expected = torch.nn.functional.cross_entropy(x.double(), target, weight.double(), ignore_index=7)
    assert_close(loss, expected.float(), torch.float32, 'loss')
    assert torch.all(xd.grad[::5] == 0)


def test_autocast_returns_fp32_loss_and_gradient() -> None:
    x = randn((32, 1000), 1, torch.float16, 2.0)
    target = make_targets(32, 1000, 2, 0.1)
    xd = x.cuda().requires_grad_(True)
    with torch.autocast('cuda', dtype=torch.float16):
        loss = attorch_amd.CrossEntropyLoss()(xd, target.cuda())
    assert loss.dtype is torch.float32
    loss.backward()
    ref, _ = oracle.cross_entropy_forward(x, target, None, -100, torch.float32)
    assert_close(loss, ref, torch.float32, 'loss')
    grad_ref = oracle.cross_entropy_backward(torch.tensor(1.0), x, target, None, -100, torch.float32)
    assert_close(xd.grad.float() * 29, grad_ref * 29, torch.float16, 'input_grad')


def test_unaligned_base_pointer() -> None:
    flat = randn((10 * 50257 + 3,), 1, torch.float16, 2.0).cuda()
    x = flat[3:].view(10, 50257)                                           # rows start 6 bytes off the 16-byte grid
    target = make_targets(10, 50257, 2, 0.2).cuda()
    xd = x.detach().requires_grad_(True)
    loss = attorch_amd.CrossEntropyLossAutoGrad.apply(xd, target, None, -100)
    loss.backward()
    ref, _ = oracle.cross_entropy_forward(x.cpu(), target.cpu(), None, -100, torch.float16)
    assert_close(loss, ref, torch.float16, 'loss')
    grad_ref = oracle.cross_entropy_backward(torch.tensor(1.0), x.cpu(), target.cpu(), None, -100, torch.float16)
    assert_close(xd.grad.float() * 8, grad_ref.float() * 8, torch.float16, 'input_grad')
