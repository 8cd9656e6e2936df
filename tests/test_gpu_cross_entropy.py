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
          (5, 7), (48, 50257), (9, 12345), (4, 131075),
          # rows of more than 4096 vectors: 1024 lanes per row with 6, 7 or 8 vectors each
          (6, 20001), (5, 32768), (3, 65536), (3, 57003)]


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


@pytest.mark.parametrize('dtype', DTYPES)
def test_backward_twice_through_a_retained_graph(dtype) -> None:
    # every backward through a retained graph gives output_grad times the unit gradient, whatever
    # came before; the tensor a call returned is never written again
    x = randn((48, 1000), 1, dtype, 2.0)
    target = make_targets(48, 1000, 2, 0.1)
    cd = compute_dtype(dtype)
    xd = x.cuda().requires_grad_(True)
    loss = attorch_amd.CrossEntropyLossAutoGrad.apply(xd, target.cuda(), None, -100)
    kept = float((target != -100).sum())
    results = []
    for upstream in (3.0, 3.0, 1.0, 0.25):
        (grad,) = torch.autograd.grad(loss, xd, torch.tensor(upstream, dtype=loss.dtype, device='cuda'),
                                      retain_graph=True)
        ref = oracle.cross_entropy_backward(torch.tensor(upstream), x, target, None, -100, dtype, compute=cd)
        results.append((grad, grad.clone(), ref))
    for grad, snapshot, ref in results:
        assert torch.equal(grad, snapshot), 'a gradient handed out earlier was modified by a later call'
        assert_close(grad * kept, ref.to(cd) * kept, dtype, 'input_grad')
    assert len({g.data_ptr() for g, _, _ in results}) == len(results), 'calls must not share a buffer'


def test_backward_with_upstream_one_returns_the_forward_gradient_without_a_copy() -> None:
    x = randn((16, 512), 1, torch.float32, 2.0)
    target = make_targets(16, 512, 2, 0.0)
    xd = x.cuda().requires_grad_(True)
    loss = attorch_amd.CrossEntropyLossAutoGrad.apply(xd, target.cuda(), None, -100)
    loss.backward()
    ref = oracle.cross_entropy_backward(torch.tensor(1.0), x, target, None, -100, torch.float32,
                                        compute=torch.float64)
    assert_close(xd.grad * 16, ref * 16, torch.float32, 'input_grad')


def test_fp16_loss_scale_is_applied_before_rounding() -> None:
    # vocabulary-wide rows: probability / rows is far below fp16's smallest subnormal, so a
    # gradient rounded at upstream 1 and scaled afterwards would be all zeros off the target column
    rows, vocab, scale = 1024, 50257, 32768.0   # the largest power of two below fp16's maximum
    x = randn((rows, vocab), 1, torch.float16, 2.0)
    target = make_targets(rows, vocab, 2, 0.05)
    xd = x.cuda().requires_grad_(True)
    loss = attorch_amd.CrossEntropyLossAutoGrad.apply(xd, target.cuda(), None, -100)
    loss.backward(torch.tensor(scale, dtype=torch.float16, device='cuda'))
    ref = oracle.cross_entropy_backward(torch.tensor(scale), x, target, None, -100, torch.float16)
    kept = target != -100
    got = xd.grad.cpu()
    assert torch.all(got[~kept] == 0)
    nonzero_ref = (ref[kept] != 0).float().mean().item()
    nonzero_got = (got[kept] != 0).float().mean().item()
    assert nonzero_ref > 0.5, 'the case must exercise values that survive only with the scale applied first'
    assert abs(nonzero_got - nonzero_ref) < 0.01
    mass_ref, mass_got = ref.float().abs().sum().item(), got.float().abs().sum().item()
    assert abs(mass_got - mass_ref) < 2e-2 * mass_ref
    per_row = float(kept.sum()) / scale
    assert_close(got.float() * per_row, ref.float() * per_row, torch.float16, 'input_grad')


def test_autocast_at_vocabulary_width() -> None:
    # the reference's policy: fp16 logits under autocast give an fp32 loss and an fp32 gradient, which
    # autograd rounds to the leaf's fp16
    rows, vocab = 8192, 50257
    x = randn((rows, vocab), 3001, torch.float16, 2.0)
    gen = torch.Generator().manual_seed(3002)
    target = torch.randint(0, vocab, (rows,), generator=gen)
    target[torch.rand(rows, generator=gen) < 0.05] = -100
    xd = x.cuda().requires_grad_(True)
    with torch.autocast('cuda', dtype=torch.float16):
        loss = attorch_amd.CrossEntropyLoss()(xd, target.cuda())
    loss.backward()
    assert loss.dtype is torch.float32 and xd.grad.dtype is torch.float16
    keep = target != -100
    denom = float(keep.sum())
    total = torch.zeros((), dtype=torch.float64)
    for start in range(0, rows, 1024):
        sl = slice(start, start + 1024)
        part, part_denom = oracle.cross_entropy_forward(x[sl], target[sl], None, -100, torch.float64)
        total += part * part_denom.double()
    assert_close(loss, (total / denom).float(), torch.float32, 'loss')
    # the fp32 gradient itself (autograd casts it to the leaf's dtype): the same call through the C ABI
    from attorch_amd import _lib
    lib = _lib.load()
    logits_d, target_d = x.cuda(), target.cuda()
    grad = torch.empty(rows, vocab, dtype=torch.float32, device='cuda')
    loss32 = torch.empty((), dtype=torch.float32, device='cuda')
    ws_bytes = lib.at_cross_entropy_workspace_bytes(rows)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device='cuda')
    _lib.check(lib.at_cross_entropy_fwd_bwd(
        logits_d.data_ptr(), target_d.data_ptr(), None, loss32.data_ptr(), grad.data_ptr(), ws.data_ptr(), ws_bytes,
        rows, vocab, vocab, vocab, -100, _lib.dtype_id(torch.float16), 0, _lib.dtype_id(torch.float32),
        _lib.dtype_id(torch.float32), _lib.stream_of(logits_d)), 'at_cross_entropy_fwd_bwd')
    assert torch.equal(loss32, loss.detach())
    for start in (0, 4096, 8192 - 128):
        sl = slice(start, start + 128)
        local = float(keep[sl].sum())
        ref = oracle.cross_entropy_backward(torch.tensor(local / denom), x[sl], target[sl], None, -100,
                                            torch.float32, compute=torch.float64)
        assert_close(grad[sl] * denom, ref * denom, torch.float32, 'input_grad slice', atol_scale=10)
    assert torch.all(grad[(~keep).cuda()] == 0)
    # the module writes the fp16 gradient directly: the same fp32 values, rounded once
    assert torch.equal(xd.grad, grad.half())


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_fp32_gradient_with_targets_at_every_kind_of_position(dtype) -> None:
    # fp32 gradient of 16-bit logits: the values change lanes before they are stored, and the target
    # column is patched by the lane that stored it.  Targets at the first and last elements of rows
    # (which start at different offsets from a 16-byte boundary, the width being odd), at both
    # halves of a 16-byte vector, and around the points where a wave's and a workgroup's share of
    # the row ends.
    from attorch_amd import _lib
    lib = _lib.load()
    vocab = 50257
    picks = [0, 1, 3, 4, 6, 7, 8, 9, 15, 16, 255, 256, 259, 260, 511, 512, 515, 516, 4091, 4092, 4095, 4096, 4099,
             4100, 8191, 8192, 32767, 32768, 50248, 50249, 50252, 50253, 50255, 50256]
    rows = len(picks)
    x = randn((rows, vocab), 4001, dtype, 2.0)
    target = torch.tensor(picks, dtype=torch.int64)
    logits_d, target_d = x.cuda(), target.cuda()
    grad = torch.full((rows, vocab), float('nan'), dtype=torch.float32, device='cuda')
    loss = torch.empty((), dtype=torch.float32, device='cuda')
    ws_bytes = lib.at_cross_entropy_workspace_bytes(rows)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device='cuda')
    _lib.check(lib.at_cross_entropy_fwd_bwd(
        logits_d.data_ptr(), target_d.data_ptr(), None, loss.data_ptr(), grad.data_ptr(), ws.data_ptr(), ws_bytes,
        rows, vocab, vocab, vocab, -100, _lib.dtype_id(dtype), 0, _lib.dtype_id(torch.float32),
        _lib.dtype_id(torch.float32), _lib.stream_of(logits_d)), 'at_cross_entropy_fwd_bwd')
    ref = oracle.cross_entropy_backward(torch.tensor(1.0), x, target, None, -100, torch.float32,
                                        compute=torch.float64)
    assert not torch.isnan(grad).any()
    assert_close(grad * rows, ref * rows, torch.float32, 'input_grad', atol_scale=10)
    at_target = grad.cpu()[torch.arange(rows), target]
    assert torch.all(at_target < 0), 'softmax - 1 at every target column'
    assert_close(at_target * rows, ref[torch.arange(rows), target] * rows, torch.float32, 'target columns',
                 atol_scale=10)


def test_empty_batch_gives_nan_loss_and_empty_gradient() -> None:
    x = torch.empty(0, 7, device='cuda', requires_grad=True)
    loss = attorch_amd.CrossEntropyLoss()(x, torch.empty(0, dtype=torch.int64, device='cuda'))
    assert math.isnan(loss.item())
    loss.backward()
    assert x.grad.shape == (0, 7)


def test_host_tensors_raise_instead_of_faulting() -> None:
    x = randn((4, 9), 1).cuda().requires_grad_(True)
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.CrossEntropyLoss()(x, torch.zeros(4, dtype=torch.int64))          # target on the host
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.CrossEntropyLoss(weight=torch.ones(9))(x, torch.zeros(4, dtype=torch.int64, device='cuda'))
