"""
Seeded random sweep over shapes, layouts and dtypes for Linear and Conv2d, against float64
references computed by torch from the same (rounded) operands.  The fixed cases elsewhere pin the
arithmetic; this sweep is about dispatch: every combination of extents selects some kernel, tile
size, padding or fallback path, and each must agree with the same closed form.
"""

import random

import pytest
import torch
import torch.nn.functional as F

import attorch_amd
from .helpers import assert_close

pytestmark = pytest.mark.gpu

EXTENTS = [1, 2, 3, 7, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 96, 100, 127, 128, 129, 192, 255, 256,
           257, 300, 384, 511, 512, 513, 640, 777, 1000, 1024, 1025, 1536, 2048, 2050]
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _linear_case(rng: random.Random, index: int) -> None:
    batch, in_dim, out_dim = rng.choice(EXTENTS), rng.choice(EXTENTS), rng.choice(EXTENTS)
    if rng.random() < 0.15:
        batch = rng.choice([4096, 5000, 8192])
    dtype = rng.choice(DTYPES)
    act_func = rng.choice([None, 'relu', 'geluapprox', 'silu', 'leaky_relu_0.1', 'tanh'])
    bias = rng.random() < 0.7
    layout = rng.choice(['plain', 'plain', 'wide', 'transposed'])
    what = f'linear case {index}: [{batch}, {in_dim}] -> {out_dim} {dtype} {act_func} bias={bias} {layout}'
    gen = torch.Generator().manual_seed(index)
    if layout == 'wide':        # rows longer than the features: row stride > in_dim
        x = torch.randn(batch, in_dim + rng.choice([1, 5, 8]), generator=gen).to(dtype).cuda()[:, :in_dim]
    elif layout == 'transposed':  # unit stride along the rows
        x = torch.randn(in_dim, batch, generator=gen).to(dtype).cuda().T
    else:
        x = torch.randn(batch, in_dim, generator=gen).to(dtype).cuda()
    x = x.detach().requires_grad_(True)
    layer = attorch_amd.Linear(in_dim, out_dim, bias=bias, act_func=act_func, device='cuda', dtype=dtype)
    dy = torch.randn(batch, out_dim, generator=gen).to(dtype).cuda()
    y = layer(x)
    y.backward(dy)

    xr = x.detach().double().requires_grad_(True)
    wr = layer.weight.detach().double().requires_grad_(True)
    br = layer.bias.detach().double().requires_grad_(True) if bias else None
    z = xr @ wr + (br if bias else 0)
    if act_func in ('relu', 'leaky_relu_0.1'):
        # the derivative mask comes from the device's own signs: a last-bit difference at z = 0
        # would flip it, and the fixed cases already compare the pre-activations
        slope = 0.0 if act_func == 'relu' else 0.1
        yr = torch.where(z > 0, z, slope * z)
        z.backward(dy.double() * torch.where(y.detach().double() > 0, 1.0, slope))
    else:
        yr = {None: lambda t: t, 'geluapprox': lambda t: F.gelu(t, approximate='tanh'), 'silu': F.silu,
              'tanh': torch.tanh}[act_func](z)
        yr.backward(dy.double())
    assert_close(y, yr, dtype, what + ' output')
    assert_close(x.grad, xr.grad, dtype, what + ' input_grad')
    assert_close(layer.weight.grad, wr.grad, dtype, what + ' weight_grad', batch_reduction=True)
    if bias:
        assert_close(layer.bias.grad, br.grad, dtype, what + ' bias_grad', batch_reduction=True)


def _conv_case(rng: random.Random, index: int) -> None:
    dtype = rng.choice(DTYPES)
    groups = rng.choice([1, 1, 1, 2, 3])
    # odd cases: thin and unaligned channel counts; even cases: counts the matrix-core path pads or takes as they are
    in_choices, out_choices = (([1, 3, 8, 64, 72, 128], [1, 2, 24, 32, 64, 96]) if index % 2 else
                               ([16, 32, 48, 64, 96, 128], [16, 32, 64, 80, 128, 192]))
    in_per_group, out_per_group = rng.choice(in_choices), rng.choice(out_choices)
    kernel = rng.choice([(1, 1), (3, 3), (3, 3), (5, 5), (3, 1), (2, 4), (7, 7)])
    stride = rng.choice([(1, 1), (1, 1), (2, 2), (1, 2)])
    padding = (rng.choice([0, 1, 2, 3]), rng.choice([0, 1, 2, 3]))
    batch = rng.choice([1, 2, 5, 9])
    height, width = rng.choice([1, 5, 7, 14, 23, 28, 56]), rng.choice([1, 4, 9, 14, 31, 56, 64])
    if height + 2 * padding[0] < kernel[0] or width + 2 * padding[1] < kernel[1]:
        return
    bias = rng.random() < 0.5
    channels_last = rng.random() < 0.5      # tensors in torch.channels_last memory format
    what = (f'conv case {index}: [{batch}, {in_per_group * groups}, {height}, {width}] -> {out_per_group * groups} '
            f'k{kernel} s{stride} p{padding} g{groups} {dtype} bias={bias} channels_last={channels_last}')
    torch.manual_seed(index)
    layer = attorch_amd.Conv2d(in_per_group * groups, out_per_group * groups, kernel, stride=stride,
                               padding=padding, groups=groups, bias=bias, device='cuda', dtype=dtype)
    x = torch.randn(batch, in_per_group * groups, height, width, device='cuda', dtype=dtype)
    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)
    x.requires_grad_(True)
    xr = x.detach().double().contiguous().requires_grad_(True)
    wr = layer.weight.detach().double().requires_grad_(True)
    br = layer.bias.detach().double().requires_grad_(True) if bias else None
    y = layer(x)
    yr = F.conv2d(xr, wr, br, stride, padding, 1, groups)
    dy = torch.randn(y.shape, device='cuda', dtype=dtype)
    if channels_last:
        dy = dy.contiguous(memory_format=torch.channels_last)
    y.backward(dy)
    yr.backward(dy.double())
    assert_close(y, yr, dtype, what + ' output')
    assert_close(x.grad, xr.grad, dtype, what + ' input_grad')
    assert_close(layer.weight.grad, wr.grad, dtype, what + ' weight_grad', batch_reduction=True)
    if bias:
        assert_close(layer.bias.grad, br.grad, dtype, what + ' bias_grad', batch_reduction=True)


FEATS = [1, 2, 3, 5, 8, 15, 16, 31, 33, 64, 100, 127, 128, 255, 256, 300, 511, 512, 1000, 1024, 2047, 2048,
         4096, 5000, 8192, 10000, 20000, 50257, 70001]
ROWS = [1, 2, 3, 7, 16, 33, 100, 257, 1000, 1025, 4096]


def _row_case(rng: random.Random, index: int) -> None:
    kind = rng.choice(['layer_norm', 'rms_norm', 'softmax', 'log_softmax', 'softmin', 'cross_entropy'])
    dtype = rng.choice(DTYPES)
    rows, feat = rng.choice(ROWS), rng.choice(FEATS)
    if rows * feat > 2e7:
        rows = max(1, int(2e7 // feat))
    what = f'row case {index}: {kind} [{rows}, {feat}] {dtype}'
    gen = torch.Generator().manual_seed(index)
    if kind == 'cross_entropy':
        feat = max(feat, 2)
        x = (2 * torch.randn(rows, feat, generator=gen)).to(dtype).cuda().requires_grad_(True)
        target = torch.randint(0, feat, (rows,), generator=gen).cuda()
        if rows > 1:   # an all-ignored batch is 0 / 0 in both implementations
            target[torch.rand(rows, generator=gen).cuda() < 0.3] = -100
            target[0] = 0
        weight = (0.5 + torch.rand(feat, generator=gen)).to(dtype).cuda() if rng.random() < 0.5 else None
        xr = x.detach().double().requires_grad_(True)
        y = attorch_amd.CrossEntropyLoss(weight=weight)(x, target)
        yr = F.cross_entropy(xr, target, weight=None if weight is None else weight.double(), ignore_index=-100)
        y.backward()
        yr.backward()
        assert_close(y, yr.to(y.dtype), dtype, what + ' loss')
        assert_close(x.grad, xr.grad, dtype, what + ' input_grad')
        return
    wide = rng.random() < 0.3   # rows longer than the features: row stride > feat
    base = torch.randn(rows, feat + (rng.choice([1, 3, 8]) if wide else 0), generator=gen).to(dtype).cuda()
    x = base[:, :feat].detach().requires_grad_(True)
    xr = x.detach().double().requires_grad_(True)
    dy = torch.randn(rows, feat, generator=gen).to(dtype).cuda()
    if kind == 'layer_norm':
        layer = attorch_amd.LayerNorm(feat, device='cuda', dtype=dtype)
        with torch.no_grad():
            layer.weight.normal_(1, 0.2), layer.bias.normal_(0, 0.2)
        yr = F.layer_norm(xr, (feat,), layer.weight.double(), layer.bias.double(), layer.eps)
    elif kind == 'rms_norm':
        layer = attorch_amd.RMSNorm(feat, eps=1e-5, device='cuda', dtype=dtype)
        with torch.no_grad():
            layer.weight.normal_(1, 0.2)
        yr = xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + 1e-5) * layer.weight.double()
    else:
        layer = {'softmax': attorch_amd.Softmax, 'log_softmax': attorch_amd.LogSoftmax,
                 'softmin': attorch_amd.Softmin}[kind](dim=-1)
        yr = {'softmax': F.softmax, 'log_softmax': F.log_softmax, 'softmin': F.softmin}[kind](xr, dim=-1)
    y = layer(x)
    y.backward(dy)
    yr.backward(dy.double())
    assert_close(y, yr, dtype, what + ' output')
    # a row of one feature has a zero gradient up to rounding of inv_std * (g - g)
    assert_close(x.grad, xr.grad, dtype, what + ' input_grad', atol_scale=1.0 if feat > 1 else 100.0)


@pytest.mark.parametrize('chunk', range(3))
def test_row_kernels_random_shapes(chunk) -> None:
    rng = random.Random(3000 + chunk)
    for index in range(chunk * 30, chunk * 30 + 30):
        _row_case(rng, index)


@pytest.mark.parametrize('chunk', range(4))
def test_linear_random_shapes(chunk) -> None:
    rng = random.Random(1000 + chunk)
    for index in range(chunk * 30, chunk * 30 + 30):
        _linear_case(rng, index)


@pytest.mark.parametrize('chunk', range(4))
def test_conv_random_shapes(chunk) -> None:
    rng = random.Random(2000 + chunk)
    for index in range(chunk * 25, chunk * 25 + 25):
        _conv_case(rng, index)
