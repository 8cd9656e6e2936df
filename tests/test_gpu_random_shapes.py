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
    assert_close(y, yr, dtype, what + ' output', normalize=True)
    assert_close(x.grad, xr.grad, dtype, what + ' input_grad', normalize=True)
    assert_close(layer.weight.grad, wr.grad, dtype, what + ' weight_grad', normalize=True)
    if bias:
        assert_close(layer.bias.grad, br.grad, dtype, what + ' bias_grad', normalize=True)


def _conv_case(rng: random.Random, index: int) -> None:
    dtype = rng.choice(DTYPES)
    groups = rng.choice([1, 1, 1, 2, 3])
    in_per_group, out_per_group = rng.choice([1, 3, 8, 64, 72, 128]), rng.choice([1, 2, 24, 32, 64, 96])
    kernel = rng.choice([(1, 1), (3, 3), (3, 3), (5, 5), (3, 1), (2, 4), (7, 7)])
    stride = rng.choice([(1, 1), (1, 1), (2, 2), (1, 2)])
    padding = (rng.choice([0, 1, 2, 3]), rng.choice([0, 1, 2, 3]))
    batch = rng.choice([1, 2, 5, 9])
    height, width = rng.choice([1, 5, 7, 14, 23, 28, 56]), rng.choice([1, 4, 9, 14, 31, 56, 64])
    if height + 2 * padding[0] < kernel[0] or width + 2 * padding[1] < kernel[1]:
        return
    bias = rng.random() < 0.5
    what = (f'conv case {index}: [{batch}, {in_per_group * groups}, {height}, {width}] -> {out_per_group * groups} '
            f'k{kernel} s{stride} p{padding} g{groups} {dtype} bias={bias}')
    torch.manual_seed(index)
    layer = attorch_amd.Conv2d(in_per_group * groups, out_per_group * groups, kernel, stride=stride,
                               padding=padding, groups=groups, bias=bias, device='cuda', dtype=dtype)
    x = torch.randn(batch, in_per_group * groups, height, width, device='cuda', dtype=dtype, requires_grad=True)
    xr = x.detach().double().requires_grad_(True)
    wr = layer.weight.detach().double().requires_grad_(True)
    br = layer.bias.detach().double().requires_grad_(True) if bias else None
    y = layer(x)
    yr = F.conv2d(xr, wr, br, stride, padding, 1, groups)
    dy = torch.randn_like(y)
    y.backward(dy)
    yr.backward(dy.double())
    assert_close(y, yr, dtype, what + ' output', normalize=True)
    assert_close(x.grad, xr.grad, dtype, what + ' input_grad', normalize=True)
    assert_close(layer.weight.grad, wr.grad, dtype, what + ' weight_grad', normalize=True)
    if bias:
        assert_close(layer.bias.grad, br.grad, dtype, what + ' bias_grad', normalize=True)


@pytest.mark.parametrize('chunk', range(4))
def test_linear_random_shapes(chunk) -> None:
    rng = random.Random(1000 + chunk)
    for index in range(chunk * 30, chunk * 30 + 30):
        _linear_case(rng, index)


@pytest.mark.parametrize('chunk', range(3))
def test_conv_random_shapes(chunk) -> None:
    rng = random.Random(2000 + chunk)
    for index in range(chunk * 25, chunk * 25 + 25):
        _conv_case(rng, index)
