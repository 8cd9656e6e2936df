"""
GPU parity tests of the row-reduction layers (LayerNorm, RMSNorm, Softmax family) against
the CPU oracle, on the shapes of the reference's tests (tests/utils.py:14-66,
tests/test_layer_norm_layer.py:70-109) plus wide / unaligned rows.
"""

import pytest
import torch

import attorch_amd
import oracle
from .helpers import DTYPES, assert_close, compute_dtype, randn

pytestmark = pytest.mark.gpu

SHAPES = [(96,), (768,), (8000,), (1, 8000), (4, 2000), (8, 1024), (32, 1024), (2048, 768), (6144, 256),
          (8096, 32), (12288, 1), (2049, 2), (4097, 4), (8, 960, 196), (2048, 64, 16), (33, 4096),
          (7, 8200), (5, 12345), (3, 40000), (2, 70001),
          # more row-blocks than the persistent grids hold at once: several rows per workgroup
          (100001, 40), (20000, 520), (600000, 8),
          # many row-blocks per resident workgroup and a ragged last one: the softmax backward runs
          # one row-block per workgroup here
          (70001, 512), (9001, 4096)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('affine, bias', [(False, False), (True, False), (True, True)])
def test_layer_norm(shape, dtype, affine, bias) -> None:
    feat = shape[-1]
    x = randn(shape, 1, dtype)
    w = randn((feat,), 2, dtype, 0.1, 1.0) if affine else None
    b = randn((feat,), 3, dtype, 0.1) if bias else None
    dy = randn(shape, 4, dtype)
    cd = compute_dtype(dtype)
    y_ref, mean, inv_std = oracle.layer_norm_forward(x, w, b, 1e-5, dtype, compute=cd)
    dx_ref, dw_ref, db_ref = oracle.layer_norm_backward(dy, x, mean, inv_std, w, dtype, compute=cd)

    xd = x.cuda().requires_grad_(True)
    wd = w.cuda().requires_grad_(True) if affine else None
    bd = b.cuda().requires_grad_(True) if bias else None
    y = attorch_amd.LayerNormAutoGrad.apply(xd, wd, bd, 1e-5, True)
    y.backward(dy.cuda())
    assert y.dtype is dtype and y.shape == x.shape
    assert_close(y, y_ref, dtype, 'output')
    # With one to four features the input gradient is a difference of nearly equal terms
    # scaled by inv_std (up to 1/sqrt(eps)): ill-conditioned, so those rows get the tolerance of
    # the reference's own test (tests/test_layer_norm_layer.py:109, rtol = atol = 1e-3).
    assert_close(xd.grad, dx_ref, dtype, 'input_grad', reference_tolerance=feat <= 4)
    if affine:
        assert_close(wd.grad, dw_ref.to(dtype), dtype, 'weight_grad', batch_reduction=True)
    if bias:
        assert_close(bd.grad, db_ref.to(dtype), dtype, 'bias_grad', batch_reduction=True)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('affine', [False, True])
@pytest.mark.parametrize('eps', [None, 1e-5])
def test_rms_norm(shape, dtype, affine, eps) -> None:
    feat = shape[-1]
    x = randn(shape, 1, dtype)
    w = randn((feat,), 2, dtype, 0.1, 1.0) if affine else None
    dy = randn(shape, 4, dtype)
    cd = compute_dtype(dtype)
    y_ref, inv_rms = oracle.rms_norm_forward(x, w, eps, compute=cd)
    dx_ref, dw_ref = oracle.rms_norm_backward(dy, x, inv_rms, w, compute=cd)

    xd = x.cuda().requires_grad_(True)
    wd = w.cuda().requires_grad_(True) if affine else None
    y = attorch_amd.RMSNormAutoGrad.apply(xd, wd, eps)
    y.backward(dy.cuda())
    assert y.dtype is dtype
    assert_close(y, y_ref, dtype, 'output')
    # same conditioning remark as for LayerNorm (tests/test_rms_norm_layer.py:87-100 uses 1e-3)
    assert_close(xd.grad, dx_ref, dtype, 'input_grad', reference_tolerance=feat <= 4)
    if affine:
        assert_close(wd.grad, dw_ref.to(dtype), dtype, 'weight_grad', batch_reduction=True)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('neg, log', [(False, False), (False, True), (True, False)])
def test_softmax_family(shape, dtype, neg, log) -> None:
    x = randn(shape, 1, dtype, 2.0)
    dy = randn(shape, 2, dtype)
    cd = compute_dtype(dtype)
    y_ref = oracle.softmax_forward(x, neg, log, dtype, compute=cd)

    xd = x.cuda().requires_grad_(True)
    y = attorch_amd.SoftmaxAutoGrad.apply(xd, neg, log)
    y.backward(dy.cuda())
    assert y.dtype is dtype
    assert_close(y, y_ref, dtype, 'output')
    # backward starts from the saved (rounded) output, so feed the oracle the device's own
    assert_close(xd.grad, oracle.softmax_backward(dy, y.detach().cpu(), neg, log, compute=cd), dtype,
                 'input_grad')


def test_modules_and_autocast() -> None:
    x = randn((16, 256), 1, torch.float16).cuda().requires_grad_(True)
    layer_norm = attorch_amd.LayerNorm(256)
    rms_norm = attorch_amd.RMSNorm(256, eps=1e-6, dtype=torch.float16)
    with torch.autocast('cuda', dtype=torch.float16):
        assert layer_norm(x).dtype is torch.float32             # 'fp32' autocast policy
        assert attorch_amd.Softmax(dim=-1)(x).dtype is torch.float32
        assert attorch_amd.LogSoftmax(dim=1)(x).dtype is torch.float32
        assert rms_norm(x).dtype is torch.float16               # dtype flows through
        out = attorch_amd.LayerNorm(256, autocast_to_fp32=False, dtype=torch.float16)(x)
        assert out.dtype is torch.float16
    y = layer_norm(x.float())
    y.sum().backward()
    assert layer_norm.weight.grad.dtype is torch.float32 and layer_norm.weight.grad.shape == (256,)
    torch.testing.assert_close(attorch_amd.Softmin(dim=-1)(x.float()).sum(dim=-1),
                               torch.ones(16, device='cuda'))


def test_non_contiguous_and_repeatable() -> None:
    base = randn((64, 512), 1).cuda()
    x = base[:, ::2]                                            # strided view: wrapper must cope
    y = attorch_amd.SoftmaxAutoGrad.apply(x, False, False)
    torch.testing.assert_close(y, torch.softmax(x, dim=-1), rtol=1e-4, atol=1e-5)
    rows = base[::2]                                            # row stride 1024, unit inner stride
    w = torch.ones(512, device='cuda', requires_grad=True)
    a = attorch_amd.LayerNormAutoGrad.apply(rows.clone().requires_grad_(True), w, None, 1e-5, True)
    b = attorch_amd.LayerNormAutoGrad.apply(rows, w, None, 1e-5, True)
    assert torch.equal(a, b)                                    # bit-reproducible, stride-agnostic
