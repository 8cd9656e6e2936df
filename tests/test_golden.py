"""
Golden-vector tests: tests/golden/hot_path_small.npz (written by tests/golden/make_golden.py
from torch.nn.functional in float64) pins the CPU oracle here and the HIP kernels in the
gpu-marked half.
"""

from pathlib import Path

import numpy as np
import pytest
import torch

import oracle

GOLDEN = np.load(Path(__file__).resolve().parent / 'golden' / 'hot_path_small.npz')
D = torch.float64


def g(key, dtype=D):
    value = torch.from_numpy(GOLDEN[key])
    return value if value.dtype == torch.int64 else value.to(dtype)


def check(actual, key, rtol=1e-9, atol=1e-10):
    expected = g(key)
    torch.testing.assert_close(actual.detach().cpu().to(D), expected, rtol=rtol, atol=atol,
                               msg=lambda m: f'{key}: {m}')


def test_oracle_matches_golden_vectors() -> None:
    w = g('linear.w').T.contiguous()
    y, pre = oracle.linear_forward(g('linear.x'), w, g('linear.b'), 'geluapprox', None, D, compute=D)
    dx, dw, db = oracle.linear_backward(g('linear.dy'), g('linear.x'), w, pre, 'geluapprox', None, D, compute=D)
    check(y, 'linear.y', 1e-7, 1e-7), check(dx, 'linear.dx', 1e-7, 1e-7)
    check(dw.T, 'linear.dw', 1e-7, 1e-7), check(db, 'linear.db', 1e-7, 1e-7)

    x, wt, b, dy = g('layer_norm.x'), g('layer_norm.w'), g('layer_norm.b'), g('layer_norm.dy')
    y, mean, inv_std = oracle.layer_norm_forward(x, wt, b, 1e-5, D, compute=D)
    dx, dw, db = oracle.layer_norm_backward(dy, x, mean, inv_std, wt, D, compute=D)
    check(y, 'layer_norm.y'), check(dx, 'layer_norm.dx'), check(dw, 'layer_norm.dw'), check(db, 'layer_norm.db')
    y, inv_rms = oracle.rms_norm_forward(x, wt, 1e-6, compute=D)
    dx, dw = oracle.rms_norm_backward(dy, x, inv_rms, wt, compute=D)
    check(y, 'rms_norm.y'), check(dx, 'rms_norm.dx'), check(dw, 'rms_norm.dw')

    x, dy = g('softmax.x'), g('softmax.dy')
    for name, neg, log in (('softmax', False, False), ('log_softmax', False, True), ('softmin', True, False)):
        y = oracle.softmax_forward(x, neg, log, D, compute=D)
        check(y, f'{name}.y'), check(oracle.softmax_backward(dy, y, neg, log, compute=D), f'{name}.dx')

    x, t, wt = g('cross_entropy.x'), g('cross_entropy.target'), g('cross_entropy.w')
    loss, _ = oracle.cross_entropy_forward(x, t, wt, -100, D, compute=D)
    check(loss, 'cross_entropy.loss')
    check(oracle.cross_entropy_backward(torch.tensor(1.0, dtype=D), x, t, wt, -100, D, compute=D), 'cross_entropy.dx')

    x, wt, b, dy = g('conv2d.x'), g('conv2d.w'), g('conv2d.b'), g('conv2d.dy')
    check(oracle.conv2d_forward(x, wt, b, (2, 1), (1, 1), 2, D, compute=D), 'conv2d.y')
    dx, dw, db = oracle.conv2d_backward(dy, x, wt, (2, 1), (1, 1), 2, D, compute=D)
    check(dx, 'conv2d.dx'), check(dw, 'conv2d.dw'), check(db, 'conv2d.db')

    x, wt, b, res, dy = (g(f'batch_norm.{k}') for k in ('x', 'w', 'b', 'res', 'dy'))
    y, pre, mean, inv_std, rm, rv = oracle.batch_norm_forward(x, True, wt, b, g('batch_norm.rm0'), g('batch_norm.rv0'),
                                                              0.1, 1e-5, True, res, 'relu', None, compute=D)
    check(y, 'batch_norm.y'), check(rm, 'batch_norm.rm1'), check(rv, 'batch_norm.rv1')
    dx, dw, db, dres = oracle.batch_norm_backward(dy, x, mean, inv_std, wt, True, pre, 'relu', None, compute=D)
    check(dx, 'batch_norm.dx'), check(dw, 'batch_norm.dw'), check(db, 'batch_norm.db'), check(dres, 'batch_norm.dres')


@pytest.mark.gpu
def test_hip_kernels_match_golden_vectors() -> None:
    import attorch_amd
    F32 = torch.float32
    tol = dict(rtol=1e-4, atol=1e-5)

    def dev(key, grad=True):
        t = g(key, F32).cuda()
        return t.requires_grad_(True) if grad and t.is_floating_point() else t

    x, w, b = dev('linear.x'), g('linear.w', F32).T.contiguous().cuda().requires_grad_(True), dev('linear.b')
    y = attorch_amd.LinearAutoGrad.apply(x, w, b, 'geluapprox')
    y.backward(dev('linear.dy', False))
    check(y, 'linear.y', **tol), check(x.grad, 'linear.dx', **tol)
    check(w.grad.T, 'linear.dw', 1e-4, 1e-4), check(b.grad, 'linear.db', 1e-4, 1e-4)

    x, w, b, dy = dev('layer_norm.x'), dev('layer_norm.w'), dev('layer_norm.b'), dev('layer_norm.dy', False)
    y = attorch_amd.LayerNormAutoGrad.apply(x, w, b, 1e-5, True)
    y.backward(dy)
    check(y, 'layer_norm.y', **tol), check(x.grad, 'layer_norm.dx', **tol)
    check(w.grad, 'layer_norm.dw', 1e-4, 1e-4), check(b.grad, 'layer_norm.db', 1e-4, 1e-4)
    x, w = dev('layer_norm.x'), dev('layer_norm.w')
    y = attorch_amd.RMSNormAutoGrad.apply(x, w, 1e-6)
    y.backward(dy)
    check(y, 'rms_norm.y', **tol), check(x.grad, 'rms_norm.dx', **tol), check(w.grad, 'rms_norm.dw', 1e-4, 1e-4)

    for name, neg, log in (('softmax', False, False), ('log_softmax', False, True), ('softmin', True, False)):
        x = dev('softmax.x')
        y = attorch_amd.SoftmaxAutoGrad.apply(x, neg, log)
        y.backward(dev('softmax.dy', False))
        check(y, f'{name}.y', **tol), check(x.grad, f'{name}.dx', **tol)

    x = dev('cross_entropy.x')
    loss = attorch_amd.CrossEntropyLossAutoGrad.apply(x, dev('cross_entropy.target'), dev('cross_entropy.w', False), -100)
    loss.backward()
    check(loss, 'cross_entropy.loss', **tol), check(x.grad, 'cross_entropy.dx', **tol)

    x, w, b = dev('conv2d.x'), dev('conv2d.w'), dev('conv2d.b')
    y = attorch_amd.Conv2dAutoGrad.apply(x, w, b, 2, 1, 1, 1, 2)
    y.backward(dev('conv2d.dy', False))
    check(y, 'conv2d.y', **tol), check(x.grad, 'conv2d.dx', **tol)
    check(w.grad, 'conv2d.dw', 1e-4, 1e-4), check(b.grad, 'conv2d.db', 1e-4, 1e-4)

    x, w, b, res = dev('batch_norm.x'), dev('batch_norm.w'), dev('batch_norm.b'), dev('batch_norm.res')
    rm, rv = dev('batch_norm.rm0', False), dev('batch_norm.rv0', False)
    y = attorch_amd.BatchNormAutoGrad.apply(x, True, w, b, rm, rv, 0.1, 1e-5, True, res, 'relu')
    y.backward(dev('batch_norm.dy', False))
    check(y, 'batch_norm.y', **tol), check(rm, 'batch_norm.rm1', **tol), check(rv, 'batch_norm.rv1', **tol)
    check(x.grad, 'batch_norm.dx', **tol), check(w.grad, 'batch_norm.dw', 1e-4, 1e-4)
    check(b.grad, 'batch_norm.db', 1e-4, 1e-4), check(res.grad, 'batch_norm.dres', **tol)
