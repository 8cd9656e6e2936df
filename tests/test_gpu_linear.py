"""
GPU parity tests of Linear (fused GEMM + bias + activation, both backward products, bias
gradient) against the CPU oracle; parameter grid follows the reference's
tests/test_linear_layer.py and adds 'geluapprox', bfloat16 and tile-edge shapes.
"""

import pytest
import torch

import attorch_amd
import oracle
from .helpers import ACT_FUNCS, DTYPES, assert_close, compute_dtype, randn

pytestmark = pytest.mark.gpu


def run_case(shape, out_dim, bias, act_func, dtype) -> None:
    in_dim = shape[-1]
    x = randn(shape, 1, dtype)
    w = randn((in_dim, out_dim), 2, dtype, in_dim ** -0.5)
    b = randn((out_dim,), 3, dtype, 0.1) if bias else None
    dy = randn((*shape[:-1], out_dim), 4, dtype)
    cd = compute_dtype(dtype)
    name, param = oracle.parse_act_func(act_func)

    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    bd = b.cuda().requires_grad_(True) if bias else None
    y = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, act_func)
    saved_pre_act = y.grad_fn.saved_tensors[1]
    saved_pre_act = None if saved_pre_act is None else saved_pre_act.detach().cpu()
    y.backward(dy.cuda())
    assert y.dtype is dtype and tuple(y.shape) == (*shape[:-1], out_dim)

    y_ref, pre_act_ref = oracle.linear_forward(x, w, b, name, param, dtype, compute=cd)
    assert_close(y, y_ref, dtype, 'output')
    # The activation derivative is discontinuous for the piecewise activations: evaluate the
    # oracle's backward at the pre-activation the device saved (compared separately above
    # through the output), so a last-bit difference cannot flip a branch.
    pre_act = None
    if name is not None:
        pre_act = saved_pre_act
        assert_close(pre_act, pre_act_ref, dtype, 'pre_act')
    dx_ref, dw_ref, db_ref = oracle.linear_backward(dy, x, w, pre_act, name, param, dtype, compute=cd)
    assert_close(xd.grad, dx_ref, dtype, 'input_grad', normalize=True)
    assert_close(wd.grad, dw_ref, dtype, 'weight_grad', normalize=True)
    assert tuple(wd.grad.shape) == (in_dim, out_dim)
    if bias:
        assert_close(bd.grad, db_ref, dtype, 'bias_grad', normalize=True)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape, out_dim', [((4, 2000), 96), ((8, 1024), 16), ((32, 1024), 128),
                                            ((2048, 768), 768), ((6144, 256), 384), ((8096, 32), 196),
                                            ((12288, 1), 512), ((1, 1024, 3072), 1024), ((8, 960, 196), 128),
                                            ((512, 784), 256), ((300, 264), 520), ((513, 512), 257),
                                            ((256, 72), 256), ((1000, 1000), 1000)])
@pytest.mark.parametrize('bias', [False, True])
@pytest.mark.parametrize('act_func', [None, 'relu', 'geluapprox'])
def test_linear_shapes(shape, out_dim, bias, act_func, dtype) -> None:
    run_case(shape, out_dim, bias, act_func, dtype)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('act_func', ACT_FUNCS)
@pytest.mark.parametrize('shape, out_dim', [((64, 96), 80), ((512, 256), 512)])
def test_linear_every_activation(shape, out_dim, act_func, dtype) -> None:
    run_case(shape, out_dim, True, act_func, dtype)


def test_module_matches_torch_linear_and_autocast() -> None:
    torch.manual_seed(0)
    ours = attorch_amd.Linear(384, 192, act_func='silu')
    torch.manual_seed(0)
    theirs = torch.nn.Linear(384, 192, device='cuda')
    torch.testing.assert_close(ours.weight, theirs.weight.T.contiguous())
    x = randn((50, 384), 1).cuda()
    torch.testing.assert_close(ours(x), torch.nn.functional.silu(theirs(x)), rtol=1e-4, atol=1e-5)
    with torch.autocast('cuda', dtype=torch.float16):
        y16 = ours(x)
    assert y16.dtype is torch.float16                                      # 'fp16' autocast policy
    torch.testing.assert_close(y16.float(), torch.nn.functional.silu(theirs(x)), rtol=2e-2, atol=2e-2)
    with torch.autocast('cuda', dtype=torch.bfloat16):
        assert ours(x).dtype is torch.bfloat16


def test_no_grad_path_saves_nothing() -> None:
    x = randn((128, 256), 1).cuda()
    w = randn((256, 256), 2).cuda()
    y = attorch_amd.LinearAutoGrad.apply(x, w, None, 'relu')
    assert y.grad_fn is None
    torch.testing.assert_close(y, torch.relu(x @ w), rtol=1e-4, atol=1e-4)
