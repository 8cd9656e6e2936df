"""
GPU parity tests of Conv2d / Conv1d (forward and the three gradients) and BatchNorm1d/2d
(training statistics, running statistics, residual, fused activation, eval mode) against the
CPU oracle; grids follow the reference's tests/test_conv_layer.py and
tests/test_batch_norm_layer.py.
"""

import pytest
import torch

import attorch_amd
import oracle
from .helpers import DTYPES, assert_close, compute_dtype, randn

pytestmark = pytest.mark.gpu

CONV_CASES = [
    # input shape, out channels, kernel, stride, padding, groups
    ((2, 8, 11, 9), 12, (3, 3), (1, 1), (1, 1), 1),
    ((2, 8, 11, 9), 12, (5, 3), (2, 1), (3, 0), 2),
    ((2, 8, 11, 9), 8, (2, 4), (1, 2), (1, 3), 8),
    ((2, 6, 12, 12), 6, (1, 1), (1, 1), (0, 0), 1),
    ((1, 3, 64, 64), 16, (7, 7), (2, 2), (3, 3), 1),
    ((2, 16, 9, 9), 32, (4, 4), (2, 2), (2, 2), 4),
    ((4, 64, 28, 28), 64, (3, 3), (1, 1), (1, 1), 1),
    ((2, 32, 14, 14), 48, (3, 5), (2, 1), (1, 2), 1),
    # channel counts per group in multiples of 64: the 16-bit dtypes take the matrix-core path;
    # odd spatial sizes, partial tiles, groups, strides and asymmetric kernels on purpose
    ((3, 64, 7, 7), 96, (3, 3), (1, 1), (1, 1), 1),
    ((2, 128, 10, 12), 128, (3, 3), (2, 2), (1, 1), 2),
    ((2, 128, 9, 8), 64, (1, 1), (1, 1), (0, 0), 1),
    ((1, 64, 12, 10), 64, (5, 3), (1, 1), (2, 0), 1),
    ((5, 64, 20, 24), 64, (3, 3), (1, 1), (1, 1), 1),
    # contraction channels per group that are not multiples of 64 (padded with zero channels in the
    # channels-last copy) and strided layers, whose input gradient runs over the spread-out gradient
    ((2, 32, 14, 14), 64, (3, 3), (1, 1), (1, 1), 1),
    ((2, 96, 9, 11), 80, (3, 3), (1, 1), (1, 1), 1),
    ((2, 96, 12, 12), 96, (3, 3), (2, 2), (1, 1), 2),
    ((3, 64, 15, 17), 128, (3, 3), (2, 2), (1, 1), 1),
    ((2, 128, 10, 10), 64, (1, 1), (2, 2), (0, 0), 1),
    ((2, 16, 8, 9), 16, (3, 3), (1, 2), (1, 1), 1),
    # thin groups take the direct kernels: depthwise with a channel multiplier and more taps than
    # one accumulation pass holds, a pooling-shaped depthwise layer, a three-channel stem (input
    # gradient only), and few output channels without groups
    ((3, 12, 17, 15), 24, (5, 5), (2, 1), (2, 2), 12),
    ((4, 32, 30, 30), 32, (2, 2), (2, 2), (0, 0), 32),
    ((2, 3, 20, 20), 40, (7, 7), (2, 2), (3, 3), 1),
    ((2, 20, 13, 13), 6, (3, 3), (1, 1), (1, 1), 1),
]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape, out_dim, kernel, stride, padding, groups', CONV_CASES)
@pytest.mark.parametrize('bias', [False, True])
def test_conv2d(shape, out_dim, kernel, stride, padding, groups, bias, dtype) -> None:
    fan_in = shape[1] // groups * kernel[0] * kernel[1]
    x = randn(shape, 1, dtype)
    w = randn((out_dim, shape[1] // groups, *kernel), 2, dtype, fan_in ** -0.5)
    b = randn((out_dim,), 3, dtype) if bias else None
    cd = compute_dtype(dtype)
    y_ref = oracle.conv2d_forward(x, w, b, stride, padding, groups, dtype, compute=cd)
    dy = randn(y_ref.shape, 4, dtype)
    dx_ref, dw_ref, db_ref = oracle.conv2d_backward(dy, x, w, stride, padding, groups, dtype, compute=cd)

    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    bd = b.cuda().requires_grad_(True) if bias else None
    y = attorch_amd.Conv2dAutoGrad.apply(xd, wd, bd, *stride, *padding, groups)
    y.backward(dy.cuda())
    assert y.dtype is dtype
    assert_close(y, y_ref, dtype, 'output')
    assert_close(xd.grad, dx_ref, dtype, 'input_grad')
    assert_close(wd.grad, dw_ref, dtype, 'weight_grad', batch_reduction=True)
    if bias:
        assert_close(bd.grad, db_ref, dtype, 'bias_grad', batch_reduction=True)


def test_conv_modules_match_torch() -> None:
    torch.manual_seed(0)
    ours = attorch_amd.Conv2d(8, 16, 3, stride=2, padding=1, groups=2)
    torch.manual_seed(0)
    theirs = torch.nn.Conv2d(8, 16, 3, stride=2, padding=1, groups=2, device='cuda')
    x = randn((3, 8, 17, 13), 1).cuda()
    torch.testing.assert_close(ours(x), theirs(x), rtol=1e-4, atol=1e-5)
    torch.manual_seed(0)
    ours1d = attorch_amd.Conv1d(6, 4, 5, stride=2, padding=2)
    torch.manual_seed(0)
    theirs1d = torch.nn.Conv1d(6, 4, 5, stride=2, padding=2, device='cuda')
    x1 = randn((3, 6, 50), 2).cuda()
    torch.testing.assert_close(ours1d(x1), theirs1d(x1), rtol=1e-4, atol=1e-5)
    with torch.autocast('cuda', dtype=torch.float16):
        assert ours(x).dtype is torch.float16


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_conv_matrix_core_path_agrees_with_generic_kernel(dtype) -> None:
    """
    Straight through the C ABI: with its workspace the 16-bit convolution runs on the matrix
    cores from channels-last copies, without it on the generic gather kernel; both must agree
    to 16-bit rounding, and the shared channels-last copies must not change a result.
    """
    from attorch_amd import _lib
    lib = _lib.load()
    n, c, h, w, o, k = 3, 64, 9, 10, 128, 3
    dims = (n, c, h, w, o, h, w, k, k, 1, 1, 1, 1, 1)
    dt = _lib.dtype_id(dtype)
    x = randn((n, c, h, w), 1, dtype).cuda()
    wt = randn((o, c, k, k), 2, dtype, (c * k * k) ** -0.5).cuda()
    dy = randn((n, o, h, w), 3, dtype).cuda()
    stream = _lib.stream_of(x)

    def workspace(n_bytes):
        assert n_bytes > 0
        return torch.empty(n_bytes, dtype=torch.uint8, device='cuda'), n_bytes

    ws_f, nb_f = workspace(lib.at_conv2d_fwd_workspace_bytes(*dims, dt, dt))
    ws_x, nb_x = workspace(lib.at_conv2d_bwd_input_workspace_bytes(*dims, dt))
    ws_w, nb_w = workspace(lib.at_conv2d_bwd_weight_workspace_bytes(*dims, dt))
    y_fast, y_slow = torch.empty_like(dy), torch.empty_like(dy)
    _lib.check(lib.at_conv2d_fwd(_lib.ptr(x), _lib.ptr(wt), None, _lib.ptr(y_fast), _lib.ptr(ws_f), nb_f,
                                 *dims, dt, dt, dt, stream), 'fwd')
    _lib.check(lib.at_conv2d_fwd(_lib.ptr(x), _lib.ptr(wt), None, _lib.ptr(y_slow), None, 0,
                                 *dims, dt, dt, dt, stream), 'fwd')
    assert_close(y_fast, y_slow.cpu(), dtype, 'output')
    # the forward workspace starts with the channels-last input
    x_nhwc = ws_f[:x.numel() * 2].view(dtype).view(n, h, w, c)
    assert torch.equal(x_nhwc, x.permute(0, 2, 3, 1))

    dy_nhwc = torch.empty_like(dy)
    _lib.check(lib.at_nchw_to_nhwc(_lib.ptr(dy), _lib.ptr(dy_nhwc), n, o, h * w, dt, stream), 'nhwc')
    assert torch.equal(dy_nhwc.view(n, h, w, o), dy.permute(0, 2, 3, 1))

    dx_own, dx_shared, dx_slow = (torch.empty_like(x) for _ in range(3))
    _lib.check(lib.at_conv2d_bwd_input(_lib.ptr(dy), None, _lib.ptr(wt), _lib.ptr(dx_own), _lib.ptr(ws_x), nb_x,
                                       *dims, dt, stream), 'dx')
    _lib.check(lib.at_conv2d_bwd_input(_lib.ptr(dy), _lib.ptr(dy_nhwc), _lib.ptr(wt), _lib.ptr(dx_shared),
                                       _lib.ptr(ws_x), nb_x, *dims, dt, stream), 'dx')
    _lib.check(lib.at_conv2d_bwd_input(_lib.ptr(dy), None, _lib.ptr(wt), _lib.ptr(dx_slow), None, 0,
                                       *dims, dt, stream), 'dx')
    assert torch.equal(dx_own, dx_shared)
    assert_close(dx_own, dx_slow.cpu(), dtype, 'input_grad')

    dw_own, dw_shared = torch.empty_like(wt), torch.empty_like(wt)
    _lib.check(lib.at_conv2d_bwd_weight(_lib.ptr(dy), None, _lib.ptr(x), None, _lib.ptr(dw_own), _lib.ptr(ws_w),
                                        nb_w, *dims, dt, stream), 'dw')
    _lib.check(lib.at_conv2d_bwd_weight(_lib.ptr(dy), _lib.ptr(dy_nhwc), _lib.ptr(x), _lib.ptr(ws_f),
                                        _lib.ptr(dw_shared), _lib.ptr(ws_w), nb_w, *dims, dt, stream), 'dw')
    assert torch.equal(dw_own, dw_shared)
    # a weight-gradient call without workspace is an error, not a silent fallback
    assert lib.at_conv2d_bwd_weight(_lib.ptr(dy), None, _lib.ptr(x), None, _lib.ptr(dw_own), None, 0,
                                    *dims, dt, stream) == -5


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('n, c, h, w, o, pad, groups, bias', [
    (44, 64, 56, 56, 64, 1, 1, False),     # the ResNet 3x3 / 64-channel layer, whole 16-byte output segments
    (40, 64, 57, 59, 96, 1, 1, True),      # odd image (element stores), second channel tile partly empty
    (44, 128, 56, 56, 128, 1, 2, True),    # two groups of 64 channels
    (44, 64, 58, 58, 64, 0, 1, False),     # no padding: output smaller than the input
    (41, 64, 56, 56, 64, 2, 1, False),     # padding wider than the filter reach (forward only)
    (96, 64, 23, 23, 64, 1, 1, False),     # two output rows per k-tile of the weight gradient, odd row count
    (128, 128, 7, 7, 192, 1, 1, True),     # whole 7x7 images per k-tile, several channel tiles
    # more than 8 tiles per CU: the kernel that keeps the 3x3 x 64-channel weights in registers and walks over tiles
    (88, 64, 56, 56, 64, 1, 1, True),
    (90, 64, 55, 55, 128, 1, 1, True),     # last tile partly empty, two channel tiles
    (96, 128, 56, 56, 128, 1, 2, False),   # two groups
    (100, 64, 57, 57, 40, 1, 1, True),     # element stores, channel tile partly empty
    (128, 64, 56, 56, 64, 1, 1, True),     # the benchmark's layer at its batch size
    (140, 64, 30, 84, 40, 1, 1, False),    # wide, short images; channel tile partly empty
])
def test_conv_window_kernel_agrees_with_generic_kernel_at_size(n, c, h, w, o, pad, groups, bias, dtype) -> None:
    """
    ResNet-sized 3x3 layers (hundreds of tiles per CU, image borders, odd images, groups, a partly
    empty channel tile): the matrix-core window kernel, forward and input gradient, must agree with
    the generic gather kernel (same C ABI call without workspace) to 16-bit rounding.
    """
    from attorch_amd import _lib
    lib = _lib.load()
    k = 3
    oh, ow = h + 2 * pad - k + 1, w + 2 * pad - k + 1
    dims = (n, c, h, w, o, oh, ow, k, k, 1, 1, pad, pad, groups)
    dt = _lib.dtype_id(dtype)
    x = randn((n, c, h, w), 1, dtype).cuda()
    wt = randn((o, c // groups, k, k), 2, dtype, (c // groups * k * k) ** -0.5).cuda()
    b = randn((o,), 4, dtype).cuda() if bias else None
    dy = randn((n, o, oh, ow), 3, dtype).cuda()
    stream = _lib.stream_of(x)
    nb_f = lib.at_conv2d_fwd_workspace_bytes(*dims, dt, dt)
    assert nb_f > 0
    ws_f = torch.empty(nb_f, dtype=torch.uint8, device='cuda')
    y_fast = torch.full_like(dy, float('nan'))
    y_slow = torch.empty_like(dy)
    _lib.check(lib.at_conv2d_fwd(_lib.ptr(x), _lib.ptr(wt), _lib.ptr(b), _lib.ptr(y_fast), _lib.ptr(ws_f), nb_f,
                                 *dims, dt, dt, dt, stream), 'fwd')
    _lib.check(lib.at_conv2d_fwd(_lib.ptr(x), _lib.ptr(wt), _lib.ptr(b), _lib.ptr(y_slow), None, 0,
                                 *dims, dt, dt, dt, stream), 'fwd')
    assert_close(y_fast, y_slow.cpu(), dtype, 'output')
    # weight gradient: the matrix-core path (all taps per workgroup for pad 1) against torch in fp32
    nb_w = lib.at_conv2d_bwd_weight_workspace_bytes(*dims, dt)
    ws_w = torch.empty(nb_w, dtype=torch.uint8, device='cuda')
    dw_fast = torch.full_like(wt, float('nan'))
    _lib.check(lib.at_conv2d_bwd_weight(_lib.ptr(dy), None, _lib.ptr(x), None, _lib.ptr(dw_fast), _lib.ptr(ws_w),
                                        nb_w, *dims, dt, stream), 'dw')
    dw_ref = torch.nn.grad.conv2d_weight(x.float(), wt.shape, dy.float(), stride=1, padding=pad, groups=groups)
    assert_close(dw_fast, dw_ref.cpu(), dtype, 'weight_grad', batch_reduction=True)
    nb_x = lib.at_conv2d_bwd_input_workspace_bytes(*dims, dt)
    if pad > k - 1:
        assert nb_x == 0                    # the input gradient as a convolution needs pad <= k - 1
        return
    ws_x = torch.empty(nb_x, dtype=torch.uint8, device='cuda')
    dx_fast = torch.full_like(x, float('nan'))
    dx_slow = torch.empty_like(x)
    _lib.check(lib.at_conv2d_bwd_input(_lib.ptr(dy), None, _lib.ptr(wt), _lib.ptr(dx_fast), _lib.ptr(ws_x), nb_x,
                                       *dims, dt, stream), 'dx')
    _lib.check(lib.at_conv2d_bwd_input(_lib.ptr(dy), None, _lib.ptr(wt), _lib.ptr(dx_slow), None, 0,
                                       *dims, dt, stream), 'dx')
    assert_close(dx_fast, dx_slow.cpu(), dtype, 'input_grad')


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('n, c, h, w, o, groups', [
    (64, 72, 14, 14, 40, 1),       # channel counts that are multiples of 8 only: partly empty 64-wide tiles
    (48, 48, 30, 20, 96, 2),       # two groups, three output rows per k-tile, rows do not divide the image
    (256, 8, 9, 64, 16, 1),        # a full 64-pixel row per k-tile, very few channels
])
def test_conv_weight_gradient_all_taps_kernel(n, c, h, w, o, groups, dtype) -> None:
    """
    3x3 / stride 1 / padding 1 weight gradients large enough for the kernel that handles all taps
    in one workgroup, at channel counts and image shapes its tiles do not divide, against torch in
    fp32 from the same operands.
    """
    from attorch_amd import _lib
    lib = _lib.load()
    dims = (n, c, h, w, o, h, w, 3, 3, 1, 1, 1, 1, groups)
    dt = _lib.dtype_id(dtype)
    x = randn((n, c, h, w), 1, dtype).cuda()
    dy = randn((n, o, h, w), 3, dtype).cuda()
    nb = lib.at_conv2d_bwd_weight_workspace_bytes(*dims, dt)
    ws = torch.empty(nb, dtype=torch.uint8, device='cuda')
    dw = torch.full((o, c // groups, 3, 3), float('nan'), dtype=dtype, device='cuda')
    _lib.check(lib.at_conv2d_bwd_weight(_lib.ptr(dy), None, _lib.ptr(x), None, _lib.ptr(dw), _lib.ptr(ws), nb,
                                        *dims, dt, _lib.stream_of(x)), 'dw')
    ref = torch.nn.grad.conv2d_weight(x.float(), dw.shape, dy.float(), stride=1, padding=1, groups=groups)
    assert_close(dw, ref.cpu(), dtype, 'weight_grad', batch_reduction=True)


BN_SHAPES = [(6, 5), (128, 1024), (2048, 768), (300, 2048), (77, 40, 1), (260, 4104), (33, 6152), (8, 960, 196), (2048, 64, 16), (2, 3, 224, 224),
             (16, 64, 56, 56), (32, 128, 7, 7), (3, 7, 3, 5)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', BN_SHAPES)
@pytest.mark.parametrize('affine', [False, True])
@pytest.mark.parametrize('residual', [False, True])
@pytest.mark.parametrize('act_func', [None, 'relu', 'silu', 'leaky_relu_0.01'])
def test_batch_norm_training(shape, dtype, affine, residual, act_func) -> None:
    feat = shape[1]
    x = randn(shape, 1, dtype)
    w = randn((feat,), 2, dtype) if affine else None
    b = randn((feat,), 3, dtype) if affine else None
    res = randn(shape, 4, dtype) if residual else None
    dy = randn(shape, 5, dtype)
    running_mean = randn((feat,), 6)
    running_var = randn((feat,), 7).abs() + 0.5
    cd = compute_dtype(dtype)
    name, param = oracle.parse_act_func(act_func)
    y_ref, pre_act_ref, mean, inv_std, rm_ref, rv_ref = oracle.batch_norm_forward(
        x, True, w, b, running_mean, running_var, 0.2, 1e-5, True, res, name, param, compute=cd)

    xd = x.cuda().requires_grad_(True)
    wd = w.cuda().requires_grad_(True) if affine else None
    bd = b.cuda().requires_grad_(True) if affine else None
    rd = res.cuda().requires_grad_(True) if residual else None
    rm, rv = running_mean.cuda(), running_var.cuda()
    y = attorch_amd.BatchNormAutoGrad.apply(xd, True, wd, bd, rm, rv, 0.2, 1e-5, True, rd, act_func)
    saved = [None if t is None else t.detach().cpu() for t in y.grad_fn.saved_tensors]
    y.backward(dy.cuda())
    assert y.dtype is dtype and y.shape == x.shape
    assert_close(y, y_ref, dtype, 'output')
    assert_close(rm, rm_ref, torch.float32, 'running_mean')
    assert_close(rv, rv_ref, torch.float32, 'running_var')     # unbiased variance in the running stat

    pre_act = saved[4] if name is not None else None            # device's own pre-activation, see Linear test
    if name == 'relu':
        # relu has the same derivative at its output as at its input, so the layer keeps the output
        # in place of the pre-activation (and never writes the latter)
        assert_close(pre_act, y_ref, dtype, 'output kept for backward')
        assert torch.equal(pre_act > 0, pre_act_ref.to(dtype) > 0) or dtype is not torch.float32
    elif name is not None:
        assert_close(pre_act, pre_act_ref, dtype, 'pre_act')
    dx_ref, dw_ref, db_ref, dres_ref = oracle.batch_norm_backward(
        dy, x, saved[1], saved[2], w, affine, pre_act, name, param, compute=cd)
    assert_close(xd.grad, dx_ref, dtype, 'input_grad')
    if affine:
        assert_close(wd.grad, dw_ref.to(dtype), dtype, 'weight_grad', batch_reduction=True)
        assert_close(bd.grad, db_ref.to(dtype), dtype, 'bias_grad', batch_reduction=True)
    if residual:
        assert_close(rd.grad, dres_ref, dtype, 'residual_grad')


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('act_func', [None, 'relu'])
def test_batch_norm_eval_backward_follows_the_reference(act_func, dtype) -> None:
    """
    In eval mode the reference's backward (batch_norm_layer.py:191-245, no is_train argument)
    still applies the batch-statistics formula, with the running statistics in the place of the
    batch ones; torch treats them as constants.  The kernels keep the reference's result.
    """
    shape, feat = (6, 10, 7, 5), 10
    x, w, b = randn(shape, 1, dtype), randn((feat,), 2, dtype), randn((feat,), 3, dtype)
    res, dy = randn(shape, 4, dtype), randn(shape, 5, dtype)
    running_mean, running_var = randn((feat,), 6) * 0.1, randn((feat,), 7).abs() + 0.5
    cd = compute_dtype(dtype)
    name, param = oracle.parse_act_func(act_func)
    y_ref, _, mean, inv_std, rm_ref, rv_ref = oracle.batch_norm_forward(
        x, False, w, b, running_mean, running_var, 0.1, 1e-5, True, res, name, param, compute=cd)
    xd, rd = x.cuda().requires_grad_(True), res.cuda().requires_grad_(True)
    wd, bd = w.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    rm, rv = running_mean.cuda(), running_var.cuda()
    y = attorch_amd.BatchNormAutoGrad.apply(xd, False, wd, bd, rm, rv, 0.1, 1e-5, True, rd, act_func)
    saved = [None if t is None else t.detach().cpu() for t in y.grad_fn.saved_tensors]
    y.backward(dy.cuda())
    assert_close(y, y_ref, dtype, 'output')
    torch.testing.assert_close(rm.cpu(), running_mean), torch.testing.assert_close(rv.cpu(), running_var)
    assert_close(saved[1], running_mean, torch.float32, 'saved mean = running mean')
    dx_ref, dw_ref, db_ref, dres_ref = oracle.batch_norm_backward(
        dy, x, saved[1], saved[2], w, True, saved[4] if name is not None else None, name, param, compute=cd)
    assert_close(xd.grad, dx_ref, dtype, 'input_grad')
    assert_close(wd.grad, dw_ref.to(dtype), dtype, 'weight_grad', batch_reduction=True)
    assert_close(bd.grad, db_ref.to(dtype), dtype, 'bias_grad', batch_reduction=True)
    assert_close(rd.grad, dres_ref, dtype, 'residual_grad')


@pytest.mark.parametrize('track_running_stats', [False, True])
def test_batch_norm_modules_train_then_eval(track_running_stats) -> None:
    torch.manual_seed(0)
    ours = attorch_amd.BatchNorm2d(12, momentum=0.2, act_func='relu', track_running_stats=track_running_stats)
    theirs = torch.nn.BatchNorm2d(12, momentum=0.2, track_running_stats=track_running_stats, device='cuda')
    with torch.no_grad():
        ours.weight.normal_(), ours.bias.normal_()
        theirs.weight.copy_(ours.weight), theirs.bias.copy_(ours.bias)
    x, res = randn((8, 12, 9, 7), 1).cuda(), randn((8, 12, 9, 7), 2).cuda()
    for _ in range(2):
        torch.testing.assert_close(ours(x, res), torch.relu(theirs(x) + res), rtol=1e-4, atol=1e-5)
    if track_running_stats:
        torch.testing.assert_close(ours.running_mean, theirs.running_mean, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(ours.running_var, theirs.running_var, rtol=1e-4, atol=1e-5)
    ours.eval(), theirs.eval()
    torch.testing.assert_close(ours(x, res), torch.relu(theirs(x) + res), rtol=1e-4, atol=1e-5)
    ours1d = attorch_amd.BatchNorm1d(12)
    torch.testing.assert_close(ours1d(x.flatten(2)), torch.nn.BatchNorm1d(12, device='cuda')(x.flatten(2)),
                               rtol=1e-4, atol=1e-5)


def test_matrix_core_path_covers_padded_channels_and_strided_input_gradients() -> None:
    # which shapes get the 16-bit matrix-core path (a non-zero workspace request is how it shows)
    from attorch_amd import _lib
    lib = _lib.load()
    bf16 = _lib.dtype_id(torch.bfloat16)

    def dims(shape, out_dim, kernel, stride, padding, groups):
        n, c, h, w = shape
        oh = (h + 2 * padding[0] - kernel[0]) // stride[0] + 1
        ow = (w + 2 * padding[1] - kernel[1]) // stride[1] + 1
        return (n, c, h, w, out_dim, oh, ow, *kernel, *stride, *padding, groups)

    for case in (((2, 32, 14, 14), 64, (3, 3), (1, 1), (1, 1), 1), ((2, 96, 12, 12), 96, (3, 3), (2, 2), (1, 1), 2),
                 ((3, 64, 15, 17), 128, (3, 3), (2, 2), (1, 1), 1), ((2, 16, 8, 9), 16, (3, 3), (1, 2), (1, 1), 1)):
        d = dims(*case)
        assert lib.at_conv2d_fwd_workspace_bytes(*d, bf16, bf16) > 0, case
        assert lib.at_conv2d_bwd_input_workspace_bytes(*d, bf16) > 0, case
    # fewer than 16 contraction channels per group, or strides beyond 2 x 2, stay on the other kernels
    d = dims((2, 8, 8, 8), 64, (3, 3), (1, 1), (1, 1), 1)
    assert lib.at_conv2d_fwd_workspace_bytes(*d, bf16, bf16) == 0
    d = dims((2, 64, 16, 16), 64, (3, 3), (3, 2), (1, 1), 1)
    assert lib.at_conv2d_bwd_input_workspace_bytes(*d, bf16) == 0


CHANNELS_LAST_CASES = [
    # shape, out_dim, kernel, stride, padding, groups
    ((4, 64, 28, 28), 64, (3, 3), (1, 1), (1, 1), 1),      # every product stays channels-last
    ((3, 64, 7, 9), 96, (3, 3), (1, 1), (1, 1), 1),        # partial tiles; 96 output channels: dX falls back
    ((2, 128, 10, 12), 128, (3, 3), (2, 2), (1, 1), 2),    # groups, strided: dX falls back
    ((2, 128, 9, 8), 64, (1, 1), (1, 1), (0, 0), 1),
    ((1, 64, 12, 10), 64, (5, 3), (1, 1), (2, 0), 1),
    ((2, 32, 14, 14), 64, (3, 3), (1, 1), (1, 1), 1),      # 32 input channels: the forward product falls back
    # enough steps of 8 rows x 28 columns for every resident workgroup: image rows in a ring of LDS slots
    ((74, 64, 56, 28), 64, (3, 3), (1, 1), (1, 1), 1),     # one band
    ((44, 64, 30, 84), 48, (3, 3), (1, 1), (1, 1), 1),     # three bands, 6 rows in the last step, 48 output channels
    ((30, 64, 57, 52), 72, (3, 3), (1, 1), (1, 1), 1),     # last band 24 columns, one row in the last step, two channel tiles
    ((38, 128, 56, 56), 128, (3, 3), (1, 1), (1, 1), 2),   # two groups
]


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('shape, out_dim, kernel, stride, padding, groups', CHANNELS_LAST_CASES)
@pytest.mark.parametrize('bias', [False, True])
def test_conv2d_channels_last(shape, out_dim, kernel, stride, padding, groups, bias, dtype) -> None:
    # tensors in torch.channels_last memory format: same values as the oracle, and the layout is kept
    fan_in = shape[1] // groups * kernel[0] * kernel[1]
    x = randn(shape, 1, dtype)
    w = randn((out_dim, shape[1] // groups, *kernel), 2, dtype, fan_in ** -0.5)
    b = randn((out_dim,), 3, dtype) if bias else None
    cd = compute_dtype(dtype)
    y_ref = oracle.conv2d_forward(x, w, b, stride, padding, groups, dtype, compute=cd)
    dy = randn(y_ref.shape, 4, dtype)
    dx_ref, dw_ref, db_ref = oracle.conv2d_backward(dy, x, w, stride, padding, groups, dtype, compute=cd)

    xd = x.cuda().contiguous(memory_format=torch.channels_last).requires_grad_(True)
    wd = w.cuda().requires_grad_(True)
    bd = b.cuda().requires_grad_(True) if bias else None
    y = attorch_amd.Conv2dAutoGrad.apply(xd, wd, bd, *stride, *padding, groups)
    y.backward(dy.cuda().contiguous(memory_format=torch.channels_last))
    assert y.dtype is dtype and y.shape == y_ref.shape
    if shape[1] // groups % 64 == 0:
        assert y.is_contiguous(memory_format=torch.channels_last)
    assert_close(y, y_ref, dtype, 'output')
    assert_close(xd.grad, dx_ref, dtype, 'input_grad')
    assert_close(wd.grad, dw_ref, dtype, 'weight_grad', batch_reduction=True)
    if bias:
        assert_close(bd.grad, db_ref, dtype, 'bias_grad', batch_reduction=True)


def test_conv2d_channels_last_matches_channels_first_bitwise() -> None:
    # the same kernels run on both layouts: identical results for the block of BASELINE config 5
    dtype = torch.bfloat16
    x = randn((8, 64, 56, 56), 1, dtype).cuda()
    w = randn((64, 64, 3, 3), 2, dtype, 576 ** -0.5).cuda()
    dy = randn((8, 64, 56, 56), 3, dtype).cuda()
    results = []
    for fmt in (torch.contiguous_format, torch.channels_last):
        xd = x.detach().clone(memory_format=fmt).requires_grad_(True)
        wd = w.clone().requires_grad_(True)
        y = attorch_amd.Conv2dAutoGrad.apply(xd, wd, None, 1, 1, 1, 1, 1)
        y.backward(dy.contiguous(memory_format=fmt))
        results.append((y.detach(), xd.grad, wd.grad))
    assert results[1][0].is_contiguous(memory_format=torch.channels_last)
    assert results[1][1].is_contiguous(memory_format=torch.channels_last)
    for first, last in zip(*results):
        assert torch.equal(first, last)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('batch, feat, spatial', [(5, 7, 64), (3, 5, 63), (130, 3, 1000), (1, 1, 8), (2, 9, 1)])
def test_channel_sum(batch, feat, spatial, dtype) -> None:
    # the bias gradient of a channels-first tensor, output_grad.sum((0, 2, 3)) (conv_layer.py:162):
    # planes that are whole 16-byte vectors and planes that are not
    from attorch_amd import _lib
    lib = _lib.load()
    x = randn((batch, feat, spatial), 5, dtype).cuda()
    out = torch.empty(feat, dtype=dtype, device='cuda')
    dt = _lib.dtype_id(dtype)
    _lib.check(lib.at_channel_sum(_lib.ptr(x), _lib.ptr(out), batch, feat, spatial, dt, dt, _lib.stream_of(x)),
               'at_channel_sum')
    assert_close(out, x.double().sum((0, 2)).cpu(), dtype, 'channel sum', batch_reduction=True)


@pytest.mark.parametrize('shape, out_dim, bias', [((88, 64, 56, 56), 64, True), ((90, 64, 55, 55), 40, False),
                                                  ((128, 64, 56, 56), 64, True), ((100, 64, 57, 56), 40, False)])
def test_conv2d_weights_resident_kernel_same_on_both_layouts(shape, out_dim, bias) -> None:
    # batch sizes at which a workgroup walks over several tiles with the weights in registers
    dtype = torch.bfloat16
    x = randn(shape, 1, dtype).cuda()
    w = randn((out_dim, shape[1], 3, 3), 2, dtype, 576 ** -0.5).cuda()
    b = randn((out_dim,), 4, dtype).cuda() if bias else None
    dy = randn((shape[0], out_dim, shape[2], shape[3]), 3, dtype).cuda()
    results = []
    for fmt in (torch.contiguous_format, torch.channels_last):
        xd = x.detach().clone(memory_format=fmt).requires_grad_(True)
        wd = w.clone().requires_grad_(True)
        y = attorch_amd.Conv2dAutoGrad.apply(xd, wd, b, 1, 1, 1, 1, 1)
        y.backward(dy.contiguous(memory_format=fmt))
        results.append((y.detach(), xd.grad, wd.grad))
    for first, last in zip(*results):
        assert torch.equal(first, last)
    ref = torch.nn.functional.conv2d(x.float(), w.float(), None if b is None else b.float(), 1, 1)
    assert_close(results[1][0], ref.cpu(), dtype, 'output')


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(4, 64, 7, 7), (2, 96, 5, 6), (3, 8, 4, 4), (5, 24, 3, 5), (2, 2048, 2, 3), (2, 4104, 3, 2),
                                   # every power of two of 16-byte chunks per row up to a wave's 64, over enough
                                   # rows for several rounds of loads per lane
                                   (16, 512, 9, 9), (8, 256, 7, 9), (8, 128, 14, 14), (6, 32, 31, 17),
                                   (32, 16, 12, 10), (9, 64, 33, 35)])
@pytest.mark.parametrize('affine, residual, act_func', [(True, True, 'relu'), (False, False, None),
                                                        (True, False, 'silu'), (True, True, 'leaky_relu_0.01')])
def test_batch_norm_channels_last(shape, dtype, affine, residual, act_func) -> None:
    # torch.channels_last tensors: a [batch * height * width, feat] matrix with statistics per column
    feat = shape[1]
    x = randn(shape, 1, dtype)
    w = randn((feat,), 2, dtype) if affine else None
    b = randn((feat,), 3, dtype) if affine else None
    res = randn(shape, 4, dtype) if residual else None
    dy = randn(shape, 5, dtype)
    running_mean = randn((feat,), 6)
    running_var = randn((feat,), 7).abs() + 0.5
    cd = compute_dtype(dtype)
    name, param = oracle.parse_act_func(act_func)
    y_ref, pre_act_ref, mean, inv_std, rm_ref, rv_ref = oracle.batch_norm_forward(
        x, True, w, b, running_mean, running_var, 0.2, 1e-5, True, res, name, param, compute=cd)

    last = torch.channels_last
    xd = x.cuda().contiguous(memory_format=last).requires_grad_(True)
    wd = w.cuda().requires_grad_(True) if affine else None
    bd = b.cuda().requires_grad_(True) if affine else None
    rd = res.cuda().contiguous(memory_format=last).requires_grad_(True) if residual else None
    rm, rv = running_mean.cuda(), running_var.cuda()
    y = attorch_amd.BatchNormAutoGrad.apply(xd, True, wd, bd, rm, rv, 0.2, 1e-5, True, rd, act_func)
    saved = [None if t is None else t.detach().cpu() for t in y.grad_fn.saved_tensors]
    y.backward(dy.cuda().contiguous(memory_format=last))
    vec = 4 if dtype is torch.float32 else 8
    supported = feat % vec == 0     # otherwise the layer converts to channels-first
    if supported:
        assert y.is_contiguous(memory_format=last) and xd.grad.is_contiguous(memory_format=last)
    assert_close(y, y_ref, dtype, 'output')
    assert_close(rm, rm_ref, torch.float32, 'running_mean')
    assert_close(rv, rv_ref, torch.float32, 'running_var')
    assert_close(saved[1], mean, torch.float32, 'mean')
    pre_act = saved[4] if name is not None else None
    dx_ref, dw_ref, db_ref, dres_ref = oracle.batch_norm_backward(
        dy, x, saved[1], saved[2], w, affine, pre_act, name, param, compute=cd)
    assert_close(xd.grad, dx_ref, dtype, 'input_grad')
    if affine:
        assert_close(wd.grad, dw_ref.to(dtype), dtype, 'weight_grad', batch_reduction=True)
        assert_close(bd.grad, db_ref.to(dtype), dtype, 'bias_grad', batch_reduction=True)
    if residual:
        assert_close(rd.grad, dres_ref, dtype, 'residual_grad')


def test_batch_norm_channels_last_eval_and_block() -> None:
    # evaluation mode on running statistics, and conv -> batch norm staying channels-last end to end
    dtype = torch.bfloat16
    last = torch.channels_last
    x = randn((4, 64, 14, 14), 1, dtype).cuda()
    conv = attorch_amd.Conv2d(64, 64, 3, padding=1, bias=False, dtype=dtype)
    bn = attorch_amd.BatchNorm2d(64, act_func='relu', dtype=dtype)
    results = []
    for fmt in (torch.contiguous_format, last):
        xin = x.detach().clone(memory_format=fmt).requires_grad_(True)
        bn.train()
        bn.running_mean.zero_(), bn.running_var.fill_(1.0)
        out = bn(conv(xin), xin)
        out.float().square().mean().backward()
        bn.eval()
        with torch.no_grad():
            out_eval = bn(conv(xin), xin)
        results.append((out.detach(), xin.grad, out_eval, conv.weight.grad.clone(), bn.weight.grad.clone()))
        conv.weight.grad = None
        bn.weight.grad = bn.bias.grad = None
        if fmt is last:
            assert out.is_contiguous(memory_format=last) and xin.grad.is_contiguous(memory_format=last)
            assert out_eval.is_contiguous(memory_format=last)
    names = ('output', 'input_grad', 'eval output', 'conv weight_grad', 'bn weight_grad')
    for name, first, second in zip(names, *results):
        assert_close(second, first.cpu(), dtype, name, batch_reduction='weight_grad' in name)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_channels_last_layers_take_an_upstream_gradient_in_the_default_format(dtype) -> None:
    """
    A channels-last Conv2d / BatchNorm2d whose upstream gradient arrives NCHW-contiguous (another
    operator produced it) converts it with the library's transpose: same gradients, bit for bit, as
    with a channels-last upstream gradient.
    """
    x = randn((6, 64, 20, 24), 1, dtype).cuda().contiguous(memory_format=torch.channels_last)
    w = randn((64, 64, 3, 3), 2, dtype, 576 ** -0.5).cuda()
    res = randn((6, 64, 20, 24), 5, dtype).cuda().contiguous(memory_format=torch.channels_last)
    dy = randn((6, 64, 20, 24), 3, dtype).cuda()
    assert dy.is_contiguous() and not dy.is_contiguous(memory_format=torch.channels_last)
    results = []
    for grad in (dy, dy.contiguous(memory_format=torch.channels_last)):
        xd, wd, rd = x.clone().requires_grad_(True), w.clone().requires_grad_(True), res.clone().requires_grad_(True)
        bn = attorch_amd.BatchNorm2d(64, act_func='relu', device='cuda', dtype=dtype)
        y = bn(attorch_amd.Conv2dAutoGrad.apply(xd, wd, None, 1, 1, 1, 1, 1), rd)
        assert y.is_contiguous(memory_format=torch.channels_last)
        y.backward(grad)
        results.append((xd.grad, wd.grad, rd.grad, bn.weight.grad, bn.bias.grad))
    for a, b in zip(*results):
        assert torch.equal(a, b)
