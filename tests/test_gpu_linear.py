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
    # dX sums out_dim products of dy (unit scale) and w (scale in_dim ** -0.5)
    assert_close(xd.grad, dx_ref, dtype, 'input_grad', dot_terms=out_dim, term_scale=in_dim ** -0.5)
    assert_close(wd.grad, dw_ref, dtype, 'weight_grad', batch_reduction=True)
    assert tuple(wd.grad.shape) == (in_dim, out_dim)
    if bias:
        assert_close(bd.grad, db_ref, dtype, 'bias_grad', batch_reduction=True)


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


HALF_DTYPES = [torch.float16, torch.bfloat16]


@pytest.mark.parametrize('dtype', HALF_DTYPES)
@pytest.mark.parametrize('act_func', [None, 'geluapprox'])
@pytest.mark.parametrize('shape, out_dim', [
    ((1024, 333), 77),      # both feature sizes odd: the host pads input, weight and gradient
    ((512, 200), 1001),     # odd output size only (a vocabulary-like head)
    ((640, 257), 264),      # odd input size only
    ((4096, 512), 10),      # skinny output: generic 16-bit kernel, all waves along the batch
    ((96, 1000), 24),       # skinny output, contraction not a multiple of 64
    ((2048, 512), 384),     # 128x128 tiles
    ((4096, 256), 256),     # 128x128 tiles, weight gradient split over the batch
    ((16384, 192), 320),    # split with a ragged last k-tile range
    ((1000, 520), 776),     # 128x128 tiles, fewer than CUs: two k-groups per tile, an odd number of k-tiles
    # 256x256 tiles walked by a grid smaller than their number (each workgroup takes two), with
    # ragged last row and column tiles among full ones: forward, input gradient and weight
    # gradient in turn
    ((8100, 256), 4088),
    ((8100, 4088), 520),
    ((300, 8104), 4088),
])
def test_linear_16bit_kernel_selection(shape, out_dim, act_func, dtype) -> None:
    run_case(shape, out_dim, True, act_func, dtype)


@pytest.mark.parametrize('dtype', HALF_DTYPES)
@pytest.mark.parametrize('batch, in_dim, out_dim', [(4096, 256, 256), (8000, 320, 136), (1000, 264, 200)])
def test_weight_grad_split_agrees_with_one_piece(batch, in_dim, out_dim, dtype) -> None:
    """
    C ABI: at_linear_bwd_weight with its workspace (batch split into slices, fp32 partial sums)
    against the same call without one, and against float64.
    """
    from attorch_amd import _lib
    lib = _lib.load()
    x = randn((batch, in_dim), 1, dtype).cuda()
    dz = randn((batch, out_dim), 2, dtype).cuda()
    did = _lib.dtype_id(dtype)
    stream = _lib.stream_of(x)
    workspace_bytes = lib.at_linear_bwd_weight_workspace_bytes(batch, in_dim, out_dim, did)
    if batch >= 4096:
        assert workspace_bytes > 0
    results = []
    for use_workspace in (False, True):
        dw = torch.full((in_dim, out_dim), float('nan'), dtype=dtype, device='cuda')
        workspace = torch.empty(max(workspace_bytes, 16), dtype=torch.uint8, device='cuda') if use_workspace else None
        _lib.check(lib.at_linear_bwd_weight(
            _lib.ptr(x), _lib.ptr(dz), _lib.ptr(dw), _lib.ptr(workspace), workspace_bytes if use_workspace else 0,
            batch, in_dim, out_dim, in_dim, out_dim, out_dim, did, did, stream), 'at_linear_bwd_weight')
        results.append(dw.double().cpu())
    expected = x.double().cpu().T @ dz.double().cpu()
    scale = expected.abs().max().item()
    for got in results:
        torch.testing.assert_close(got / scale, expected / scale, rtol=2e-2, atol=2e-2 / 8)
    # both round the same fp32-accurate sums: they differ by an ulp of the 16-bit format at most
    torch.testing.assert_close(results[0] / scale, results[1] / scale, rtol=2 ** -7, atol=2 ** -9)
    # a short workspace is not an error: the one-piece path runs
    dw = torch.empty((in_dim, out_dim), dtype=dtype, device='cuda')
    tiny = torch.empty(16, dtype=torch.uint8, device='cuda')
    _lib.check(lib.at_linear_bwd_weight(
        _lib.ptr(x), _lib.ptr(dz), _lib.ptr(dw), _lib.ptr(tiny), 16, batch, in_dim, out_dim, in_dim, out_dim,
        out_dim, did, did, stream), 'at_linear_bwd_weight')
    torch.testing.assert_close(dw.double().cpu(), results[0], rtol=0, atol=0)


@pytest.mark.parametrize('batch, in_dim, out_dim', [(32768, 256, 256), (5000, 100, 96), (8192, 64, 384), (2048, 32, 36)])
def test_fp32_weight_grad_slices_of_the_batch(batch, in_dim, out_dim) -> None:
    """
    C ABI: a small fp32 weight gradient with a long batch is computed in slices of the batch when
    the caller passes the workspace (fixed-order sum of fp32 partial tiles); with and without it
    the result is the float64 product to fp32 accumulation error.
    """
    from attorch_amd import _lib
    lib = _lib.load()
    x = randn((batch, in_dim), 1).cuda()
    dz = randn((batch, out_dim), 2).cuda()
    stream = _lib.stream_of(x)
    workspace_bytes = lib.at_linear_bwd_weight_workspace_bytes(batch, in_dim, out_dim, 0)
    assert workspace_bytes > 0
    expected = x.double().cpu().T @ dz.double().cpu()
    for use_workspace in (False, True):
        dw = torch.full((in_dim, out_dim), float('nan'), device='cuda')
        workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device='cuda') if use_workspace else None
        _lib.check(lib.at_linear_bwd_weight(
            _lib.ptr(x), _lib.ptr(dz), _lib.ptr(dw), _lib.ptr(workspace), workspace_bytes if use_workspace else 0,
            batch, in_dim, out_dim, in_dim, out_dim, out_dim, 0, 0, stream), 'at_linear_bwd_weight')
        assert_close(dw, expected, torch.float32, f'weight_grad, workspace={use_workspace}', batch_reduction=True,
                     dot_terms=batch)


@pytest.mark.parametrize('dtype', DTYPES)
def test_extent_one_dimensions_with_arbitrary_strides(dtype) -> None:
    """
    PyTorch leaves the stride of an extent-1 dimension arbitrary: the [1, out] weight of a layer
    with one input feature is a transposed [out, 1] tensor whose stride(0) is 1, and a [feat, 1]
    tensor transposed to one row of feat elements reports a row stride of 1 as well.
    """
    lin = attorch_amd.Linear(1, 63, device='cuda', dtype=dtype)
    assert tuple(lin.weight.shape) == (1, 63) and lin.weight.stride(0) < 63
    x = randn((2048, 1), 1, dtype).cuda().requires_grad_(True)
    dy = randn((2048, 63), 2, dtype).cuda()
    y = lin(x)
    y.backward(dy)
    w, b = lin.weight.detach().double(), lin.bias.detach().double()
    assert_close(y, x.detach().double() @ w + b, dtype, 'output')
    assert_close(x.grad, dy.double() @ w.T, dtype, 'input_grad')
    assert_close(lin.weight.grad, x.detach().double().T @ dy.double(), dtype, 'weight_grad', batch_reduction=True)
    assert_close(lin.bias.grad, dy.double().sum(0), dtype, 'bias_grad', batch_reduction=True)

    row = randn((300, 1), 3, dtype).cuda().T            # one row of 300 elements, stride(0) == 1
    assert tuple(row.shape) == (1, 300) and row.stride(0) == 1
    row.requires_grad_(True)
    out = attorch_amd.Softmax(dim=-1)(row)
    out.backward(torch.ones_like(out) * torch.arange(300, device='cuda', dtype=dtype))
    ref_in = row.detach().double().requires_grad_(True)
    ref = torch.softmax(ref_in, dim=-1)
    ref.backward(torch.arange(300, device='cuda', dtype=dtype).double().expand(1, 300))
    assert_close(out, ref, dtype, 'softmax of one strided row')
    assert_close(row.grad, ref_in.grad, dtype, 'softmax input_grad')
    norm = attorch_amd.LayerNorm(300, device='cuda', dtype=dtype)
    assert_close(norm(row), torch.nn.functional.layer_norm(row.detach().double(), (300,), norm.weight.double(),
                                                           norm.bias.double(), norm.eps), dtype, 'layer norm')


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('act_func', [None, 'relu', 'geluapprox'])
@pytest.mark.parametrize('shape, out_dim', [((4096, 2048), 10), ((1000, 512), 1), ((37, 264), 16),
                                            ((3, 5, 1024), 7), ((130, 256), 13), ((2050, 768), 2)])
def test_linear_classifier_heads(shape, out_dim, act_func, dtype) -> None:
    """
    At most 16 output features with a wide, 16-byte aligned input: the three products run on the
    vector-ALU kernels (row counts that do not fill a workgroup, one to sixteen columns, several
    chunks of the contraction).
    """
    run_case(shape, out_dim, True, act_func, dtype)
    run_case(shape, out_dim, False, act_func, dtype)


SMALL_BWD_CASES = [
    # batch, in_feat, out_feat, act_func, bias, input needs a gradient
    (512, 784, 256, 'relu', True, True),         # the MNIST-sized layer
    (512, 784, 256, 'relu', True, False),        # first layer of a network: no input gradient
    (128, 36, 128, 'gelu', False, True),
    (200, 100, 132, None, True, True),           # no activation: dZ is the output gradient itself
    (1000, 260, 512, 'leaky_relu_0.01', True, True),
    (130, 1028, 640, 'geluapprox', True, True),
]


@pytest.mark.parametrize('batch, in_dim, out_dim, act_func, bias, input_grad', SMALL_BWD_CASES)
def test_small_fp32_backward_in_one_launch(batch, in_dim, out_dim, act_func, bias, input_grad) -> None:
    # shapes the one-launch backward serves: same results as the oracle, and as the three separate calls
    from attorch_amd import _lib
    lib = _lib.load()
    dtype = torch.float32
    assert lib.at_linear_bwd_small_supported(batch, in_dim, out_dim, _lib.dtype_id(dtype)) == 1
    x = randn((batch, in_dim), 1, dtype)
    w = randn((in_dim, out_dim), 2, dtype, in_dim ** -0.5)
    b = randn((out_dim,), 3, dtype, 0.1) if bias else None
    dy = randn((batch, out_dim), 4, dtype)
    name, param = oracle.parse_act_func(act_func)
    xd, wd = x.cuda().requires_grad_(input_grad), w.cuda().requires_grad_(True)
    bd = b.cuda().requires_grad_(True) if bias else None
    y = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, act_func)
    pre_act = y.grad_fn.saved_tensors[1]
    pre_act = None if pre_act is None else pre_act.detach()
    y.backward(dy.cuda())
    dx_ref, dw_ref, db_ref = oracle.linear_backward(dy, x, w, None if pre_act is None else pre_act.cpu(), name, param,
                                                    dtype, compute=torch.float64)
    if input_grad:
        assert_close(xd.grad, dx_ref, dtype, 'input_grad', dot_terms=out_dim, term_scale=in_dim ** -0.5)
    else:
        assert xd.grad is None
    assert_close(wd.grad, dw_ref, dtype, 'weight_grad', batch_reduction=True)
    if bias:
        assert_close(bd.grad, db_ref, dtype, 'bias_grad', batch_reduction=True)

    # the separate calls on the same operands
    stream = _lib.stream_of(xd)
    dyd, act = dy.cuda(), attorch_amd.act.act_id(name, param)
    dz = dyd
    if name is not None:
        dz = torch.empty_like(dyd)
        _lib.check(lib.at_act_bwd(dyd.data_ptr(), pre_act.data_ptr(), dz.data_ptr(), None, None, 0, batch, out_dim,
                                  out_dim, out_dim, out_dim, act, 0.0 if param is None else param, 0, 0, 0, stream),
                   'at_act_bwd')
    dw_sep = torch.empty_like(wd)
    _lib.check(lib.at_linear_bwd_weight(xd.data_ptr(), dz.data_ptr(), dw_sep.data_ptr(), None, 0, batch, in_dim,
                                        out_dim, in_dim, out_dim, out_dim, 0, 0, stream), 'at_linear_bwd_weight')
    assert_close(wd.grad, dw_sep.cpu(), dtype, 'weight_grad against the separate call', batch_reduction=True)
    if input_grad:
        dx_sep = torch.empty_like(xd)
        _lib.check(lib.at_linear_bwd_input(dz.data_ptr(), wd.data_ptr(), dx_sep.data_ptr(), batch, in_dim, out_dim,
                                           out_dim, out_dim, in_dim, 0, 0, stream), 'at_linear_bwd_input')
        assert_close(xd.grad, dx_sep.cpu(), dtype, 'input_grad against the separate call', dot_terms=out_dim,
                     term_scale=in_dim ** -0.5)


def test_small_backward_declines_other_shapes() -> None:
    from attorch_amd import _lib
    lib = _lib.load()
    f32, bf16 = _lib.dtype_id(torch.float32), _lib.dtype_id(torch.bfloat16)
    assert lib.at_linear_bwd_small_supported(512, 784, 256, bf16) == 0       # fp32 only
    assert lib.at_linear_bwd_small_supported(512, 783, 256, f32) == 0        # rows must allow 16-byte vectors
    assert lib.at_linear_bwd_small_supported(16384, 4096, 4096, f32) == 0    # large layers take the tiled products
    assert lib.at_linear_bwd_small_supported(64, 784, 256, f32) == 0
    t = torch.zeros(4, device='cuda')
    p = t.data_ptr()
    assert lib.at_linear_bwd_small(p, p, p, p, p, p, None, 512, 783, 256, 256, 256, 783, 256, 783, 256, 4, 0.0, f32,
                                   _lib.stream_of(t)) == -7                  # AT_ERR_UNSUPPORTED, nothing launched


@pytest.mark.parametrize('dtype', HALF_DTYPES)
@pytest.mark.parametrize('offset', [0, 7])
@pytest.mark.parametrize('input_grad', [True, False])
def test_padded_path_takes_a_column_slice_as_upstream_gradient(dtype, offset, input_grad) -> None:
    """
    16-bit layer whose output width is not a multiple of 8 (the zero-padded operand path), no
    activation, and an upstream gradient that is a column slice of a wider tensor whose row
    stride happens to equal the padded width — as the backward of a concatenation hands out.
    What lies outside the slice (NaN here) must never be read as padding.
    """
    batch, in_dim, out_dim, wide = 512, 200, 1001, 1008
    x = randn((batch, in_dim), 1, dtype)
    w = randn((in_dim, out_dim), 2, dtype, in_dim ** -0.5)
    b = randn((out_dim,), 3, dtype, 0.1)
    dy = randn((batch, out_dim), 4, dtype)
    holder = torch.full((batch, wide), float('nan'), dtype=dtype, device='cuda')
    upstream = holder[:, offset:offset + out_dim]
    upstream.copy_(dy)
    assert upstream.stride(0) == wide and not upstream.is_contiguous()
    xd, wd, bd = x.cuda().requires_grad_(input_grad), w.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    y = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, None)
    y.backward(upstream)
    dx_ref, dw_ref, db_ref = oracle.linear_backward(dy, x, w, None, None, None, dtype)
    if input_grad:
        assert_close(xd.grad, dx_ref, dtype, 'input_grad')
    assert_close(wd.grad, dw_ref, dtype, 'weight_grad', batch_reduction=True)
    assert_close(bd.grad, db_ref, dtype, 'bias_grad', batch_reduction=True)


@pytest.mark.parametrize('amp_dtype', HALF_DTYPES)
@pytest.mark.parametrize('act_func', [None, 'relu', 'geluapprox'])
@pytest.mark.parametrize('shape, out_dim', [((512, 256), 512), ((2048, 768), 768), ((4, 100, 333), 77),
                                            ((1024, 200), 1001), ((64, 96), 80)])
def test_linear_under_autocast_with_fp32_parameters(shape, out_dim, act_func, amp_dtype) -> None:
    """
    The reference's default training mode (examples/utils.py:13-36, tests/test_linear_layer.py
    amp=True): float32 input and parameters under torch.autocast.  Operands and bias are rounded
    to the autocast dtype for the product (linear_kernels.py:161-163,171-172), output and
    pre-activation have that dtype, and the gradients reach the float32 leaves as float32.
    """
    in_dim = shape[-1]
    x = randn(shape, 1)
    w = randn((in_dim, out_dim), 2, torch.float32, in_dim ** -0.5)
    b = randn((out_dim,), 3, torch.float32, 0.1)
    dy = randn((*shape[:-1], out_dim), 4, amp_dtype)
    name, param = oracle.parse_act_func(act_func)
    xd, wd, bd = (t.cuda().requires_grad_(True) for t in (x, w, b))
    with torch.autocast('cuda', dtype=amp_dtype):
        y = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, act_func)
    assert y.dtype is amp_dtype
    # nothing float32 and operand-sized is kept for backward: the casts made for the forward
    # product are (zero-padded layers keep the originals and pad afresh)
    saved = y.grad_fn.saved_tensors
    if in_dim % 8 == 0 and out_dim % 8 == 0:
        assert saved[0].dtype is amp_dtype and saved[2].dtype is amp_dtype
    pre_act = None if saved[1] is None else saved[1].detach().cpu()
    y.backward(dy.cuda())
    assert xd.grad.dtype is torch.float32 and wd.grad.dtype is torch.float32 and bd.grad.dtype is torch.float32
    y_ref, pre_ref = oracle.linear_forward(x, w, b, name, param, amp_dtype)
    assert_close(y, y_ref, amp_dtype, 'output')
    if name is not None:
        assert_close(pre_act, pre_ref, amp_dtype, 'pre_act')
    dx_ref, dw_ref, db_ref = oracle.linear_backward(dy, x, w, pre_act, name, param, amp_dtype)
    assert_close(xd.grad, dx_ref.float(), amp_dtype, 'input_grad')
    assert_close(wd.grad, dw_ref.float(), amp_dtype, 'weight_grad', batch_reduction=True)
    assert_close(bd.grad, db_ref.float(), amp_dtype, 'bias_grad', batch_reduction=True)
    # a second backward pass through a retained graph reads the same saved casts
    xd.grad = wd.grad = bd.grad = None
    with torch.autocast('cuda', dtype=amp_dtype):
        y2 = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, act_func)
    y2.backward(dy.cuda(), retain_graph=True)
    first = wd.grad.clone()
    wd.grad = None
    y2.backward(dy.cuda())
    torch.testing.assert_close(wd.grad, first, rtol=0, atol=0)


@pytest.mark.parametrize('dtype', HALF_DTYPES)
@pytest.mark.parametrize('batch, in_dim, out_dim', [
    (8100, 520, 4088),     # 256x256 tiles with ragged edges (input gradient) / 128x128 tiles
    (4096, 256, 256),      # 128x128 tiles, weight gradient split over the batch
    (2048, 512, 384),      # 128x128 tiles
    (300, 264, 520),       # generic kernel (small problem)
    (1000, 1000, 1000),
    (1000, 520, 776),      # two k-groups per tile, an odd number of k-tiles
])
def test_backward_products_write_fp32_like_a_cast_of_the_16bit_result(batch, in_dim, out_dim, dtype) -> None:
    """
    C ABI: at_linear_bwd_input / at_linear_bwd_weight with 16-bit operands and out_dtype = fp32 give
    exactly the 16-bit result widened (the product is rounded to the operand dtype first), whichever
    kernel serves the shape.
    """
    from attorch_amd import _lib
    lib = _lib.load()
    did, f32 = _lib.dtype_id(dtype), _lib.dtype_id(torch.float32)
    x = randn((batch, in_dim), 1, dtype).cuda()
    w = randn((in_dim, out_dim), 2, dtype, in_dim ** -0.5).cuda()
    dz = randn((batch, out_dim), 3, dtype).cuda()
    stream = _lib.stream_of(x)
    workspace_bytes = lib.at_linear_bwd_weight_workspace_bytes(batch, in_dim, out_dim, did)
    workspace = torch.empty(max(workspace_bytes, 16), dtype=torch.uint8, device='cuda')
    results = {}
    for out_dtype, oid in ((dtype, did), (torch.float32, f32)):
        dx = torch.full((batch, in_dim), float('nan'), dtype=out_dtype, device='cuda')
        dw = torch.full((in_dim, out_dim), float('nan'), dtype=out_dtype, device='cuda')
        _lib.check(lib.at_linear_bwd_input(dz.data_ptr(), w.data_ptr(), dx.data_ptr(), batch, in_dim, out_dim,
                                           out_dim, out_dim, in_dim, did, oid, stream), 'at_linear_bwd_input')
        _lib.check(lib.at_linear_bwd_weight(x.data_ptr(), dz.data_ptr(), dw.data_ptr(), workspace.data_ptr(),
                                            workspace_bytes, batch, in_dim, out_dim, in_dim, out_dim, out_dim,
                                            did, oid, stream), 'at_linear_bwd_weight')
        results[out_dtype] = (dx, dw)
    for narrow, wide, what in zip(results[dtype], results[torch.float32], ('input_grad', 'weight_grad')):
        assert wide.dtype is torch.float32
        assert torch.equal(narrow.float(), wide), what
    assert_close(results[dtype][0], dz.double().cpu() @ w.double().cpu().T, dtype, 'input_grad')
