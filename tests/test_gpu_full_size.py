"""
Full-size checks at the BASELINE configurations (c1-c5).  Where the CPU oracle finishes in
seconds the whole result is compared; otherwise a slice is compared against the oracle and
size-independent properties cover the rest (rows of a softmax gradient sum to zero, ignored
rows are exactly zero, a weight gradient over the batch is the sum of the gradients of its
halves, column sums match).
"""

import pytest
import torch

import attorch_amd
import oracle
from .helpers import assert_close, randn

pytestmark = pytest.mark.gpu
BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32


def test_c1_linear_fp32_relu() -> None:
    x = randn((512, 784), 1001)
    torch.manual_seed(1002)
    lin = torch.nn.Linear(784, 256)
    w, b = lin.weight.detach().T.contiguous(), lin.bias.detach()
    dy = randn((512, 256), 1003)
    xd, wd, bd = (t.cuda().requires_grad_(True) for t in (x, w, b))
    y = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, 'relu')
    pre_act = y.grad_fn.saved_tensors[1].detach().cpu()
    y.backward(dy.cuda())
    y_ref, _ = oracle.linear_forward(x, w, b, 'relu', None, F32, compute=torch.float64)
    dx_ref, dw_ref, db_ref = oracle.linear_backward(dy, x, w, pre_act, 'relu', None, F32, compute=torch.float64)
    assert_close(y, y_ref, F32, 'output')
    assert_close(xd.grad, dx_ref, F32, 'input_grad')
    assert_close(wd.grad, dw_ref, F32, 'weight_grad', batch_reduction=True)
    assert_close(bd.grad, db_ref, F32, 'bias_grad', batch_reduction=True)


def test_c2_norms_and_softmax_bf16() -> None:
    shape = (8192, 4096)
    x, dy = randn(shape, 2001, BF16), randn(shape, 2002, BF16)
    w, b = randn((4096,), 2003, BF16, 0.1, 1.0), randn((4096,), 2004, BF16, 0.1)
    xd, wd, bd = (t.cuda().requires_grad_(True) for t in (x, w, b))
    y = attorch_amd.LayerNormAutoGrad.apply(xd, wd, bd, 1e-5, True)
    y.backward(dy.cuda())
    y_ref, mean, inv_std = oracle.layer_norm_forward(x, w, b, 1e-5, BF16)
    dx_ref, dw_ref, db_ref = oracle.layer_norm_backward(dy, x, mean, inv_std, w, BF16)
    assert_close(y, y_ref, BF16, 'layer_norm output')
    assert_close(xd.grad, dx_ref, BF16, 'layer_norm input_grad')
    assert_close(wd.grad, dw_ref.to(BF16), BF16, 'layer_norm weight_grad', batch_reduction=True)
    assert_close(bd.grad, db_ref.to(BF16), BF16, 'layer_norm bias_grad', batch_reduction=True)

    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    y = attorch_amd.RMSNormAutoGrad.apply(xd, wd, 1e-5)
    y.backward(dy.cuda())
    y_ref, inv_rms = oracle.rms_norm_forward(x, w, 1e-5)
    dx_ref, dw_ref = oracle.rms_norm_backward(dy, x, inv_rms, w)
    assert_close(y, y_ref, BF16, 'rms_norm output')
    assert_close(xd.grad, dx_ref, BF16, 'rms_norm input_grad')
    assert_close(wd.grad, dw_ref.to(BF16), BF16, 'rms_norm weight_grad', batch_reduction=True)

    for log in (False, True):
        xd = x.cuda().requires_grad_(True)
        y = attorch_amd.SoftmaxAutoGrad.apply(xd, False, log)
        y.backward(dy.cuda())
        assert_close(y, oracle.softmax_forward(x, False, log, BF16), BF16, f'softmax(log={log}) output')
        assert_close(xd.grad, oracle.softmax_backward(dy, y.detach().cpu(), False, log), BF16,
                     f'softmax(log={log}) input_grad')


@pytest.mark.parametrize('weighted', [False, True])
def test_c3_cross_entropy_fp16(weighted) -> None:
    rows, vocab = 8192, 50257
    logits = randn((rows, vocab), 3001, F16, 2.0)
    gen = torch.Generator().manual_seed(3002)
    target = torch.randint(0, vocab, (rows,), generator=gen)
    target[torch.rand(rows, generator=gen) < 0.05] = -100
    weight = 0.5 + torch.rand(vocab, generator=gen) if weighted else None
    xd = logits.cuda().requires_grad_(True)
    loss = attorch_amd.CrossEntropyLossAutoGrad.apply(xd, target.cuda(), None if weight is None else weight.cuda(),
                                                      -100)
    loss.backward()
    grad = xd.grad

    # loss: the oracle row by row in slices, combined with the global divisor
    keep = target != -100
    row_w = (weight[target.clamp(min=0)] if weighted else torch.ones(rows)) * keep
    denom = row_w.sum().double()
    total = torch.zeros((), dtype=torch.float64)
    for start in range(0, rows, 1024):
        sl = slice(start, start + 1024)
        part, part_denom = oracle.cross_entropy_forward(logits[sl], target[sl], weight, -100, torch.float64)
        total += part * part_denom.double()
    assert_close(loss, (total / denom).float(), F16, 'loss')

    # gradient: a slice against the oracle (rescaled from the slice's divisor to the global one)
    sl = slice(4096, 4096 + 256)
    local = row_w[sl].sum().double()
    ref = oracle.cross_entropy_backward((local / denom).float(), logits[sl], target[sl], weight, -100, F32)
    kept = float(keep.sum())
    assert_close(grad[sl].float() * kept, ref * kept, F16, 'input_grad slice')
    # properties over the full gradient
    assert torch.all(grad[(~keep).cuda()] == 0), 'ignored rows must be exactly zero'
    # (softmax - onehot rows sum to zero only before rounding: with ~7800 kept rows most
    # probabilities / kept fall below fp16's smallest subnormal, so the row sums sit in [-1, 0])
    row_sums = grad.float().sum(dim=1) * kept / (row_w.cuda() * kept / float(denom)).clamp(min=1e-30)
    assert row_sums.max().item() < 0.05 and row_sums.min().item() > -1.05
    picked = grad[torch.arange(rows)[keep].cuda(), target[keep].cuda()]
    assert torch.all(picked < 0), 'the target column of every kept row has a negative gradient'


def test_c4_linear_bf16_gelu() -> None:
    """
    Every element of the output, the saved pre-activation and the three gradients against the
    oracle, which runs the whole 6.6 TFLOP step on the host in row blocks.  No reference value
    depends on anything the device computed.
    """
    m, k, n = 16384, 4096, 16384
    x, w, b = randn((m, k), 4001, BF16), randn((k, n), 4002, BF16, 0.02), torch.zeros(n, dtype=BF16)
    dy = randn((m, n), 4003, BF16)
    xd, wd, bd = (t.cuda().requires_grad_(True) for t in (x, w, b))
    y = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, 'geluapprox')
    pre_act = y.grad_fn.saved_tensors[1].detach()
    y.backward(dy.cuda())
    y, dx, dw, db = y.detach(), xd.grad, wd.grad, bd.grad

    wf = w.float()
    dw_sum = torch.zeros((k, n), dtype=F32)
    db_sum = torch.zeros(n, dtype=torch.float64)
    block = 2048
    for r0 in range(0, m, block):
        rows = slice(r0, r0 + block)
        y_ref, pre_ref = oracle.linear_forward(x[rows], w, b, 'geluapprox', None, BF16)
        assert_close(y[rows], y_ref, BF16, f'output rows {r0}..')
        assert_close(pre_act[rows], pre_ref, BF16, f'pre_act rows {r0}..')
        dz = (dy[rows].float() * oracle.act_grad(pre_ref.float(), 'geluapprox')).to(BF16)
        assert_close(dx[rows], (dz.float() @ wf.T).to(BF16), BF16, f'input_grad rows {r0}..')
        dw_sum += x[rows].float().T @ dz.float()
        db_sum += dz.double().sum(dim=0)
    assert_close(dw, dw_sum.to(BF16), BF16, 'weight_grad', batch_reduction=True)
    assert_close(db, db_sum.float().to(BF16), BF16, 'bias_grad', batch_reduction=True)


def test_c4_linear_autocast_fp16() -> None:
    """
    The c4 layer the way the reference's examples run it: float32 input and parameters under
    torch.autocast(float16).  Operands and bias are rounded to float16 for the product
    (linear_kernels.py:161-163,171-172), output and saved pre-activation are float16, the
    backward products run in float16 and autograd widens the gradients to float32.
    One row of every 256-row tile (all columns) for the output, the pre-activation and the
    input gradient; a band of output features over the whole batch for the weight and bias
    gradients, its reference pre-activation computed on the host.
    """
    m, k, n = 16384, 4096, 16384
    x, w, b = randn((m, k), 4011), randn((k, n), 4012, F32, 0.02), randn((n,), 4013, F32, 0.1)
    dy = randn((m, n), 4014, F16)
    xd, wd, bd = (t.cuda().requires_grad_(True) for t in (x, w, b))
    with torch.autocast('cuda', dtype=F16):
        y = attorch_amd.LinearAutoGrad.apply(xd, wd, bd, 'geluapprox')
    assert y.dtype is F16
    pre_act = y.grad_fn.saved_tensors[1].detach()
    assert pre_act.dtype is F16
    # the saved operands are the float16 copies the forward product read, not float32 tensors
    assert y.grad_fn.saved_tensors[0].dtype is F16 and y.grad_fn.saved_tensors[2].dtype is F16
    y.backward(dy.cuda())
    assert xd.grad.dtype is F32 and wd.grad.dtype is F32 and bd.grad.dtype is F32

    rows = torch.tensor([t * 256 + (t * 37) % 256 for t in range(m // 256)] + [0, m - 1])
    y_ref, pre_ref = oracle.linear_forward(x[rows], w, b, 'geluapprox', None, F16)
    assert_close(y[rows.cuda()], y_ref, F16, 'output rows')
    assert_close(pre_act[rows.cuda()], pre_ref, F16, 'pre_act rows')
    dx_ref, _, _ = oracle.linear_backward(dy[rows], x[rows], w, pre_ref, 'geluapprox', None, F16)
    assert_close(xd.grad[rows.cuda()], dx_ref.float(), F16, 'input_grad rows')

    cols = torch.cat([torch.arange(0, 8), torch.arange(8190, 8198), torch.arange(n - 8, n)])
    x16, w16 = x.to(F16).float(), w[:, cols].to(F16).float()
    pre_band = (x16 @ w16 + b[cols].to(F16).float()).to(F16)
    dz_band = (dy[:, cols].float() * oracle.act_grad(pre_band.float(), 'geluapprox')).to(F16)
    assert_close(wd.grad[:, cols.cuda()], (x16.T @ dz_band.float()).to(F16).float(), F16, 'weight_grad band',
                 batch_reduction=True)
    assert_close(bd.grad[cols.cuda()], dz_band.float().sum(dim=0).to(F16).float(), F16, 'bias_grad band',
                 batch_reduction=True)


def test_c5_conv_bn_residual_relu_bf16() -> None:
    n, c, h, w_ = 128, 64, 56, 56
    x, res, dy = randn((n, c, h, w_), 5001, BF16), randn((n, c, h, w_), 5002, BF16), randn((n, c, h, w_), 5003, BF16)
    torch.manual_seed(5004)
    wt = torch.nn.init.kaiming_normal_(torch.empty(c, c, 3, 3)).to(BF16)
    xd, wd = x.cuda().requires_grad_(True), wt.cuda().requires_grad_(True)
    conv_out = attorch_amd.Conv2dAutoGrad.apply(xd, wd, None, 1, 1, 1, 1, 1)
    conv_out.backward(dy.cuda())
    sub = slice(60, 64)
    assert_close(conv_out[sub], oracle.conv2d_forward(x[sub], wt, None, (1, 1), (1, 1), 1, BF16), BF16,
                 'conv output slice')
    dx_ref, dw_sub_ref, _ = oracle.conv2d_backward(dy[sub], x[sub], wt, (1, 1), (1, 1), 1, BF16)
    assert_close(xd.grad[sub], dx_ref, BF16, 'conv input_grad slice')
    # weight gradient: the slice alone against the oracle, the full batch as the sum of its halves
    halves = []
    for part in (slice(0, 64), slice(64, 128), sub):
        xp, wp = x[part].cuda().requires_grad_(True), wt.cuda().requires_grad_(True)
        attorch_amd.Conv2dAutoGrad.apply(xp, wp, None, 1, 1, 1, 1, 1).backward(dy[part].cuda())
        halves.append(wp.grad.float())
    assert_close(halves[2], dw_sub_ref, BF16, 'conv weight_grad slice', batch_reduction=True)
    assert_close(wd.grad.float(), halves[0] + halves[1], BF16, 'conv weight_grad additivity', batch_reduction=True)

    bn_w, bn_b = randn((c,), 5005, BF16, 0.1, 1.0), randn((c,), 5006, BF16, 0.1)
    rm, rv = torch.zeros(c), torch.ones(c)
    conv_cpu = conv_out.detach().cpu()
    cd, rd = conv_out.detach().requires_grad_(True), res.cuda().requires_grad_(True)
    wdv, bdv = bn_w.cuda().requires_grad_(True), bn_b.cuda().requires_grad_(True)
    rmd, rvd = rm.cuda(), rv.cuda()
    out = attorch_amd.BatchNormAutoGrad.apply(cd, True, wdv, bdv, rmd, rvd, 0.1, 1e-5, True, rd, 'relu')
    saved = [t.detach().cpu() for t in out.grad_fn.saved_tensors]
    out.backward(dy.cuda())
    out_ref, _, _, _, rm_ref, rv_ref = oracle.batch_norm_forward(conv_cpu, True, bn_w, bn_b, rm, rv, 0.1, 1e-5, True,
                                                                 res, 'relu', None)
    assert_close(out, out_ref, BF16, 'batch_norm output')
    assert_close(rmd, rm_ref, F32, 'running_mean')
    assert_close(rvd, rv_ref, F32, 'running_var')
    dx_ref, dw_ref, db_ref, dres_ref = oracle.batch_norm_backward(dy, conv_cpu, saved[1], saved[2], bn_w, True, saved[4],
                                                                  'relu', None)
    assert_close(cd.grad, dx_ref, BF16, 'batch_norm input_grad')
    assert_close(wdv.grad, dw_ref.to(BF16), BF16, 'batch_norm weight_grad', batch_reduction=True)
    assert_close(bdv.grad, db_ref.to(BF16), BF16, 'batch_norm bias_grad', batch_reduction=True)
    assert_close(rd.grad, dres_ref, BF16, 'batch_norm residual_grad')


def test_batch_norm_of_2_gib_and_more() -> None:
    """
    The passes that sum over a channel read tensors below 2 GiB through a buffer resource; from
    that size on they keep plain pointers.  [2, 16, 8200, 4100] bf16 is 2.15 GB: residual and
    ReLU fused, forward and backward.  The device's own batch_norm in float32 is the checker at
    this size (the CPU oracle would take minutes on a billion elements); tolerances of bf16.
    """
    dtype = torch.bfloat16
    shape = (2, 16, 8200, 4100)
    assert shape[0] * shape[1] * shape[2] * shape[3] * 2 >= 1 << 31
    gen = torch.Generator(device='cuda').manual_seed(11)
    x = torch.randn(shape, device='cuda', dtype=dtype, generator=gen).mul_(1.5).add_(0.25).requires_grad_(True)
    res = torch.randn(shape, device='cuda', dtype=dtype, generator=gen).requires_grad_(True)
    dy = torch.randn(shape, device='cuda', dtype=dtype, generator=gen)
    w = (1 + 0.1 * torch.randn(16, device='cuda', generator=gen)).to(dtype).requires_grad_(True)
    b = (0.1 * torch.randn(16, device='cuda', generator=gen)).to(dtype).requires_grad_(True)
    rm, rv = torch.zeros(16, device='cuda', dtype=dtype), torch.ones(16, device='cuda', dtype=dtype)
    out = attorch_amd.BatchNormAutoGrad.apply(x, True, w, b, rm, rv, 0.1, 1e-5, True, res, 'relu')
    out.backward(dy)

    xr, rr = x.detach().float().requires_grad_(True), res.detach().float().requires_grad_(True)
    wr, br = w.detach().float().requires_grad_(True), b.detach().float().requires_grad_(True)
    rm_ref, rv_ref = torch.zeros(16, device='cuda'), torch.ones(16, device='cuda')
    pre = torch.nn.functional.batch_norm(xr, rm_ref, rv_ref, wr, br, True, 0.1, 1e-5) + rr
    ref = torch.relu(pre)
    ref.backward(dy.float())
    rtol, atol = 2e-2, 2e-2
    # Where the pre-activation is within float32 rounding of zero, the two sides may land on
    # different sides of the ReLU and differ by a whole gradient: a few in a million elements,
    # left out of the gradient comparison.
    boundary = pre.detach().abs() <= 1e-4
    assert boundary.sum().item() < 1e-4 * boundary.numel()
    del pre

    def check(actual, expected, what, skip=None):
        wrong = (actual.float() - expected).abs() > atol + rtol * expected.abs()
        if skip is not None:
            wrong &= ~skip
        bad = wrong.sum().item()
        assert bad == 0, f'{what}: {bad} elements out of tolerance'

    check(out, ref.detach(), 'output')
    del ref
    check(x.grad, xr.grad, 'input_grad', boundary)
    check(res.grad, rr.grad, 'residual_grad', boundary)
    scale = max(1.0, wr.grad.abs().max().item())
    check(w.grad / scale, wr.grad / scale, 'weight_grad')
    scale = max(1.0, br.grad.abs().max().item())
    check(b.grad / scale, br.grad / scale, 'bias_grad')
    check(rm, rm_ref, 'running_mean')
    check(rv, rv_ref, 'running_var')
