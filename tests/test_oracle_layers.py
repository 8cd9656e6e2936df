"""
Pins oracle.layers against independent implementations: torch.nn.functional + autograd in
float64 (the oracle of the reference's own tests), brute-force loops on tiny inputs and
closed-form invariants.  Each check is chosen so that a dropped term, a wrong sign or a
transposed operand in the oracle fails it.
"""

import math

import pytest
import torch
from torch.nn import functional as F

import oracle

D = torch.float64
TOL = dict(rtol=1e-9, atol=1e-10)


def rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return scale * torch.randn(*shape, generator=g, dtype=D)


# ------------------------------------------------------------------ Linear
@pytest.mark.parametrize('act', [None, 'relu', 'geluapprox', 'leaky_relu_0.01', 'mish'])
@pytest.mark.parametrize('bias', [False, True])
def test_linear_matches_torch_autograd(act, bias) -> None:
    x = rand(3, 5, 7, seed=1).requires_grad_(True)
    w = rand(7, 4, seed=2).requires_grad_(True)          # [in, out] layout
    b = rand(4, seed=3).requires_grad_(True) if bias else None
    dy = rand(3, 5, 4, seed=4)
    name, param = oracle.parse_act_func(act)
    z = F.linear(x, w.T, b)
    torch_act = {None: lambda t: t, 'relu': F.relu, 'geluapprox': lambda t: F.gelu(t, approximate='tanh'),
                 'leaky_relu': lambda t: F.leaky_relu(t, 0.01), 'mish': F.mish}[name]
    y = torch_act(z)
    grads = torch.autograd.grad(y, [x, w] + ([b] if bias else []), dy)
    out, pre_act = oracle.linear_forward(x.detach(), w.detach(), None if b is None else b.detach(),
                                         name, param, D, compute=D)
    torch.testing.assert_close(out, y.detach(), rtol=1e-7, atol=1e-7)
    if name is not None:
        torch.testing.assert_close(pre_act, z.detach().flatten(0, -2), **TOL)
    dx, dw, db = oracle.linear_backward(dy, x.detach(), w.detach(), pre_act, name, param, D, compute=D)
    torch.testing.assert_close(dx, grads[0], rtol=1e-7, atol=1e-7)
    torch.testing.assert_close(dw, grads[1], rtol=1e-7, atol=1e-7)   # [in, out], not transposed
    if bias:
        torch.testing.assert_close(db, grads[2], rtol=1e-7, atol=1e-7)


def test_linear_brute_force() -> None:
    x, w, b = rand(2, 3, seed=5), rand(3, 2, seed=6), rand(2, seed=7)
    out, _ = oracle.linear_forward(x, w, b, None, None, D, compute=D)
    for i in range(2):
        for j in range(2):
            acc = sum(x[i, k].item() * w[k, j].item() for k in range(3)) + b[j].item()
            assert math.isclose(out[i, j].item(), acc, rel_tol=1e-12)


def test_linear_pre_act_is_rounded_but_activation_uses_accumulator() -> None:
    x = rand(8, 16, seed=8).to(torch.bfloat16)
    w = rand(16, 8, seed=9).to(torch.bfloat16)
    out, pre_act = oracle.linear_forward(x, w, None, 'relu', None, torch.bfloat16)
    z = x.float() @ w.float()
    assert pre_act.dtype == torch.bfloat16
    torch.testing.assert_close(pre_act, z.to(torch.bfloat16), rtol=0, atol=0)
    torch.testing.assert_close(out, torch.relu(z).to(torch.bfloat16), rtol=0, atol=0)


# ------------------------------------------------------------------ LayerNorm / RMSNorm
@pytest.mark.parametrize('affine, bias', [(False, False), (True, False), (True, True)])
def test_layer_norm_matches_torch(affine, bias) -> None:
    x = rand(6, 10, seed=1).requires_grad_(True)
    w = (1 + rand(10, seed=2)).requires_grad_(True) if affine else None
    b = rand(10, seed=3).requires_grad_(True) if bias else None
    dy = rand(6, 10, seed=4)
    y = F.layer_norm(x, (10,), w, b, 1e-5)
    params = [p for p in (w, b) if p is not None]
    grads = torch.autograd.grad(y, [x] + params, dy)
    det = lambda t: None if t is None else t.detach()
    out, mean, inv_std = oracle.layer_norm_forward(det(x), det(w), det(b), 1e-5, D, compute=D)
    torch.testing.assert_close(out, y.detach(), **TOL)
    torch.testing.assert_close(mean, x.detach().mean(dim=1), **TOL)
    torch.testing.assert_close(inv_std, 1 / torch.sqrt(x.detach().var(dim=1, unbiased=False) + 1e-5), **TOL)
    dx, dw, db = oracle.layer_norm_backward(dy, det(x), mean, inv_std, det(w), D, compute=D)
    torch.testing.assert_close(dx, grads[0], **TOL)
    if affine:
        torch.testing.assert_close(dw, grads[1], **TOL)
    if bias:
        torch.testing.assert_close(db, grads[2], **TOL)


def test_layer_norm_invariants() -> None:
    x, dy = rand(5, 33, seed=1), rand(5, 33, seed=2)
    out, mean, inv_std = oracle.layer_norm_forward(x, None, None, 0.0, D, compute=D)
    torch.testing.assert_close(out.mean(dim=1), torch.zeros(5, dtype=D), atol=1e-12, rtol=0)
    torch.testing.assert_close((out * out).mean(dim=1), torch.ones(5, dtype=D), **TOL)
    dx, _, _ = oracle.layer_norm_backward(dy, x, mean, inv_std, None, D, compute=D)
    torch.testing.assert_close(dx.sum(dim=1), torch.zeros(5, dtype=D), atol=1e-10, rtol=0)


def test_layer_norm_bias_ignored_without_weight() -> None:
    x, b = rand(4, 8, seed=1), rand(8, seed=2)
    a, _, _ = oracle.layer_norm_forward(x, None, b, 1e-5, D, compute=D)
    c, _, _ = oracle.layer_norm_forward(x, None, None, 1e-5, D, compute=D)
    torch.testing.assert_close(a, c, rtol=0, atol=0)


@pytest.mark.parametrize('affine', [False, True])
def test_rms_norm_matches_torch(affine) -> None:
    x = rand(6, 10, seed=1).requires_grad_(True)
    w = (1 + rand(10, seed=2)).requires_grad_(True) if affine else None
    dy = rand(6, 10, seed=4)
    y = F.rms_norm(x, (10,), w, 1e-6)
    grads = torch.autograd.grad(y, [x] + ([w] if affine else []), dy)
    det = lambda t: None if t is None else t.detach()
    out, inv_rms = oracle.rms_norm_forward(det(x), det(w), 1e-6, compute=D)
    torch.testing.assert_close(out, y.detach(), **TOL)
    dx, dw = oracle.rms_norm_backward(dy, det(x), inv_rms, det(w), compute=D)
    torch.testing.assert_close(dx, grads[0], **TOL)
    if affine:
        torch.testing.assert_close(dw, grads[1], **TOL)


def test_rms_norm_default_eps_is_finfo_eps() -> None:
    x = rand(3, 8, seed=1).to(torch.float16)
    a, _ = oracle.rms_norm_forward(x, None, None)
    b, _ = oracle.rms_norm_forward(x, None, torch.finfo(torch.float16).eps)
    torch.testing.assert_close(a, b, rtol=0, atol=0)
    torch.testing.assert_close(a, F.rms_norm(x.float(), (8,), None, torch.finfo(torch.float16).eps).half(),
                               rtol=1e-3, atol=1e-3)


# ------------------------------------------------------------------ Softmax family
@pytest.mark.parametrize('neg, log, fn', [(False, False, F.softmax), (False, True, F.log_softmax),
                                          (True, False, F.softmin)])
def test_softmax_family_matches_torch(neg, log, fn) -> None:
    x = rand(4, 9, seed=1, scale=3.0).requires_grad_(True)
    dy = rand(4, 9, seed=2)
    y = fn(x, dim=-1)
    (gx,) = torch.autograd.grad(y, x, dy)
    out = oracle.softmax_forward(x.detach(), neg, log, D, compute=D)
    torch.testing.assert_close(out, y.detach(), **TOL)
    torch.testing.assert_close(oracle.softmax_backward(dy, out, neg, log, compute=D), gx, **TOL)


def test_softmax_invariants() -> None:
    x, dy = rand(4, 9, seed=1), rand(4, 9, seed=2)
    y = oracle.softmax_forward(x, False, False, D, compute=D)
    torch.testing.assert_close(y.sum(dim=1), torch.ones(4, dtype=D), **TOL)
    torch.testing.assert_close(oracle.softmax_forward(x + 123.0, False, False, D, compute=D), y, **TOL)
    dx = oracle.softmax_backward(dy, y, False, False, compute=D)
    torch.testing.assert_close(dx.sum(dim=1), torch.zeros(4, dtype=D), atol=1e-12, rtol=0)


# ------------------------------------------------------------------ Cross entropy
@pytest.mark.parametrize('weighted', [False, True])
@pytest.mark.parametrize('ignore', [False, True])
def test_cross_entropy_matches_torch(weighted, ignore) -> None:
    x = rand(12, 7, seed=1, scale=2.0).requires_grad_(True)
    g = torch.Generator().manual_seed(3)
    t = torch.randint(0, 7, (12,), generator=g)
    if ignore:
        t[[1, 5, 6]] = -100
    w = (0.5 + torch.rand(7, generator=g, dtype=D)) if weighted else None
    loss = F.cross_entropy(x, t, weight=w, ignore_index=-100, reduction='mean')
    (gx,) = torch.autograd.grad(loss, x, torch.tensor(1.7, dtype=D))
    out, denom = oracle.cross_entropy_forward(x.detach(), t, w, -100, D, compute=D)
    torch.testing.assert_close(out, loss.detach(), **TOL)
    grad = oracle.cross_entropy_backward(torch.tensor(1.7, dtype=D), x.detach(), t, w, -100, D, compute=D)
    torch.testing.assert_close(grad, gx, **TOL)
    if ignore:
        assert torch.all(grad[[1, 5, 6]] == 0)
    if not weighted:
        assert denom.item() == (9 if ignore else 12)


def test_cross_entropy_special_cases() -> None:
    t = torch.tensor([0, 3, 2, 1])
    out, _ = oracle.cross_entropy_forward(torch.zeros(4, 5, dtype=D), t, None, -100, D, compute=D)
    assert math.isclose(out.item(), math.log(5), rel_tol=1e-12)      # uniform logits -> log V
    out, _ = oracle.cross_entropy_forward(torch.zeros(4, 5, dtype=D), torch.full((4,), -100), None, -100, D,
                                          compute=D)
    assert math.isnan(out.item())                                     # all ignored -> 0/0, as torch
    x = rand(4, 5, seed=1)
    grad = oracle.cross_entropy_backward(torch.tensor(1.0, dtype=D), x, t, None, -100, D, compute=D)
    sm = torch.softmax(x, dim=1)
    assert math.isclose(grad[1, 3].item(), (sm[1, 3].item() - 1) / 4, rel_tol=1e-12)
    torch.testing.assert_close(grad.sum(dim=1), torch.zeros(4, dtype=D), atol=1e-14, rtol=0)


# ------------------------------------------------------------------ NLL loss
@pytest.mark.parametrize('weighted', [False, True])
@pytest.mark.parametrize('reduction', ['none', 'mean', 'sum'])
@pytest.mark.parametrize('shape', [(12, 7), (5, 6, 9), (3, 4, 2, 5)])
def test_nll_loss_matches_torch(shape, reduction, weighted) -> None:
    feat = shape[1]
    x = torch.log_softmax(rand(*shape, seed=1, scale=2.0), dim=1).requires_grad_(True)
    g = torch.Generator().manual_seed(3)
    t = torch.randint(0, feat, (shape[0], *shape[2:]), generator=g)
    w = (0.5 + torch.rand(feat, generator=g, dtype=D)) if weighted else None
    loss = F.nll_loss(x, t, weight=w, reduction=reduction)
    dy = rand(*loss.shape, seed=4) if reduction == 'none' else torch.tensor(1.7, dtype=D)
    (gx,) = torch.autograd.grad(loss, x, dy)
    out, sum_weights = oracle.nll_loss_forward(x.detach(), t, w, reduction, D, compute=D)
    torch.testing.assert_close(out, loss.detach(), **TOL)
    grad = oracle.nll_loss_backward(dy, x.shape, t, w, reduction, D, compute=D)
    torch.testing.assert_close(grad, gx, **TOL)
    if weighted:
        torch.testing.assert_close(sum_weights, w[t].sum(), **TOL)


def test_nll_loss_brute_force() -> None:
    x = rand(3, 4, 2, seed=5)
    t = torch.tensor([[0, 3], [2, 2], [1, 0]])
    w = torch.tensor([0.5, 2.0, 1.5, 0.25], dtype=D)
    total, weights = 0.0, 0.0
    expected_grad = torch.zeros_like(x)
    for b in range(3):
        for s in range(2):
            c = int(t[b, s])
            total += -float(x[b, c, s]) * float(w[c])
            weights += float(w[c])
    for b in range(3):
        for s in range(2):
            c = int(t[b, s])
            expected_grad[b, c, s] = -2.0 * float(w[c]) / weights
    out, sum_weights = oracle.nll_loss_forward(x, t, w, 'mean', D, compute=D)
    assert math.isclose(out.item(), total / weights, rel_tol=1e-12)
    assert math.isclose(sum_weights.item(), weights, rel_tol=1e-12)
    grad = oracle.nll_loss_backward(torch.tensor(2.0, dtype=D), x.shape, t, w, 'mean', D, compute=D)
    torch.testing.assert_close(grad, expected_grad, **TOL)
    # unweighted mean divides by the number of entries, and log-softmax + NLL is cross entropy
    out, _ = oracle.nll_loss_forward(x, t, None, 'mean', D, compute=D)
    assert math.isclose(out.item(), -sum(float(x[b, int(t[b, s]), s]) for b in range(3) for s in range(2)) / 6,
                        rel_tol=1e-12)
    logits = rand(6, 5, seed=6)
    cls = torch.tensor([0, 4, 2, 2, 1, 3])
    via_nll, _ = oracle.nll_loss_forward(torch.log_softmax(logits, dim=1), cls, None, 'mean', D, compute=D)
    via_ce, _ = oracle.cross_entropy_forward(logits, cls, None, -100, D, compute=D)
    torch.testing.assert_close(via_nll, via_ce, **TOL)


# ------------------------------------------------------------------ GLU and p-norm losses
@pytest.mark.parametrize('dim', [-1, 0, 1])
def test_glu_matches_torch(dim) -> None:
    x = rand(4, 6, 8, seed=1).requires_grad_(True)
    y = F.glu(x, dim=dim)                                     # torch's GLU is the sigmoid case
    dy = rand(*y.shape, seed=2)
    (gx,) = torch.autograd.grad(y, x, dy)
    torch.testing.assert_close(oracle.glu_forward(x.detach(), dim, 'sigmoid', None, D, compute=D), y.detach(), **TOL)
    torch.testing.assert_close(oracle.glu_backward(dy, x.detach(), dim, 'sigmoid', None, D, compute=D), gx, **TOL)
    # another activation through autograd on the composed expression
    a, b = x.chunk(2, dim=dim)
    y2 = a * F.silu(b)
    (gx2,) = torch.autograd.grad(y2, x, dy)
    torch.testing.assert_close(oracle.glu_forward(x.detach(), dim, 'silu', None, D, compute=D), y2.detach(), **TOL)
    torch.testing.assert_close(oracle.glu_backward(dy, x.detach(), dim, 'silu', None, D, compute=D), gx2, **TOL)


@pytest.mark.parametrize('reduction', ['none', 'mean', 'sum'])
@pytest.mark.parametrize('p_loss, torch_fn, param', [
    (0, lambda x, t, r: F.smooth_l1_loss(x, t, reduction=r, beta=0.7), 0.7),
    (1, lambda x, t, r: F.l1_loss(x, t, reduction=r), 1.0),
    (2, lambda x, t, r: F.mse_loss(x, t, reduction=r), 1.0),
    (3, lambda x, t, r: F.huber_loss(x, t, reduction=r, delta=0.6), 0.6)])
def test_p_loss_matches_torch(p_loss, torch_fn, param, reduction) -> None:
    x = rand(5, 7, 3, seed=1).requires_grad_(True)
    t = rand(5, 7, 3, seed=2).requires_grad_(True)
    loss = torch_fn(x, t, reduction)
    dy = rand(*loss.shape, seed=3) if reduction == 'none' else torch.tensor(-1.3, dtype=D)
    gx, gt = torch.autograd.grad(loss, [x, t], dy)
    out = oracle.p_loss_forward(x.detach(), t.detach(), p_loss, reduction, param, D, compute=D)
    torch.testing.assert_close(out, loss.detach(), **TOL)
    dx, dt = oracle.p_loss_backward(dy, x.detach(), t.detach(), p_loss, reduction, param, D, compute=D)
    torch.testing.assert_close(dx, gx, **TOL)
    torch.testing.assert_close(dt, gt, **TOL)


def test_p_loss_known_answers() -> None:
    x = torch.tensor([0.0, 0.25, -2.0, 3.0], dtype=D)
    t = torch.zeros(4, dtype=D)
    one = torch.tensor(1.0, dtype=D)
    assert oracle.p_loss_forward(x, t, 1, 'sum', 1.0, D, compute=D).item() == 5.25
    assert oracle.p_loss_forward(x, t, 2, 'mean', 1.0, D, compute=D).item() == (0.0625 + 4 + 9) / 4
    # smooth L1, beta 0.5: 0, 0.0625, 1.75, 2.75;  Huber, delta 0.5: 0, 0.03125, 0.875, 1.375
    torch.testing.assert_close(oracle.p_loss_forward(x, t, 0, 'none', 0.5, D, compute=D),
                               torch.tensor([0.0, 0.0625, 1.75, 2.75], dtype=D), **TOL)
    torch.testing.assert_close(oracle.p_loss_forward(x, t, 3, 'none', 0.5, D, compute=D),
                               torch.tensor([0.0, 0.03125, 0.875, 1.375], dtype=D), **TOL)
    # the L1 slope at a zero difference is +1 (p_loss_kernels.py:130), not torch's 0
    dx, dt = oracle.p_loss_backward(one, x, t, 1, 'sum', 1.0, D, compute=D)
    assert dx.tolist() == [1.0, 1.0, -1.0, 1.0] and dt.tolist() == [-1.0, -1.0, 1.0, -1.0]


# ------------------------------------------------------------------ Conv2d
@pytest.mark.parametrize('kernel, stride, padding, groups',
                         [((3, 3), (1, 1), (1, 1), 1), ((1, 1), (1, 1), (0, 0), 1),
                          ((5, 3), (2, 1), (3, 0), 2), ((2, 4), (1, 2), (1, 3), 4),
                          ((7, 7), (2, 2), (3, 3), 1)])
@pytest.mark.parametrize('bias', [False, True])
def test_conv2d_matches_torch(kernel, stride, padding, groups, bias) -> None:
    x = rand(2, 8, 11, 9, seed=1).requires_grad_(True)
    w = rand(12, 8 // groups, *kernel, seed=2).requires_grad_(True)
    b = rand(12, seed=3).requires_grad_(True) if bias else None
    y = F.conv2d(x, w, b, stride, padding, 1, groups)
    dy = rand(*y.shape, seed=4)
    grads = torch.autograd.grad(y, [x, w] + ([b] if bias else []), dy)
    det = lambda t: None if t is None else t.detach()
    out = oracle.conv2d_forward(det(x), det(w), det(b), stride, padding, groups, D, compute=D)
    torch.testing.assert_close(out, y.detach(), **TOL)
    dx, dw, db = oracle.conv2d_backward(dy, det(x), det(w), stride, padding, groups, D, compute=D)
    torch.testing.assert_close(dx, grads[0], **TOL)
    torch.testing.assert_close(dw, grads[1], **TOL)
    torch.testing.assert_close(dx, torch.nn.grad.conv2d_input(x.shape, det(w), dy, stride, padding, 1, groups), **TOL)
    torch.testing.assert_close(dw, torch.nn.grad.conv2d_weight(det(x), w.shape, dy, stride, padding, 1, groups), **TOL)
    if bias:
        torch.testing.assert_close(db, grads[2], **TOL)


def test_conv2d_brute_force() -> None:
    x, w = rand(1, 2, 4, 4, seed=1), rand(3, 2, 3, 3, seed=2)
    out = oracle.conv2d_forward(x, w, None, (1, 1), (1, 1), 1, D, compute=D)
    for o in range(3):
        for i in range(4):
            for j in range(4):
                acc = 0.0
                for c in range(2):
                    for h in range(3):
                        for v in range(3):
                            a, bb = i + h - 1, j + v - 1
                            if 0 <= a < 4 and 0 <= bb < 4:
                                acc += x[0, c, a, bb].item() * w[o, c, h, v].item()
                assert math.isclose(out[0, o, i, j].item(), acc, rel_tol=1e-10, abs_tol=1e-12)


# ------------------------------------------------------------------ BatchNorm
@pytest.mark.parametrize('shape', [(6, 5), (4, 5, 7), (3, 5, 4, 6)])
@pytest.mark.parametrize('affine', [False, True])
@pytest.mark.parametrize('residual', [False, True])
@pytest.mark.parametrize('act', [None, 'relu', 'silu'])
def test_batch_norm_training_matches_torch(shape, affine, residual, act) -> None:
    x = rand(*shape, seed=1).requires_grad_(True)
    w = rand(5, seed=2).requires_grad_(True) if affine else None
    b = rand(5, seed=3).requires_grad_(True) if affine else None
    res = rand(*shape, seed=4).requires_grad_(True) if residual else None
    dy = rand(*shape, seed=5)
    rm, rv = rand(5, seed=6), rand(5, seed=7).abs() + 0.5
    t_rm, t_rv = rm.clone(), rv.clone()
    y = F.batch_norm(x, t_rm, t_rv, w, b, True, 0.2, 1e-5)
    if residual:
        y = y + res
    z = y
    y = {None: lambda t: t, 'relu': F.relu, 'silu': F.silu}[act](y)
    wanted = [x] + ([w, b] if affine else []) + ([res] if residual else [])
    grads = list(torch.autograd.grad(y, wanted, dy))
    det = lambda t: None if t is None else t.detach()
    out, pre_act, mean, inv_std, new_rm, new_rv = oracle.batch_norm_forward(
        det(x), True, det(w), det(b), rm, rv, 0.2, 1e-5, True, det(res), act, None, compute=D)
    torch.testing.assert_close(out, y.detach(), **TOL)
    torch.testing.assert_close(new_rm, t_rm, **TOL)
    torch.testing.assert_close(new_rv, t_rv, **TOL)       # unbiased variance in the running stat
    if act is not None:
        torch.testing.assert_close(pre_act, z.detach(), **TOL)
    dx, dw, db, dres = oracle.batch_norm_backward(dy, det(x), mean, inv_std, det(w), affine, pre_act, act,
                                                  None, compute=D)
    torch.testing.assert_close(dx, grads.pop(0), **TOL)
    if affine:
        torch.testing.assert_close(dw, grads.pop(0), **TOL)
        torch.testing.assert_close(db, grads.pop(0), **TOL)
    if residual:
        torch.testing.assert_close(dres, grads.pop(0), **TOL)


def test_batch_norm_eval_uses_running_stats() -> None:
    x, rm, rv = rand(4, 5, 3, seed=1), rand(5, seed=2), rand(5, seed=3).abs() + 0.5
    w, b = rand(5, seed=4), rand(5, seed=5)
    out, _, _, _, new_rm, new_rv = oracle.batch_norm_forward(x, False, w, b, rm, rv, 0.1, 1e-5, True, None,
                                                             None, None, compute=D)
    torch.testing.assert_close(out, F.batch_norm(x, rm, rv, w, b, False, 0.1, 1e-5), **TOL)
    assert new_rm is rm and new_rv is rv
    # without tracked running statistics the batch statistics are used even in eval mode
    out2, _, _, _, _, _ = oracle.batch_norm_forward(x, False, w, b, None, None, 0.1, 1e-5, False, None, None,
                                                    None, compute=D)
    torch.testing.assert_close(out2, F.batch_norm(x, None, None, w, b, True, 0.1, 1e-5), **TOL)


# ---------------------------------------------------------------------------------------------
# activation layers with fused dropout
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize('act_func, param, torch_fn', [
    ('relu', None, F.relu), ('geluapprox', None, lambda x: F.gelu(x, approximate='tanh')),
    ('leaky_relu', 0.2, lambda x: F.leaky_relu(x, 0.2)), (None, None, lambda x: x)])
@pytest.mark.parametrize('drop_p', [0.0, 0.3])
def test_act_dropout_matches_torch_with_the_same_mask(act_func, param, torch_fn, drop_p) -> None:
    # Independent statement: torch's activation + autograd, the mask applied as a constant
    # multiplier mask / (1 - p) (what F.dropout does with its own mask).
    torch.manual_seed(0)
    x = torch.randn(64, 33, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(64, 33, dtype=torch.float64)
    dropped = (torch.rand(64, 33) < drop_p) if drop_p > 0 else None
    scale = torch.ones_like(x) if dropped is None else (~dropped).double() / (1 - drop_p)
    expected = torch_fn(x) * scale
    (expected_grad,) = torch.autograd.grad(expected, x, dy)
    got = oracle.act_dropout_forward(x.detach(), act_func, param, dropped, drop_p, compute=torch.float64)
    got_grad = oracle.act_dropout_backward(dy, x.detach(), act_func, param, dropped, drop_p,
                                           compute=torch.float64)
    torch.testing.assert_close(got, expected.detach(), rtol=1e-7, atol=1e-7)
    torch.testing.assert_close(got_grad, expected_grad, rtol=1e-7, atol=1e-7)
    if dropped is not None:
        assert torch.count_nonzero(got[dropped]) == 0 and torch.count_nonzero(got_grad[dropped]) == 0
