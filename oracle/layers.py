"""
Oracle (test infrastructure): CPU restatements of the reference's layer kernels and of the
host arithmetic of its autograd Functions.  Everything is computed in `compute` precision
(float32 by default, float64 for tight pins) from the stored-dtype inputs, and rounded to the
storage dtype at the same points as the reference.
"""

from typing import Optional, Tuple

import torch
from torch import Tensor

from .acts import act_forward, act_grad


def _c(t: Optional[Tensor], compute: torch.dtype) -> Optional[Tensor]:
    return None if t is None else t.to(compute)


# ---------------------------------------------------------------------------------------------
# Linear — attorch/linear_kernels.py:59-188, attorch/linear_layer.py:24-161
# ---------------------------------------------------------------------------------------------
def linear_forward(
    input: Tensor, weight: Tensor, bias: Optional[Tensor], act_func: Optional[str],
    param: Optional[float], output_dtype: torch.dtype, compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Optional[Tensor]]:
    """
    output = act(input @ weight + bias) with weight stored [in, out]
    (linear_kernels.py:143-165 accumulate, :167-174 bias, :176-183 pre-activation store and
    activation on the unrounded accumulator, :185-188 store).  Operands are first rounded
    to the output dtype when that is a 16-bit type (:161-163, :171-172).

    Returns:
        (output [.., out] in output_dtype, pre_act in output_dtype or None without act).
    """
    x = input.flatten(0, -2)
    if output_dtype in (torch.float16, torch.bfloat16):
        x, weight = x.to(output_dtype), weight.to(output_dtype)
        bias = None if bias is None else bias.to(output_dtype)
    accum = _c(x, compute) @ _c(weight, compute)
    if bias is not None:
        accum = accum + _c(bias, compute)
    pre_act = None
    if act_func is not None:
        pre_act = accum.to(output_dtype)
        accum = act_forward(accum, act_func, param)
    output = accum.to(output_dtype).view(*input.shape[:-1], weight.shape[1])
    return output, pre_act


def linear_backward(
    output_grad: Tensor, input: Tensor, weight: Tensor, pre_act: Optional[Tensor],
    act_func: Optional[str], param: Optional[float], output_dtype: torch.dtype,
    compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Tensor, Tensor]:
    """
    linear_layer.py:133-156: pre_act_grad = output_grad * act'(pre_act) stored in pre_act's
    dtype (:138, act_kernels.py:919-927); input_grad = pre_act_grad @ weight.T;
    weight_grad = input.T @ pre_act_grad (layout [in, out]); bias_grad = column sum of
    pre_act_grad.  The two products run under autocast to the output dtype (:152).

    Returns:
        (input_grad, weight_grad, bias_grad).
    """
    dy = output_grad.flatten(0, -2)
    x = input.flatten(0, -2)
    if act_func is None:
        dz = dy
    else:
        dz = (_c(dy, compute) * act_grad(_c(pre_act, compute), act_func, param)).to(pre_act.dtype)
    low = output_dtype in (torch.float16, torch.bfloat16)
    dz_mm = dz.to(output_dtype) if low else dz
    x_mm = x.to(output_dtype) if low else x
    w_mm = weight.to(output_dtype) if low else weight
    input_grad = (_c(dz_mm, compute) @ _c(w_mm, compute).T).to(output_dtype).view_as(input)
    weight_grad = (_c(x_mm, compute).T @ _c(dz_mm, compute)).to(output_dtype)
    bias_grad = _c(dz, compute).sum(dim=0).to(dz.dtype)
    return input_grad, weight_grad, bias_grad


# ---------------------------------------------------------------------------------------------
# LayerNorm — attorch/layer_norm_kernels.py:21-101, :111-224
# ---------------------------------------------------------------------------------------------
def layer_norm_forward(
    input: Tensor, weight: Optional[Tensor], bias: Optional[Tensor], eps: float,
    output_dtype: torch.dtype, compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Tensor, Tensor]:
    """
    layer_norm_kernels.py:82-101: mean over features, diff, inv_std = rsqrt(mean(diff^2)+eps),
    output = diff*inv_std (*weight (+bias)); bias only with weight (layer_norm_layer.py:60).

    Returns:
        (output, mean [rows], inv_std [rows]); statistics in `compute` precision.
    """
    x = _c(input.reshape(-1, input.shape[-1]), compute)
    mean = x.sum(dim=1) / x.shape[1]
    diff = x - mean[:, None]
    inv_std = torch.rsqrt((diff * diff).sum(dim=1) / x.shape[1] + eps)
    out = diff * inv_std[:, None]
    if weight is not None:
        out = out * _c(weight, compute)
        if bias is not None:
            out = out + _c(bias, compute)
    return out.to(output_dtype).view(input.shape), mean, inv_std


def layer_norm_backward(
    output_grad: Tensor, input: Tensor, mean: Tensor, inv_std: Tensor, weight: Optional[Tensor],
    output_dtype: torch.dtype, compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Optional[Tensor], Optional[Tensor]]:
    """
    layer_norm_kernels.py:189-224 and the sums at layer_norm_layer.py:150-153.

    Returns:
        (input_grad in output_dtype, weight_grad, bias_grad) — parameter gradients in
        `compute` precision, None without weight.
    """
    dy = _c(output_grad.reshape(-1, input.shape[-1]), compute)
    x = _c(input.reshape(-1, input.shape[-1]), compute)
    feat = x.shape[1]
    pre_lin = (x - _c(mean, compute)[:, None]) * _c(inv_std, compute)[:, None]
    g = dy * _c(weight, compute) if weight is not None else dy
    term1 = pre_lin * ((pre_lin * g).sum(dim=1) / feat)[:, None]
    term2 = (g.sum(dim=1) / feat)[:, None]
    dx = _c(inv_std, compute)[:, None] * (g - (term1 + term2))
    dw = (dy * pre_lin).sum(dim=0) if weight is not None else None
    db = dy.sum(dim=0) if weight is not None else None
    return dx.to(output_dtype).view(input.shape), dw, db


# ---------------------------------------------------------------------------------------------
# RMSNorm — attorch/rms_norm_kernels.py:21-88, :98-193
# ---------------------------------------------------------------------------------------------
def rms_norm_forward(
    input: Tensor, weight: Optional[Tensor], eps: Optional[float],
    compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Tensor]:
    """
    rms_norm_kernels.py:73-88; eps=None selects torch.finfo(input.dtype).eps
    (rms_norm_layer.py:50); the output keeps the input dtype (:52).

    Returns:
        (output, inv_rms [rows]).
    """
    eps = torch.finfo(input.dtype).eps if eps is None else eps
    x = _c(input.reshape(-1, input.shape[-1]), compute)
    inv_rms = torch.rsqrt((x * x).sum(dim=1) / x.shape[1] + eps)
    out = x * inv_rms[:, None]
    if weight is not None:
        out = out * _c(weight, compute)
    return out.to(input.dtype).view(input.shape), inv_rms


def rms_norm_backward(
    output_grad: Tensor, input: Tensor, inv_rms: Tensor, weight: Optional[Tensor],
    compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Optional[Tensor]]:
    """
    rms_norm_kernels.py:170-193 and the sum at rms_norm_layer.py:126-127.

    Returns:
        (input_grad in the input dtype, weight_grad or None).
    """
    dy = _c(output_grad.reshape(-1, input.shape[-1]), compute)
    x = _c(input.reshape(-1, input.shape[-1]), compute)
    feat = x.shape[1]
    r = _c(inv_rms, compute)[:, None]
    pre_lin = x * r
    g = dy * _c(weight, compute) if weight is not None else dy
    term1 = x * (x * g).sum(dim=1)[:, None]
    dx = r * (g - term1 * (r * r) / feat)
    dw = (dy * pre_lin).sum(dim=0) if weight is not None else None
    return dx.to(input.dtype).view(input.shape), dw


# ---------------------------------------------------------------------------------------------
# Softmax family — attorch/softmax_kernels.py:43-103, :113-181
# ---------------------------------------------------------------------------------------------
def softmax_forward(
    input: Tensor, neg: bool, log: bool, output_dtype: torch.dtype,
    compute: torch.dtype = torch.float32,
    ) -> Tensor:
    """
    softmax_kernels.py:88-103: optional negation, subtract the row max, exponentiate,
    normalise; the log variant returns (x - max) - log(sum).
    """
    x = _c(input.reshape(-1, input.shape[-1]), compute)
    if neg:
        x = -x
    x = x - x.max(dim=1).values[:, None]
    num = torch.exp(x)
    den = num.sum(dim=1)[:, None]
    out = x - torch.log(den) if log else num / den
    return out.to(output_dtype).view(input.shape)


def softmax_backward(
    output_grad: Tensor, output: Tensor, neg: bool, log: bool,
    compute: torch.dtype = torch.float32,
    ) -> Tensor:
    """
    softmax_kernels.py:166-181, from the SAVED (already rounded) output
    (softmax_layers.py:57-58): softmax dx = y*(dy - sum(dy*y)); log-softmax
    dx = dy - exp(y)*sum(dy); negated for softmin.  The result has the output's dtype.
    """
    dy = _c(output_grad.reshape(-1, output.shape[-1]), compute)
    y = _c(output.reshape(-1, output.shape[-1]), compute)
    if log:
        dx = dy - torch.exp(y) * dy.sum(dim=1)[:, None]
    else:
        dx = y * (dy - (dy * y).sum(dim=1)[:, None])
    if neg:
        dx = -dx
    return dx.to(output.dtype).view(output.shape)


# ---------------------------------------------------------------------------------------------
# Cross entropy — attorch/cross_entropy_loss_kernels.py:21-86, :96-172 (+ ignore_index)
# ---------------------------------------------------------------------------------------------
def cross_entropy_forward(
    input: Tensor, target: Tensor, weight: Optional[Tensor], ignore_index: int,
    output_dtype: torch.dtype, compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Tensor]:
    """
    cross_entropy_loss_kernels.py:69-86 per row: loss = log(sum(exp(x - max))) - x[target] + max,
    times weight[target] when weighted; cross_entropy_loss_layer.py:76-80: mean = sum / sum of
    the selected weights (or / rows when unweighted, kernel :84).  Extension not in the
    reference: rows whose target equals ignore_index are dropped from both sums, so the
    unweighted divisor is the number of kept rows.

    Returns:
        (loss scalar in output_dtype, divisor in `compute` precision).
    """
    x = _c(input, compute)
    keep = target != ignore_index
    safe_target = torch.where(keep, target, torch.zeros_like(target))
    mx = x.max(dim=1).values
    lse = torch.log(torch.exp(x - mx[:, None]).sum(dim=1))
    pred = x.gather(1, safe_target[:, None])[:, 0]
    loss = lse - pred + mx
    if weight is not None:
        w = _c(weight, compute)[safe_target] * keep
    else:
        w = keep.to(compute)
    denom = w.sum()
    total = (loss * w).sum() / denom
    return total.to(output_dtype), denom


def cross_entropy_backward(
    output_grad: Tensor, input: Tensor, target: Tensor, weight: Optional[Tensor],
    ignore_index: int, output_dtype: torch.dtype, compute: torch.dtype = torch.float32,
    ) -> Tensor:
    """
    cross_entropy_loss_kernels.py:149-172: input_grad = output_grad * (softmax - onehot) *
    weight[target] / sum_weights (or / rows); ignored rows get zero (extension).
    """
    x = _c(input, compute)
    keep = target != ignore_index
    safe_target = torch.where(keep, target, torch.zeros_like(target))
    x = x - x.max(dim=1).values[:, None]
    num = torch.exp(x)
    softmax = num / num.sum(dim=1)[:, None]
    onehot = torch.zeros_like(softmax)
    onehot.scatter_(1, safe_target[:, None], 1.0)
    if weight is not None:
        w = _c(weight, compute)[safe_target] * keep
    else:
        w = keep.to(compute)
    grad = _c(output_grad, compute) * (softmax - onehot) * (w / w.sum())[:, None]
    return grad.to(output_dtype)


# ---------------------------------------------------------------------------------------------
# Negative log likelihood — attorch/nll_loss_kernels.py:39-138, :141-235, nll_loss_layer.py:55-93
# ---------------------------------------------------------------------------------------------
def _nll_views(input: Tensor, target: Tensor) -> Tuple[Tensor, Tensor]:
    """nll_loss_layer.py:58-62: [batch, feat, spatial] and [batch, spatial] views."""
    flat_input = input.unsqueeze(-1) if input.ndim == 2 else input
    flat_target = target.unsqueeze(-1) if target.ndim == 1 else target
    return flat_input.flatten(2, -1), flat_target.flatten(1, -1)


def nll_loss_forward(
    input: Tensor, target: Tensor, weight: Optional[Tensor], reduction: str,
    output_dtype: torch.dtype, compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Optional[Tensor]]:
    """
    nll_loss_kernels.py:108-138: output[b, s] = -input[b, target[b, s], s], times
    weight[target[b, s]] when weighted; 'sum' adds all entries; 'mean' divides the sum by
    batch * spatial (kernel :132-134) or, weighted, by the sum of the selected weights
    (nll_loss_layer.py:88-93).

    Returns:
        (loss in output_dtype, sum of the selected weights in `compute` precision or None).
    """
    x, t = _nll_views(_c(input, compute), target)
    picked = x.gather(1, t[:, None, :])[:, 0, :]
    loss = -picked
    sum_weights = None
    if weight is not None:
        w = _c(weight, compute)[t]
        loss = loss * w
        sum_weights = w.sum()
    if reduction == 'none':
        return loss.view(target.shape).to(output_dtype), sum_weights
    total = loss.sum()
    if reduction == 'mean':
        total = total / sum_weights if weight is not None else total / t.numel()
    return total.to(output_dtype), sum_weights


def nll_loss_backward(
    output_grad: Tensor, input_shape: Tuple[int, ...], target: Tensor, weight: Optional[Tensor],
    reduction: str, output_dtype: torch.dtype, compute: torch.dtype = torch.float32,
    ) -> Tensor:
    """
    nll_loss_kernels.py:207-235 on a zeroed gradient (nll_loss_layer.py:120): at
    [b, target[b, s], s] the value -output_grad (per entry for 'none', the scalar otherwise),
    times weight[target] when weighted, divided for 'mean' by the summed selected weights
    (weighted) or by batch * spatial.
    """
    batch, feat = input_shape[:2]
    flat_target = (target.unsqueeze(-1) if target.ndim == 1 else target).flatten(1, -1)
    spatial = flat_target.shape[1]
    g = _c(output_grad, compute)
    coef = -g.reshape(batch, spatial) if reduction == 'none' else (-g).expand(batch, spatial)
    if weight is not None:
        w = _c(weight, compute)[flat_target]
        coef = coef * w
        if reduction == 'mean':
            coef = coef / w.sum()
    elif reduction == 'mean':
        coef = coef / (batch * spatial)
    grad = torch.zeros((batch, feat, spatial), dtype=compute)
    grad.scatter_(1, flat_target[:, None, :], coef[:, None, :])
    return grad.view(input_shape).to(output_dtype)


# ---------------------------------------------------------------------------------------------
# Conv2d — attorch/conv_kernels.py:68-207, attorch/conv_layer.py:43-164
# ---------------------------------------------------------------------------------------------
def _conv_out(size: int, kernel: int, stride: int, padding: int) -> int:
    return (size + 2 * padding - kernel) // stride + 1   # conv_layer.py:18-36


def conv2d_forward(
    input: Tensor, weight: Tensor, bias: Optional[Tensor], stride: Tuple[int, int],
    padding: Tuple[int, int], groups: int, output_dtype: torch.dtype,
    compute: torch.dtype = torch.float32,
    ) -> Tensor:
    """
    conv_kernels.py:162-196: for every kernel tap (h, w) the zero-padded, strided input
    window is contracted with weight[:, :, h, w] over the channels of the group and
    accumulated; bias is added afterwards (conv_layer.py:114-116).  NCHW.
    """
    n, c, ih, iw = input.shape
    co, cg, kh, kw = weight.shape
    sh, sw = stride
    ph, pw = padding
    oh, ow = _conv_out(ih, kh, sh, ph), _conv_out(iw, kw, sw, pw)
    low = output_dtype in (torch.float16, torch.bfloat16)
    x = _c(input.to(output_dtype) if low else input, compute)
    w = _c(weight.to(output_dtype) if low else weight, compute)
    xp = torch.zeros((n, c, ih + 2 * ph, iw + 2 * pw), dtype=compute)
    xp[:, :, ph:ph + ih, pw:pw + iw] = x
    out = torch.zeros((n, co, oh, ow), dtype=compute)
    og = co // groups
    for g in range(groups):
        for h in range(kh):
            for v in range(kw):
                win = xp[:, g * cg:(g + 1) * cg, h:h + sh * (oh - 1) + 1:sh, v:v + sw * (ow - 1) + 1:sw]
                out[:, g * og:(g + 1) * og] += torch.einsum('nchw,oc->nohw', win,
                                                            w[g * og:(g + 1) * og, :, h, v])
    out = out.to(output_dtype)
    if bias is not None:
        out += bias.view(1, -1, 1, 1).to(output_dtype)
    return out


def conv2d_backward(
    output_grad: Tensor, input: Tensor, weight: Tensor, stride: Tuple[int, int],
    padding: Tuple[int, int], groups: int, output_dtype: torch.dtype,
    compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Tensor, Tensor]:
    """
    conv_layer.py:147-162 (the reference calls torch.nn.grad.conv2d_input / conv2d_weight
    on operands cast to the output dtype): input_grad scatters output_grad through every tap,
    weight_grad correlates the padded input with output_grad, bias_grad sums output_grad
    over batch and space.

    Returns:
        (input_grad, weight_grad, bias_grad), all in output_dtype.
    """
    n, c, ih, iw = input.shape
    co, cg, kh, kw = weight.shape
    sh, sw = stride
    ph, pw = padding
    oh, ow = output_grad.shape[2:]
    x = _c(input.to(output_dtype), compute)
    w = _c(weight.to(output_dtype), compute)
    dy = _c(output_grad, compute)
    xp = torch.zeros((n, c, ih + 2 * ph, iw + 2 * pw), dtype=compute)
    xp[:, :, ph:ph + ih, pw:pw + iw] = x
    dxp = torch.zeros_like(xp)
    dw = torch.zeros((co, cg, kh, kw), dtype=compute)
    og = co // groups
    for g in range(groups):
        dyg = dy[:, g * og:(g + 1) * og]
        for h in range(kh):
            for v in range(kw):
                hs = slice(h, h + sh * (oh - 1) + 1, sh)
                ws = slice(v, v + sw * (ow - 1) + 1, sw)
                dxp[:, g * cg:(g + 1) * cg, hs, ws] += torch.einsum('nohw,oc->nchw', dyg,
                                                                     w[g * og:(g + 1) * og, :, h, v])
                dw[g * og:(g + 1) * og, :, h, v] = torch.einsum('nohw,nchw->oc', dyg,
                                                                xp[:, g * cg:(g + 1) * cg, hs, ws])
    dx = dxp[:, :, ph:ph + ih, pw:pw + iw]
    db = dy.sum(dim=(0, 2, 3))
    return dx.to(output_dtype), dw.to(output_dtype), db.to(output_dtype)


# ---------------------------------------------------------------------------------------------
# BatchNorm — attorch/batch_norm_kernels.py:44-236, :246-381; attorch/batch_norm_layer.py:43-245
# ---------------------------------------------------------------------------------------------
def batch_norm_forward(
    input: Tensor, training: bool, weight: Optional[Tensor], bias: Optional[Tensor],
    running_mean: Optional[Tensor], running_var: Optional[Tensor], momentum: float, eps: float,
    track_running_stats: bool, pre_act_add: Optional[Tensor], act_func: Optional[str],
    param: Optional[float], compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Optional[Tensor], Tensor, Tensor, Optional[Tensor], Optional[Tensor]]:
    """
    batch_norm_kernels.py:138-236 for an input [N, C, *]: batch statistics when training or
    when running statistics are not tracked (:138), biased variance for normalisation
    (:165-166), running statistics updated with the unbiased variance n/(n-1) (:172-183),
    otherwise the running statistics normalise (:185-187); then affine only when both weight
    and bias exist (batch_norm_layer.py:116), residual, pre-activation (input dtype) and
    activation.

    Returns:
        (output, pre_act or None, mean, inv_std, new_running_mean, new_running_var); the
        running statistics are returned, not updated in place.
    """
    x = _c(input.reshape(input.shape[0], input.shape[1], -1), compute)
    dims = (0, 2)
    n = x.shape[0] * x.shape[2]
    new_rm, new_rv = running_mean, running_var
    if training or not track_running_stats:
        mean = x.mean(dim=dims)
        var = ((x - mean[None, :, None]) ** 2).sum(dim=dims) / n
        inv_std = torch.rsqrt(var + eps)
        if track_running_stats:
            new_rm = ((1 - momentum) * _c(running_mean, compute) + momentum * mean).to(running_mean.dtype)
            new_rv = ((1 - momentum) * _c(running_var, compute) +
                      momentum * var * n / (n - 1)).to(running_var.dtype)
    else:
        mean = _c(running_mean, compute)
        inv_std = torch.rsqrt(_c(running_var, compute) + eps)
    affine = weight is not None and bias is not None
    w = _c(weight, compute) if affine else torch.ones(x.shape[1], dtype=compute)
    b = _c(bias, compute) if affine else torch.zeros(x.shape[1], dtype=compute)
    out = w[None, :, None] * (x - mean[None, :, None]) * inv_std[None, :, None] + b[None, :, None]
    if pre_act_add is not None:
        out = out + _c(pre_act_add.reshape(x.shape), compute)
    pre_act = None
    if act_func is not None:
        pre_act = out.to(input.dtype).view(input.shape)
        out = act_forward(out, act_func, param)
    return out.to(input.dtype).view(input.shape), pre_act, mean, inv_std, new_rm, new_rv


def batch_norm_backward(
    output_grad: Tensor, input: Tensor, mean: Tensor, inv_std: Tensor, weight: Optional[Tensor],
    affine: bool, pre_act: Optional[Tensor], act_func: Optional[str], param: Optional[float],
    compute: torch.dtype = torch.float32,
    ) -> Tuple[Tensor, Optional[Tensor], Optional[Tensor], Tensor]:
    """
    batch_norm_layer.py:191-245: pre_act_grad = output_grad * act'(pre_act) in pre_act's dtype
    (:196-208), then batch_norm_kernels.py:301-381: term1 = sum(x_hat*g), term2 = sum(g),
    input_grad = inv_std*(w*g - (term1*w/n*x_hat + term2*w/n)), weight_grad = term1,
    bias_grad = term2.  The residual gradient is pre_act_grad itself (:244).

    Returns:
        (input_grad, weight_grad, bias_grad, pre_act_grad).
    """
    shape3 = (input.shape[0], input.shape[1], -1)
    dy = _c(output_grad.reshape(shape3), compute)
    if act_func is not None:
        g_store = (dy * act_grad(_c(pre_act.reshape(shape3), compute), act_func, param)).to(pre_act.dtype)
    else:
        g_store = output_grad.reshape(shape3)
    g = _c(g_store, compute)
    x = _c(input.reshape(shape3), compute)
    n = x.shape[0] * x.shape[2]
    m = _c(mean, compute)[None, :, None]
    r = _c(inv_std, compute)[None, :, None]
    pre_lin = (x - m) * r
    term1 = (pre_lin * g).sum(dim=(0, 2))
    term2 = g.sum(dim=(0, 2))
    w = _c(weight, compute) if affine else torch.ones(x.shape[1], dtype=compute)
    t1 = (term1 * w / n)[None, :, None]
    t2 = (term2 * w / n)[None, :, None]
    dx = r * (w[None, :, None] * g - (t1 * pre_lin + t2))
    return (dx.to(input.dtype).view(input.shape), term1 if affine else None,
            term2 if affine else None, g_store.view(input.shape))


# ---------------------------------------------------------------------------------------------
# Activation layers with fused dropout, Dropout — attorch/act_kernels.py:631-927,
# attorch/dropout_kernels.py:13-112, attorch/act_layers.py:20-117, attorch/dropout_layer.py:19-96
# ---------------------------------------------------------------------------------------------
def act_dropout_forward(
    input: Tensor, act_func: Optional[str], param: Optional[float], dropped: Optional[Tensor],
    drop_p: float, compute: torch.dtype = torch.float32,
    ) -> Tensor:
    """
    output = dropout(act(input)) in the input's dtype: the activation is evaluated on the
    widened input (act_kernels.py:654-727), then elements of the mask `dropped` become 0 and
    the others are divided by 1 - drop_p (act_kernels.py:729-730, dropout_kernels.py:26-27).
    The random mask itself is implementation defined (the reference draws it with tl.rand), so
    it is an argument here: callers read it off the device result, as the reference's own
    tests do (tests/test_act_layers.py:49-51, tests/test_dropout_layer.py:30).
    `dropped` None means no dropout.
    """
    x = input.to(compute)
    out = x if act_func is None else act_forward(x, act_func, param)
    if dropped is not None:
        out = torch.where(dropped, torch.zeros((), dtype=compute), out / (1 - drop_p))
    return out.to(input.dtype)


def act_dropout_backward(
    output_grad: Tensor, input: Optional[Tensor], act_func: Optional[str], param: Optional[float],
    dropped: Optional[Tensor], drop_p: float, compute: torch.dtype = torch.float32,
    ) -> Tensor:
    """
    input_grad = dropout'(output_grad) * act'(input) (act_kernels.py:834-837): the upstream
    gradient goes through the same mask and scale (dropout_kernels.py:45-46) and is multiplied
    by the derivative of the activation at the forward input.
    """
    g = output_grad.to(compute)
    if dropped is not None:
        g = torch.where(dropped, torch.zeros((), dtype=compute), g / (1 - drop_p))
    if act_func is not None:
        g = g * act_grad(input.to(compute), act_func, param)
    dtype = output_grad.dtype if input is None else input.dtype
    return g.to(dtype)


# ---------------------------------------------------------------------------------------------
# Gated linear unit — attorch/glu_kernels.py:18-57, :60-105, attorch/glu_layer.py:60-62, :113
# ---------------------------------------------------------------------------------------------
def glu_forward(input: Tensor, dim: int, name: str, param: Optional[float], output_dtype: torch.dtype,
                compute: torch.dtype = torch.float32) -> Tensor:
    """
    glu_layer.py:60 and glu_kernels.py:53-56: the input is cut in two along `dim`;
    output = first half * act(second half).
    """
    x1, x2 = _c(input, compute).chunk(2, dim=dim)
    return (x1 * act_forward(x2, name, param)).to(output_dtype)


def glu_backward(output_grad: Tensor, input: Tensor, dim: int, name: str, param: Optional[float],
                 output_dtype: torch.dtype, compute: torch.dtype = torch.float32) -> Tensor:
    """
    glu_kernels.py:96-104: first-half gradient = output_grad * act(second half), second-half
    gradient = output_grad * first half * act'(second half); concatenated along `dim`
    (glu_layer.py:113).
    """
    x1, x2 = _c(input, compute).chunk(2, dim=dim)
    g = _c(output_grad, compute)
    grad1 = g * act_forward(x2, name, param)
    grad2 = g * x1 * act_grad(x2, name, param)
    return torch.concat([grad1, grad2], dim=dim).to(output_dtype)


# ---------------------------------------------------------------------------------------------
# p-norm losses — attorch/p_loss_kernels.py:17-79, :82-143, attorch/p_loss_layers.py:57-76
# ---------------------------------------------------------------------------------------------
def p_loss_forward(input: Tensor, target: Tensor, p_loss: int, reduction: str, param: float,
                   output_dtype: torch.dtype, compute: torch.dtype = torch.float32) -> Tensor:
    """
    p_loss_kernels.py:58-79 with diff = input - target: 0 smooth L1 (|d| < beta ? d^2 / (2 beta) :
    |d| - beta / 2), 1 L1 (|d|), 2 squared L2 (d^2), 3 Huber (|d| < delta ? d^2 / 2 :
    delta (|d| - delta / 2)); 'mean' divides the sum by the number of elements.
    """
    d = _c(input, compute) - _c(target, compute)
    a = d.abs()
    if p_loss == 0:
        error = torch.where(a < param, 0.5 * d * d / param, a - 0.5 * param)
    elif p_loss == 1:
        error = a
    elif p_loss == 2:
        error = d * d
    else:
        error = torch.where(a < param, 0.5 * d * d, param * (a - 0.5 * param))
    if reduction == 'none':
        return error.to(output_dtype)
    total = error.sum()
    if reduction == 'mean':
        total = total / error.numel()
    return total.to(output_dtype)


def p_loss_backward(output_grad: Tensor, input: Tensor, target: Tensor, p_loss: int, reduction: str,
                    param: float, output_dtype: torch.dtype,
                    compute: torch.dtype = torch.float32) -> Tuple[Tensor, Tensor]:
    """
    p_loss_kernels.py:126-143: slope of the loss in diff (sign taken as +1 at diff == 0, :128-136),
    divided by the number of elements for 'mean', times output_grad; the target's gradient is
    the negative.
    """
    d = _c(input, compute) - _c(target, compute)
    sign = torch.where(d >= 0, torch.ones_like(d), -torch.ones_like(d))
    if p_loss == 0:
        grad = torch.where(d.abs() < param, d / param, sign)
    elif p_loss == 1:
        grad = sign
    elif p_loss == 2:
        grad = 2 * d
    else:
        grad = torch.where(d.abs() < param, d, param * sign)
    if reduction == 'mean':
        grad = grad / d.numel()
    grad = grad * _c(output_grad, compute)
    return grad.to(output_dtype), (-grad).to(output_dtype)
