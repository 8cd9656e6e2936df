"""
Writes tests/golden/hot_path_small.npz: small input / expected-output vectors for every
hot-path layer, computed with torch.nn.functional + autograd in float64 on the CPU (the
implementation the reference's own tests compare against; the reference holds no stored
vectors).  Neither the oracle nor the HIP library is involved, so the file pins both.

    python tests/golden/make_golden.py
"""

from pathlib import Path

import numpy as np
import torch
from torch.nn import functional as F

OUT = Path(__file__).resolve().parent / 'hot_path_small.npz'
D = torch.float64


def rnd(gen, *shape, scale=1.0, shift=0.0):
    return (shift + scale * torch.randn(*shape, generator=gen)).to(D)


def main() -> None:
    gen = torch.Generator().manual_seed(20240607)
    out = {}

    def put(prefix, **tensors):
        for key, value in tensors.items():
            if value is not None:
                out[f'{prefix}.{key}'] = value.detach().numpy().astype(np.float64 if value.dtype.is_floating_point else np.int64)

    # Linear + geluapprox (weight kept in torch's [out, in] layout here; tests transpose)
    x, w, b, dy = rnd(gen, 24, 40).requires_grad_(), rnd(gen, 56, 40, scale=0.2).requires_grad_(), \
        rnd(gen, 56, scale=0.1).requires_grad_(), rnd(gen, 24, 56)
    y = F.gelu(F.linear(x, w, b), approximate='tanh')
    gx, gw, gb = torch.autograd.grad(y, [x, w, b], dy)
    put('linear', x=x, w=w, b=b, dy=dy, y=y, dx=gx, dw=gw, db=gb)

    # LayerNorm / RMSNorm
    x, w, b, dy = rnd(gen, 10, 96).requires_grad_(), rnd(gen, 96, scale=0.1, shift=1.0).requires_grad_(), \
        rnd(gen, 96, scale=0.1).requires_grad_(), rnd(gen, 10, 96)
    y = F.layer_norm(x, (96,), w, b, 1e-5)
    gx, gw, gb = torch.autograd.grad(y, [x, w, b], dy)
    put('layer_norm', x=x, w=w, b=b, dy=dy, y=y, dx=gx, dw=gw, db=gb)
    y = F.rms_norm(x, (96,), w, 1e-6)
    gx, gw = torch.autograd.grad(y, [x, w], dy)
    put('rms_norm', y=y, dx=gx, dw=gw)

    # Softmax family
    x, dy = rnd(gen, 6, 50, scale=2.0).requires_grad_(), rnd(gen, 6, 50)
    for name, fn in (('softmax', F.softmax), ('log_softmax', F.log_softmax), ('softmin', F.softmin)):
        y = fn(x, dim=-1)
        (gx,) = torch.autograd.grad(y, x, dy)
        put(name, y=y, dx=gx)
    put('softmax', x=x, dy=dy)

    # Cross entropy with class weights and ignored rows
    x = rnd(gen, 16, 37, scale=2.0).requires_grad_()
    t = torch.randint(0, 37, (16,), generator=gen)
    t[[2, 9, 10]] = -100
    w = (0.5 + torch.rand(37, generator=gen)).to(D)
    loss = F.cross_entropy(x, t, weight=w, ignore_index=-100)
    (gx,) = torch.autograd.grad(loss, x)
    put('cross_entropy', x=x, target=t, w=w, loss=loss, dx=gx)

    # Conv2d 3x3 stride 2 groups 2 with bias
    x, w, b = rnd(gen, 2, 8, 9, 7).requires_grad_(), rnd(gen, 6, 4, 3, 3, scale=0.2).requires_grad_(), \
        rnd(gen, 6).requires_grad_()
    y = F.conv2d(x, w, b, (2, 1), (1, 1), 1, 2)
    dy = rnd(gen, *y.shape)
    gx, gw, gb = torch.autograd.grad(y, [x, w, b], dy)
    put('conv2d', x=x, w=w, b=b, dy=dy, y=y, dx=gx, dw=gw, db=gb)

    # BatchNorm2d training + residual + relu
    x, w, b, res = rnd(gen, 4, 5, 6, 3).requires_grad_(), rnd(gen, 5).requires_grad_(), \
        rnd(gen, 5).requires_grad_(), rnd(gen, 4, 5, 6, 3).requires_grad_()
    rm, rv = rnd(gen, 5), rnd(gen, 5).abs() + 0.5
    put('batch_norm', rm0=rm, rv0=rv)
    y = F.relu(F.batch_norm(x, rm, rv, w, b, True, 0.1, 1e-5) + res)
    dy = rnd(gen, *y.shape)
    gx, gw, gb, gr = torch.autograd.grad(y, [x, w, b, res], dy)
    put('batch_norm', x=x, w=w, b=b, res=res, dy=dy, y=y, dx=gx, dw=gw, db=gb, dres=gr, rm1=rm, rv1=rv)

    np.savez_compressed(OUT, **out)
    print(f'wrote {OUT} ({OUT.stat().st_size} bytes, {len(out)} arrays)')


if __name__ == '__main__':
    main()
