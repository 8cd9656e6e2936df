"""
Shared helpers of the parity tests: seeded inputs, tolerances and comparison.

Tolerances are the ones the build targets: rtol 1e-4 / atol 1e-5 for float32 and
rtol 2e-2 / atol 2e-2 for float16 / bfloat16 outputs and gradients, applied element by
element.  Only gradients that are sums over the batch (weight and bias gradients, whose
magnitude and cancellation error grow with the number of summed rows) are compared after
dividing both sides by max(1, max|expected|): batch_reduction=True.
"""

from typing import Optional, Sequence, Tuple

import torch
from torch import Tensor

TOLERANCES = {torch.float32: (1e-4, 1e-5), torch.float16: (2e-2, 2e-2), torch.bfloat16: (2e-2, 2e-2)}
DTYPES = (torch.float32, torch.float16, torch.bfloat16)
ACT_FUNCS = (None, 'sigmoid', 'logsigmoid', 'tanh', 'relu', 'gelu', 'geluapprox', 'silu', 'relu6',
             'hardsigmoid', 'hardtanh', 'hardswish', 'selu', 'mish', 'softplus', 'softsign',
             'tanhshrink', 'leaky_relu_0.01', 'elu_1', 'celu_1', 'hardshrink_0.5', 'softshrink_0.5')


def compute_dtype(dtype: torch.dtype) -> torch.dtype:
    """
    Precision the oracle computes in for a storage dtype (float64 pins float32 kernels).
    """
    return torch.float64 if dtype is torch.float32 else torch.float32


def randn(shape: Sequence[int], seed: int, dtype: torch.dtype = torch.float32,
          scale: float = 1.0, shift: float = 0.0) -> Tensor:
    """
    Seeded CPU normal tensor, generated in float32 and rounded to dtype.
    """
    gen = torch.Generator().manual_seed(seed)
    return (shift + scale * torch.randn(tuple(shape), generator=gen)).to(dtype)


def assert_close(actual: Optional[Tensor], expected: Optional[Tensor], dtype: torch.dtype,
                 what: str, batch_reduction: bool = False, atol_scale: float = 1.0,
                 reference_tolerance: bool = False, dot_terms: int = 0, term_scale: float = 1.0) -> None:
    """
    Compares a device result with the CPU oracle at the tolerance of `dtype`, element by element.
    batch_reduction=True is for gradients summed over the batch: both sides are divided by
    max(1, max|expected|) first, so the absolute tolerance scales with the sum's magnitude.
    reference_tolerance=True widens the float32 tolerance to the rtol = atol = 1e-3 of the
    reference's own tests, for ill-conditioned cases only (see the callers).
    dot_terms / term_scale describe a float32 dot product of dot_terms products of typical
    magnitude term_scale: accumulating it in float32 rounds every partial sum, so an output that
    cancels to near zero still carries an error of about 2^-23 * dot_terms * term_scale, which
    then replaces a smaller absolute tolerance.
    """
    if expected is None:
        assert actual is None, f'{what}: expected None'
        return
    assert actual is not None, f'{what}: got None'
    rtol, atol = TOLERANCES[dtype]
    if reference_tolerance and dtype is torch.float32:
        rtol, atol = 1e-3, 1e-3
    if dtype is torch.float32:
        atol = max(atol, 2.0 ** -23 * dot_terms * term_scale)
    assert actual.shape == expected.shape, f'{what}: shape {tuple(actual.shape)} != {tuple(expected.shape)}'
    if actual.numel() >= 1 << 22 and not batch_reduction and dtype is not torch.float32:
        # large 16-bit tensors: the same element-wise criterion in float32 (exact for 16-bit
        # values) without the float64 copies; the slow path below words the failure
        where = actual.device if actual.is_cuda else expected.device   # on the GPU when either side is there
        a32, e32 = actual.detach().to(where).float(), expected.detach().to(where).float()
        if bool(torch.isclose(a32, e32, rtol=rtol, atol=atol * atol_scale, equal_nan=True).all()):
            return
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    if batch_reduction:
        scale = max(1.0, e.abs().max().item()) if e.numel() else 1.0
        a, e = a / scale, e / scale
    torch.testing.assert_close(a, e, rtol=rtol, atol=atol * atol_scale, equal_nan=True,
                               msg=lambda m: f'{what}: {m}')


def grads(*tensors: Optional[Tensor]) -> Tuple[Optional[Tensor], ...]:
    return tuple(None if t is None else t.grad for t in tensors)
