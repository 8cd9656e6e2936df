"""
Mixed-precision dtype policy shared by the layers.
"""

import functools
from typing import Optional

import torch

LOW_PRECISION = (torch.float16, torch.bfloat16)


def get_output_dtype(
    input_dtype: torch.dtype = torch.float32,
    autocast: Optional[str] = None,
    ) -> torch.dtype:
    """
    Output dtype of an operation under automatic mixed precision.
    Same rule as the reference (attorch/utils.py:27-60): outside autocast, and for
    autocast=None, the input dtype flows through; 'fp32' operations return float32;
    'fp16' operations return the low-precision autocast dtype.  One extension for
    MI355X: when the active autocast dtype is bfloat16, 'fp16' operations return
    bfloat16 (the reference only admits float16 there).

    Args:
        input_dtype: Input dtype.
        autocast: Autocast behaviour of the operation: None, 'fp16' or 'fp32'.

    Returns:
        Dtype the operation produces.
    """
    if not torch.is_autocast_enabled('cuda'):
        return input_dtype

    dtype = torch.get_autocast_dtype('cuda')
    assert dtype in (torch.float32, torch.float16, torch.bfloat16), \
        'Only fp16, bf16 and fp32 casting are supported'

    if autocast is None:
        return input_dtype
    if autocast == 'fp16':
        return dtype if dtype in LOW_PRECISION else torch.float16
    if autocast == 'fp32':
        return torch.float32
    raise RuntimeError(f'Autocast type {autocast} is invalid. '
                       'Options are None, fp16, and fp32')


def custom_bwd(bwd):
    """
    Runs ``backward`` in the autocast state its ``forward`` (decorated with
    ``torch.amp.custom_fwd(device_type='cuda')``) ran in, like
    ``torch.amp.custom_bwd(device_type='cuda')`` as the reference uses it
    (e.g. attorch/act_layers.py:83).  torch's decorator builds and enters an autocast context
    on every call; the autograd thread almost always is in that state already (no autocast in
    either pass), and then this one calls ``backward`` directly.
    """
    @functools.wraps(bwd)
    def decorate_bwd(ctx, *args, **kwargs):
        enabled = ctx._fwd_used_autocast
        if torch.is_autocast_enabled('cuda') == enabled and (
                not enabled or torch.get_autocast_dtype('cuda') == ctx._dtype):
            return bwd(ctx, *args, **kwargs)
        with torch.autocast(device_type='cuda', enabled=enabled, dtype=ctx._dtype):
            return bwd(ctx, *args, **kwargs)

    return decorate_bwd

