"""
ctypes binding of libattorch_hip.so, the C-ABI library holding the gfx950 kernels.

The library is the only compute backend: if it cannot be loaded the first call raises,
there is no fallback path.  Prototypes mirror include/attorch_hip.h one to one.
"""

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p
from pathlib import Path
from typing import Optional

import torch
from torch import Tensor

LIB_PATH = Path(__file__).resolve().parent / 'lib' / 'libattorch_hip.so'

DTYPE_IDS = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

P, I, L, F, U = c_void_p, c_int, c_int64, c_float, ctypes.c_uint32

# name -> (restype, argtypes); the order is the order of include/attorch_hip.h
PROTOTYPES = {
    'at_version': (I, []),
    'at_error_string': (ctypes.c_char_p, [I]),
    'at_mfma_probe': (I, [L, I, P, P]),
    'at_mfma_probe_flop': (L, [L]),
    'at_rms_norm_fwd': (I, [P, P, P, P, L, L, L, L, F, I, I, I, P]),
    'at_rms_norm_bwd': (I, [P, P, P, P, P, P, P, L, L, L, L, L, L, I, I, I, I, P]),
    'at_norm_bwd_workspace_bytes': (L, [L, L, I]),
    'at_layer_norm_fwd': (I, [P, P, P, P, P, P, L, L, L, L, F, I, I, I, P]),
    'at_layer_norm_bwd': (I, [P, P, P, P, P, P, P, P, P, L, L, L, L, L, L, I, I, I, I, P]),
    'at_softmax_fwd': (I, [P, P, L, L, L, L, I, I, I, I, P]),
    'at_softmax_bwd': (I, [P, P, P, L, L, L, L, L, I, I, I, I, I, P]),
    'at_cross_entropy_workspace_bytes': (L, [L]),
    'at_cross_entropy_fwd_bwd': (I, [P, P, P, P, P, P, L, L, L, L, L, L, I, I, I, I, P]),
    'at_cross_entropy_bwd': (I, [P, P, P, P, P, P, L, L, L, L, L, I, I, I, I, I, P]),
    'at_cross_entropy_scale_grad': (I, [P, P, L, L, L, I, I, P]),
    'at_cross_entropy_static_max_batch': (L, []),
    'at_cross_entropy_fwd_bwd_static': (I, [P, P, P, P, P, L, L, L, L, L, I, I, I, I, P]),
    'at_nll_loss_workspace_bytes': (L, [L, L]),
    'at_nll_loss_fwd': (I, [P, P, P, P, P, P, L, L, L, L, I, I, I, I, P]),
    'at_nll_loss_bwd': (I, [P, P, P, P, P, L, L, L, I, I, I, I, P]),
    'at_p_loss_workspace_bytes': (L, [L]),
    'at_p_loss_fwd': (I, [P, P, P, P, L, L, I, I, F, I, I, P]),
    'at_p_loss_bwd': (I, [P, P, P, P, P, L, I, I, F, I, I, I, P]),
    'at_glu_fwd': (I, [P, P, L, L, I, F, I, P]),
    'at_glu_bwd': (I, [P, P, P, L, L, I, F, I, P]),
    'at_linear_fwd': (I, [P, P, P, P, P, L, L, L, L, L, L, L, I, F, I, I, I, P]),
    'at_linear_bwd_input': (I, [P, P, P, L, L, L, L, L, L, I, I, P]),
    'at_linear_bwd_weight_workspace_bytes': (L, [L, L, L, I]),
    'at_linear_bwd_small_supported': (I, [L, L, L, I]),
    'at_linear_bwd_wide_output_supported': (I, [L, L, L, I]),
    'at_linear_bwd_small': (I, [P, P, P, P, P, P, P, L, L, L, L, L, L, L, L, L, I, F, I, P]),
    'at_linear_bwd_weight': (I, [P, P, P, P, L, L, L, L, L, L, L, I, I, P]),
    'at_act_bwd_workspace_bytes': (L, [L, L]),
    'at_act_bwd': (I, [P, P, P, P, P, L, L, L, L, L, L, I, F, I, I, I, P]),
    'at_colsum_workspace_bytes': (L, [L, L]),
    'at_colsum': (I, [P, P, P, L, L, L, L, I, I, P]),
    'at_batch_norm_workspace_bytes': (L, [L]),
    'at_batch_norm_fwd': (I, [P, P, P, P, P, P, P, P, P, P, P, L, L, L, L, F, F, I, F, I, I, I, I, I, P]),
    'at_batch_norm_nhwc_supported': (I, [L, I]),
    'at_batch_norm_fwd_nhwc': (I, [P, P, P, P, P, P, P, P, P, P, P, L, L, L, L, F, F, I, F, I, I, I, I, I, P]),
    'at_batch_norm_bwd_nhwc': (I, [P, P, P, P, P, P, P, P, P, P, P, L, L, L, L, I, F, I, I, P]),
    'at_conv2d_fwd_workspace_bytes': (L, [L] * 14 + [I, I]),
    'at_conv2d_fwd_leaves_nhwc': (I, [L] * 14 + [I, I]),
    'at_conv2d_nhwc_workspace_bytes': (L, [I] + [L] * 14 + [I]),
    'at_conv2d_fwd_nhwc': (I, [P, P, P, P, P, L] + [L] * 14 + [I, I, P]),
    'at_conv2d_bwd_input_nhwc': (I, [P, P, P, P, L] + [L] * 14 + [I, P]),
    'at_conv2d_bwd_weight_nhwc': (I, [P, P, P, P, L] + [L] * 14 + [I, P]),
    'at_conv2d_fwd': (I, [P, P, P, P, P, L] + [L] * 14 + [I, I, I, P]),
    'at_conv2d_bwd_input_workspace_bytes': (L, [L] * 14 + [I]),
    'at_conv2d_bwd_input': (I, [P, P, P, P, P, L] + [L] * 14 + [I, P]),
    'at_conv2d_bwd_weight_workspace_bytes': (L, [L] * 14 + [I]),
    'at_conv2d_bwd_weight': (I, [P, P, P, P, P, P, L] + [L] * 14 + [I, P]),
    'at_nchw_to_nhwc': (I, [P, P, L, L, L, I, P]),
    'at_channel_sum': (I, [P, P, L, L, L, I, I, P]),
    'at_act_dropout_fwd': (I, [P, P, L, I, F, F, U, I, P]),
    'at_act_dropout_bwd': (I, [P, P, P, L, I, F, F, U, I, P]),
    'at_batch_norm_bwd': (I, [P, P, P, P, P, P, P, P, P, P, P, L, L, L, L, I, F, I, I, P]),
}

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """
    Loads the shared library once and declares every prototype.

    Raises:
        RuntimeError: The library has not been built or misses an entry point.
    """
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(f'{LIB_PATH} is missing: build it with `python -m attorch_amd.build` '
                           '(the HIP library is the only backend, there is no fallback)')
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in PROTOTYPES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as err:
            raise RuntimeError(f'{LIB_PATH} does not export {name}; rebuild it') from err
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    """
    Converts a non-zero return code of the library into a RuntimeError.
    """
    if code != 0:
        msg = load().at_error_string(code).decode()
        raise RuntimeError(f'{what} failed with code {code}: {msg}')


def ptr(tensor: Optional[Tensor]) -> Optional[int]:
    """
    Device address of a tensor, None for an absent optional.
    """
    return None if tensor is None else tensor.data_ptr()


def dtype_id(dtype: torch.dtype) -> int:
    """
    AT_DTYPE_* id of a torch dtype.
    """
    try:
        return DTYPE_IDS[dtype]
    except KeyError:
        raise RuntimeError(f'dtype {dtype} is not supported; use float32, float16 or bfloat16') from None


def stream_of(tensor: Tensor) -> int:
    """
    Raw hipStream_t of the current PyTorch stream on the tensor's device.
    """
    # the raw handle straight from the C extension: torch.cuda.current_stream() builds a Stream
    # object first, several microseconds of a call that is made once per launch
    return torch._C._cuda_getCurrentRawStream(tensor.get_device())


class _NoGuard:
    """
    Stand-in for a device guard when the wanted device is already the current one.
    """
    def __enter__(self) -> None:
        return None

    def __exit__(self, *exc: object) -> bool:
        return False


_NO_GUARD = _NoGuard()


def device_guard(tensor: Tensor):
    """
    Context manager that makes the tensor's device the current one for the launches inside it;
    free of cost in the usual case that it already is.
    """
    if tensor.get_device() == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device_of(tensor)


def require_gpu(tensor: Tensor, what: str) -> None:
    """
    The kernels only run on the GPU: refuse host tensors loudly instead of falling back.
    """
    if not tensor.is_cuda:
        raise RuntimeError(f'{what}: expected a tensor on a HIP device (device type "cuda"), '
                           f'received one on {tensor.device}; there is no CPU path')


def require_same_device(what: str, reference: Tensor, *others: Optional[Tensor]) -> None:
    """
    Every tensor whose address goes to a kernel must live on the device of `reference` (the
    tensor whose device the launch runs on): a host pointer, or one of another GPU, handed to a
    kernel ends in a memory fault instead of an error.  Absent optionals (None) are skipped.
    """
    require_gpu(reference, what)
    for other in others:
        if other is None:
            continue
        if other.device != reference.device:
            raise RuntimeError(f'{what}: expected all tensors on {reference.device}, '
                               f'received one on {other.device}')


def rows(tensor: Tensor) -> Tensor:
    """
    Returns the tensor as a [rows, feat] matrix with unit stride along feat.
    """
    if tensor.ndim == 1:
        tensor = tensor.unsqueeze(0)
    tensor = tensor.flatten(0, -2) if tensor.ndim != 2 else tensor
    if tensor.stride(-1) != 1 or (tensor.shape[0] > 1 and tensor.stride(0) < tensor.shape[1]):
        tensor = tensor.contiguous()
    return tensor


def row_stride(tensor: Tensor) -> int:
    """
    Row stride of a [rows, feat] matrix in elements, as the kernels expect it.  PyTorch leaves
    the stride of an extent-1 dimension arbitrary (a [1, feat] or [feat, 1].T tensor counts as
    contiguous whatever stride(0) says), so a single row reports its extent instead.
    """
    if tensor.shape[0] <= 1:
        return max(int(tensor.shape[1]), 1)
    return int(tensor.stride(0))


def in_memory_format(tensor: Tensor, memory_format: torch.memory_format) -> Tensor:
    """
    `tensor.contiguous(memory_format=...)`, with the library's tiled transpose for the one case the
    layers meet on their hot path: a 16-bit NCHW-contiguous device tensor wanted channels-last
    (an upstream gradient that some other operator produced in the default format).
    """
    if tensor.is_contiguous(memory_format=memory_format):
        return tensor
    if (memory_format is torch.channels_last and tensor.dim() == 4 and tensor.is_cuda
            and tensor.dtype in (torch.float16, torch.bfloat16) and tensor.is_contiguous() and tensor.numel() > 0
            and tensor.shape[0] <= 65535):
        batch, feat, height, width = tensor.shape
        out = torch.empty_like(tensor, memory_format=torch.channels_last)
        with device_guard(tensor):
            check(load().at_nchw_to_nhwc(ptr(tensor), ptr(out), batch, feat, height * width, dtype_id(tensor.dtype),
                                         stream_of(tensor)), 'at_nchw_to_nhwc')
        return out
    return tensor.contiguous(memory_format=memory_format)
