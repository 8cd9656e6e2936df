"""
CPU-only tests of the host side: the C-ABI library loads and exports every symbol the header
declares, argument errors come back as negative codes without touching a GPU, the Python
wrappers raise the reference's exception types, and nothing falls back to a CPU path.
"""

import ctypes
import re
from pathlib import Path

import pytest
import torch

import attorch_amd
from attorch_amd import _lib
from attorch_amd.act import ACT_IDS, act_id, parse_act_func
from attorch_amd.utils import get_output_dtype

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / 'include' / 'attorch_hip.h').read_text()


def declared_symbols():
    return sorted(set(re.findall(r'^\s*(?:int|int64_t|const char\*)\s+(at_\w+)\s*\(', HEADER, flags=re.M)))


def test_library_exports_every_declared_symbol() -> None:
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    names = declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), f'{name} declared in include/attorch_hip.h but not exported'
    assert set(names) == set(_lib.PROTOTYPES), 'ctypes prototypes out of sync with the header'


def test_header_activation_ids_match_python_table() -> None:
    ids = dict(re.findall(r'#define AT_ACT_(\w+) (\d+)', HEADER))
    for name, value in ACT_IDS.items():
        key = 'NONE' if name is None else name.upper()
        assert int(ids[key]) == value
    assert int(ids['COUNT']) == len(ACT_IDS)


def test_version_and_error_strings() -> None:
    lib = _lib.load()
    assert lib.at_version() >= 100
    assert b'null' in lib.at_error_string(-1)
    assert b'success' in lib.at_error_string(0)
    with pytest.raises(RuntimeError, match='workspace'):
        _lib.check(-5, 'demo')


def test_argument_errors_without_gpu() -> None:
    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    # null pointers
    assert lib.at_rms_norm_fwd(None, None, None, p, 4, 8, 8, 8, 1e-5, 0, 0, 0, None) == -1
    assert lib.at_softmax_fwd(p, None, 4, 8, 8, 8, 0, 0, 0, 0, None) == -1
    assert lib.at_linear_fwd(None, p, None, None, p, 4, 8, 8, 8, 8, 8, 8, 0, 0.0, 0, 0, 0, None) == -1
    # bad dtype / dims / strides / activation
    assert lib.at_layer_norm_fwd(p, None, None, None, None, p, 4, 8, 8, 8, 1e-5, 7, 0, 0, None) == -3
    assert lib.at_layer_norm_fwd(p, None, None, None, None, p, 4, 0, 8, 8, 1e-5, 0, 0, 0, None) == -2
    assert lib.at_softmax_fwd(p, p, 4, 8, 4, 8, 0, 0, 0, 0, None) == -2
    assert lib.at_linear_fwd(p, p, None, None, p, 4, 8, 8, 8, 8, 8, 8, 99, 0.0, 0, 0, 0, None) == -4
    assert lib.at_act_bwd(p, p, p, None, None, 0, 4, 8, 8, 8, 8, 0, 0.0, 0, 0, 0, None) == -4
    assert lib.at_act_bwd(p, p, p, p, None, 0, 4, 8, 8, 8, 8, 4, 0.0, 0, 0, 0, None) == -5
    # missing / short workspace
    assert lib.at_cross_entropy_fwd_bwd(p, p, None, p, None, None, 0, 4, 8, 8, 8, -100, 0, 0, 0, 0, None) == -5
    assert lib.at_layer_norm_bwd(p, p, p, p, p, p, p, None, p, 16, 4, 8, 8, 8, 8, 0, 0, 0, 0, None) == -5
    assert lib.at_batch_norm_fwd(p, None, None, None, None, None, None, p, None, None, None, 0,
                                 4, 8, 1, 0.1, 1e-5, 0, 0.0, 0, 1, 0, 0, 0, None) == -5
    assert lib.at_act_dropout_fwd(p, p, 8, 0, 0.0, 1.5, 0, 0, None) == -2
    assert lib.at_act_dropout_bwd(p, None, p, 8, 4, 0.0, 0.0, 0, 0, None) == -1
    # NLL loss: reductions need their workspace, the reduction id must be known
    assert lib.at_nll_loss_workspace_bytes(16, 1) > 0
    assert lib.at_nll_loss_fwd(p, p, None, p, None, None, 0, 4, 8, 1, 1, 0, 0, 0, None) == -5
    assert lib.at_nll_loss_fwd(p, p, None, p, None, None, 0, 4, 8, 1, 7, 0, 0, 0, None) == -7
    assert lib.at_nll_loss_fwd(p, None, None, p, None, None, 0, 4, 8, 1, 0, 0, 0, 0, None) == -1
    assert lib.at_nll_loss_bwd(p, p, p, None, p, 4, 8, 1, 1, 0, 0, 0, None) == -1
    assert lib.at_nll_loss_bwd(p, p, None, None, p, 4, 0, 1, 1, 0, 0, 0, None) == -2
    # p-norm losses and GLU
    assert lib.at_p_loss_workspace_bytes(100) > 0
    assert lib.at_p_loss_fwd(p, p, p, None, 0, 8, 2, 1, 1.0, 0, 0, None) == -5
    assert lib.at_p_loss_fwd(p, p, p, None, 0, 8, 4, 0, 1.0, 0, 0, None) == -7
    assert lib.at_p_loss_bwd(p, p, p, None, None, 8, 2, 1, 1.0, 0, 0, 0, None) == -1
    assert lib.at_glu_fwd(p, p, 4, 8, 0, 0.0, 0, None) == -4            # the gate needs an activation
    assert lib.at_glu_fwd(p, p, 0, 8, 1, 0.0, 0, None) == 0             # nothing to do
    assert lib.at_glu_bwd(None, p, p, 4, 8, 1, 0.0, 0, None) == -1
    # inconsistent convolution geometry
    dims = [1, 4, 8, 8, 4, 9, 9, 3, 3, 1, 1, 1, 1, 1]
    assert lib.at_conv2d_fwd(p, p, None, p, None, 0, *dims, 0, 0, 0, None) == -2
    # workspace queries: the matrix-core convolution path wants 16-bit tensors and at least 16
    # contraction channels per group (padded to multiples of 64 in its channels-last copy);
    # anything else asks for no forward workspace
    good = [2, 64, 8, 8, 128, 8, 8, 3, 3, 1, 1, 1, 1, 1]
    assert lib.at_conv2d_fwd_workspace_bytes(*good, 2, 2) >= 2 * 64 * 8 * 8 * 2 + 128 * 64 * 9 * 2
    assert lib.at_conv2d_fwd_workspace_bytes(*good, 0, 0) == 0
    assert lib.at_conv2d_fwd_workspace_bytes(*dims, 2, 2) == 0
    assert lib.at_conv2d_fwd_leaves_nhwc(*good, 2, 2) == 1
    thin = list(good); thin[1] = 32                       # 32 input channels: copy padded to 64, not reusable
    assert lib.at_conv2d_fwd_workspace_bytes(*thin, 2, 2) >= 2 * 64 * 8 * 8 * 2 + 128 * 64 * 9 * 2
    assert lib.at_conv2d_fwd_leaves_nhwc(*thin, 2, 2) == 0
    thin[1] = 8
    assert lib.at_conv2d_fwd_workspace_bytes(*thin, 2, 2) == 0
    assert lib.at_conv2d_bwd_input_workspace_bytes(*good, 1) > 0
    # strided input gradient: the output gradient is spread over (OH-1)*2+1 = 7 rows and columns
    strided = list(good); strided[5] = strided[6] = 4; strided[9] = strided[10] = 2
    assert lib.at_conv2d_bwd_input_workspace_bytes(*strided, 1) >= 2 * 7 * 7 * 128 * 2 + 64 * 128 * 9 * 2
    strided[5] = strided[6] = 3; strided[9] = strided[10] = 3   # 3 x 3 strides: nine times the arithmetic, no
    assert lib.at_conv2d_bwd_input_workspace_bytes(*strided, 1) == 0
    assert lib.at_conv2d_bwd_weight_workspace_bytes(*good, 0) > 0
    # channels-last entry points: covered shapes ask for a workspace (reordered weights only), others
    # for none, and the calls say "unsupported" / "workspace" before touching the device
    assert 0 < lib.at_conv2d_nhwc_workspace_bytes(0, *good, 2) < lib.at_conv2d_fwd_workspace_bytes(*good, 2, 2)
    assert lib.at_conv2d_nhwc_workspace_bytes(1, *good, 2) > 0
    assert lib.at_conv2d_nhwc_workspace_bytes(2, *good, 2) > 0
    assert lib.at_conv2d_nhwc_workspace_bytes(0, *thin[:1], 32, *thin[2:], 2) == 0   # 32 input channels
    assert lib.at_conv2d_nhwc_workspace_bytes(0, *good, 0) == 0                       # fp32
    assert lib.at_conv2d_fwd_nhwc(p, p, None, p, None, 0, *good, 2, 0, None) == -5
    assert lib.at_conv2d_fwd_nhwc(p, p, None, p, p, 1 << 30, *good, 0, 0, None) == -7
    assert lib.at_conv2d_bwd_input_nhwc(None, p, p, p, 1 << 30, *good, 2, None) == -1
    assert lib.at_conv2d_bwd_weight_nhwc(p, p, p, None, 0, *good, 2, None) == -5
    assert lib.at_batch_norm_nhwc_supported(64, 2) == 1 and lib.at_batch_norm_nhwc_supported(1024, 0) == 1
    assert lib.at_batch_norm_nhwc_supported(7, 2) == 0 and lib.at_batch_norm_nhwc_supported(4096, 2) == 1   # wide rows: column slabs
    assert lib.at_batch_norm_fwd_nhwc(p, None, None, None, None, None, None, p, None, None, p, 1 << 30, 4, 7, 9,
                                      0.1, 1e-5, 0, 0.0, 0, 1, 2, 0, 0, None) == -7
    assert lib.at_batch_norm_bwd_nhwc(p, None, p, None, p, None, p, None, None, None, p, 1 << 30, 4, 64, 9, 0, 0.0,
                                      2, 0, None) == -1
    # one-launch backward of a small fp32 layer: argument errors before anything else
    assert lib.at_linear_bwd_small(None, p, p, p, p, p, None, 512, 784, 256, 256, 256, 784, 256, 784, 256, 4, 0.0, 0,
                                   None) == -1
    assert lib.at_linear_bwd_small(p, None, p, p, p, p, None, 512, 784, 256, 256, 256, 784, 256, 784, 256, 4, 0.0, 0,
                                   None) == -1     # an activation needs its pre-activation
    # weight gradient of the linear layer: slices of the batch for a long batch and a weight
    # matrix that is small next to the GPU
    assert lib.at_linear_bwd_weight_workspace_bytes(16384, 256, 256, 2) >= 2 * 256 * 256 * 4
    assert lib.at_linear_bwd_weight_workspace_bytes(16384, 256, 256, 0) >= 2 * 256 * 256 * 4
    assert lib.at_linear_bwd_weight_workspace_bytes(512, 256, 256, 0) == 0
    assert lib.at_linear_bwd_weight_workspace_bytes(16384, 4096, 4096, 0) == 0
    assert lib.at_linear_bwd_weight_workspace_bytes(64, 256, 256, 2) == 0
    assert lib.at_linear_bwd_weight_workspace_bytes(16384, 8192, 8192, 2) == 0
    assert lib.at_linear_bwd_weight(None, p, p, None, 0, 4, 8, 8, 8, 8, 8, 0, 0, None) == -1
    assert lib.at_norm_bwd_workspace_bytes(16, 8, 2) == 16 * 8 * 4 * 2
    assert lib.at_cross_entropy_workspace_bytes(10) == (16 + 10) * 4   # 16 partial sums of the divisor + one loss per row


def test_get_output_dtype_policy(monkeypatch) -> None:
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        for mode in (None, 'fp16', 'fp32'):
            assert get_output_dtype(dtype, mode) is dtype       # autocast disabled: flows through
    # torch refuses to enable 'cuda' autocast on a host without a GPU, so the state is faked here;
    # the GPU suite exercises the real context manager.
    monkeypatch.setattr(torch, 'is_autocast_enabled', lambda *a: True)
    monkeypatch.setattr(torch, 'get_autocast_dtype', lambda *a: torch.float16)
    assert get_output_dtype(torch.float32, None) is torch.float32
    assert get_output_dtype(torch.float32, 'fp16') is torch.float16
    assert get_output_dtype(torch.float16, 'fp32') is torch.float32
    with pytest.raises(RuntimeError):
        get_output_dtype(torch.float32, 'bf16')
    monkeypatch.setattr(torch, 'get_autocast_dtype', lambda *a: torch.bfloat16)
    assert get_output_dtype(torch.float32, 'fp16') is torch.bfloat16


def test_activation_strings() -> None:
    assert parse_act_func('leaky_relu_0.01') == ('leaky_relu', 0.01)
    assert act_id(*parse_act_func('geluapprox')) == 6
    assert act_id(None, None) == 0
    with pytest.raises(RuntimeError):
        act_id('swish', None)
    with pytest.raises(RuntimeError):
        act_id('elu', None)


def test_module_errors_match_reference() -> None:
    with pytest.raises(RuntimeError, match='integer'):
        attorch_amd.LayerNorm((8,), device='cpu')
    with pytest.raises(RuntimeError, match='integer'):
        attorch_amd.RMSNorm((8,), device='cpu')
    with pytest.raises(RuntimeError, match='averaging'):
        attorch_amd.CrossEntropyLoss(reduction='sum')
    with pytest.raises(RuntimeError, match='label smoothing'):
        attorch_amd.CrossEntropyLoss(label_smoothing=0.1)
    with pytest.raises(RuntimeError, match='dilation'):
        attorch_amd.Conv2d(4, 4, 3, dilation=2, device='cpu')
    with pytest.raises(RuntimeError, match='padding mode'):
        attorch_amd.Conv2d(4, 4, 3, padding_mode='reflect', device='cpu')
    with pytest.raises(RuntimeError, match='last dimension'):
        attorch_amd.Softmax(dim=0)(torch.zeros(2, 3))
    with pytest.raises(AssertionError):
        attorch_amd.LinearAutoGrad.apply(torch.zeros(2, 3), torch.zeros(4, 5), None, None)
    with pytest.raises(AssertionError):
        attorch_amd.CrossEntropyLossAutoGrad.apply(torch.zeros(2, 3, 4), torch.zeros(2, dtype=torch.long))


def test_linear_weight_layout_and_state_dict() -> None:
    layer = attorch_amd.Linear(6, 4, act_func='relu', device='cpu')
    assert tuple(layer.weight.shape) == (6, 4)          # [in, out], unlike torch
    assert tuple(layer.state_dict()['weight'].shape) == (6, 4)


def test_no_cpu_fallback() -> None:
    x = torch.zeros(2, 8)
    for call in (lambda: attorch_amd.LayerNorm(8, device='cpu')(x),
                 lambda: attorch_amd.RMSNorm(8, device='cpu')(x),
                 lambda: attorch_amd.Softmax(dim=-1)(x),
                 lambda: attorch_amd.Linear(8, 4, device='cpu')(x),
                 lambda: attorch_amd.CrossEntropyLoss()(x, torch.zeros(2, dtype=torch.long)),
                 lambda: attorch_amd.BatchNorm1d(8, device='cpu')(x),
                 lambda: attorch_amd.Conv2d(2, 2, 1, device='cpu')(torch.zeros(1, 2, 2, 2))):
        with pytest.raises(RuntimeError, match='no CPU path'):
            call()


def test_product_never_imports_the_oracle() -> None:
    for path in (ROOT / 'attorch_amd').rglob('*.py'):
        text = path.read_text()
        assert 'import oracle' not in text and 'from oracle' not in text, path


def test_row_stride_of_extent_one_dimensions() -> None:
    """
    PyTorch leaves the stride of an extent-1 dimension arbitrary; the C ABI checks strides against
    the row length, so a single row reports its length.
    """
    from attorch_amd import _lib
    assert _lib.row_stride(torch.zeros(5, 7)) == 7
    assert _lib.row_stride(torch.zeros(5, 12)[:, :7]) == 12
    weight = torch.zeros(63, 1).T.contiguous()            # shape [1, 63], stride(0) stays 1
    assert tuple(weight.shape) == (1, 63) and _lib.row_stride(weight) == 63
    assert _lib.row_stride(torch.zeros(0, 7)) == 7


def test_bench_final_line_stays_compact() -> None:
    """
    bench.py ends with one JSON line that a harness reads from the tail of stdout: with every
    secondary config present it must stay far below 8 KB and carry the contract fields, the
    roofline and the CPU baseline of the headline and one compact record per secondary config.
    """
    import argparse
    import json
    import bench
    head = {
        'value': 1169.123456, 'ms_per_step': 5.6412345,
        'workload': 'c4: Linear bfloat16 fwd+bwd X[16384,4096] W[4096,16384] act=geluapprox',
        'roofline': {'bound': 'mfma', 'kernel': 'linear_fwd (GEMM + bias + activation epilogue)', 'achieved': 1147.2,
                     'peak': 2500.0, 'unit': 'TFLOP/s', 'frac': 0.459, 'traffic': 4611841360},
        'cpu_baseline': {'value': 0.51, 'unit': 'TFLOP/s', 'cores': 16, 'kind': 'port',
                         'sample': 'first 2048 of 16384 rows, full K and N, oracle fwd+bwd in fp32 compute'},
        'frac_of_peak_step': 0.468,
        'kernel_ms': {'linear_fwd': 1.9, 'act_bwd_with_bias_grad': 0.28, 'linear_bwd_input': 1.7,
                      'linear_bwd_weight': 1.7, 'colsum_unfused': 0.1},
        'amp': {'ms_per_step_fp16_tensors': 5.8, 'ms_per_step_autocast_fp16_over_fp32_tensors': 6.0,
                'autocast_over_fp16': 1.03},
    }
    entry = {'tag': 'c2 GELU(tanh)+Dropout(0.1) layer', 'workload': 'x' * 200, 'value': 4234.123456, 'unit': 'GB/s',
             'roofline': {'frac': 0.5234567, 'traffic': 362346310, 'note': 'y' * 300},
             'cpu_baseline': {'value': 1.5167704445, 'unit': 'GB/s', 'cores': 16}, 'module_level': {'note': 'z' * 500}}
    head['mfma_probe'] = {'unit': 'TFLOP/s', 'tflops_constant_operands': 2465.123, 'tflops_changing_operands': 1797.456,
                          'note': 'n' * 200}
    head['frac_of_mfma_probe_step'] = 0.6534
    line = bench.compact_line(argparse.Namespace(steps=20, warmup=5), head, [dict(entry) for _ in range(24)])
    text = json.dumps(line)
    assert len(text) < 6000
    for key in ('metric', 'value', 'unit', 'n_gpus', 'steps', 'warmup', 'ms_per_step', 'higher_is_better', 'scaling',
                'vs_baseline', 'dtype', 'data', 'config', 'roofline', 'cpu_baseline'):
        assert key in line, key
    assert line['vs_baseline'] is None and line['n_gpus'] == 1
    assert set(line['roofline']) >= {'bound', 'achieved', 'peak', 'unit', 'frac', 'traffic'}
    assert set(line['cpu_baseline']) >= {'value', 'unit', 'cores', 'kind', 'sample'}
    assert len(line['configs']) == 24 and all('frac' in c and 'tag' in c for c in line['configs'])


def test_recorded_traffic_belongs_to_the_kernel_sources_in_the_tree() -> None:
    """
    bench.py reports the measured HBM traffic of its kernels only while the kernel sources have the
    digest the measurements were recorded for; a source change without a new measurement shows here.
    """
    import bench
    assert bench.kernel_source_digest() == bench.TRAFFIC_SOURCE_DIGEST
