"""
The kernels are launched on PyTorch's current stream of the tensors' device, forward and (through
the autograd engine, which restores the forward's stream) backward.
"""

import pytest
import torch

import attorch_amd

pytestmark = pytest.mark.gpu


def _pipeline(a, linear, norm, conv, bn):
    x = a
    for _ in range(12):                       # milliseconds of producer work on the same stream
        x = torch.tanh(x @ a * 0.01)
    y = norm(linear(x))
    img = y[:, :256].reshape(4, 64, 64, 64) * 0.1
    z = bn(conv(img))
    loss = y.square().mean() + z.square().mean()
    grads = torch.autograd.grad(loss, [linear.weight, linear.bias, norm.weight, conv.weight, bn.weight])
    return [y, z, *grads]


def test_layers_run_on_the_current_stream() -> None:
    """
    Inputs are produced by long matmul chains on a side stream (default priority) and consumed by
    the layers on that stream without any synchronisation in between: had a kernel been launched on
    another stream, it would read the producer's buffer before it is written.
    """
    torch.manual_seed(0)
    a = torch.randn(4096, 4096, device='cuda')
    linear = attorch_amd.Linear(4096, 512, act_func='relu', device='cuda')
    norm = attorch_amd.LayerNorm(512, device='cuda')
    conv = attorch_amd.Conv2d(64, 32, 3, padding=1, device='cuda')
    bn = attorch_amd.BatchNorm2d(32, act_func='relu', device='cuda')
    torch.cuda.synchronize()
    expected = _pipeline(a, linear, norm, conv, bn)
    torch.cuda.synchronize()
    bn.running_mean.zero_(), bn.running_var.fill_(1.0)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            bn.running_mean.zero_(), bn.running_var.fill_(1.0)
            got = _pipeline(a, linear, norm, conv, bn)
    side.synchronize()
    for e, g in zip(expected, got):
        torch.testing.assert_close(g, e, rtol=0, atol=0)


def test_matrix_core_probe_runs_and_counts_its_work() -> None:
    """
    at_mfma_probe launches on the given stream and returns; at_mfma_probe_flop is 2 workgroups x 4
    waves per CU x iters x 64 MFMAs of 32 x 32 x 16.  Changing operands must not come out faster
    than a constant pair by more than measurement noise.
    """
    from attorch_amd import _lib
    lib = _lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    iters = 500
    assert lib.at_mfma_probe_flop(iters) == cus * 2 * 4 * iters * 64 * 2 * 32 * 32 * 16
    assert lib.at_mfma_probe_flop(0) == 0
    scratch = torch.zeros(4, dtype=torch.uint8, device='cuda')
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.at_mfma_probe(iters, 0, None, stream) == -1          # null scratch
    assert lib.at_mfma_probe(0, 0, scratch.data_ptr(), stream) == -2
    times = []
    for rnd in (0, 1):
        for _ in range(2):
            _lib.check(lib.at_mfma_probe(iters, rnd, scratch.data_ptr(), stream), 'probe')
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        _lib.check(lib.at_mfma_probe(iters, rnd, scratch.data_ptr(), stream), 'probe')
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end))
    assert scratch.sum().item() == 0
    assert times[1] > 0.9 * times[0]
