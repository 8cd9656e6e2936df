"""
The allocation-free cross-entropy entry point (workspace inside the library) against the
entry point that takes a caller-allocated workspace: same kernels, so loss and gradient must be
bit-identical.  Two calls in a row, the second on a smaller input (the library's workspace keeps
what the first call left in it), each through the raw C ABI.
"""

import pytest
import torch

from attorch_amd import _lib
from .helpers import randn

pytestmark = pytest.mark.gpu


def run_pair(lib, rows, vocab, dtype, out_dtype, weighted, seed):
    x = randn((rows, vocab), seed, dtype, 2.0).cuda()
    gen = torch.Generator().manual_seed(seed + 1)
    target = torch.randint(0, vocab, (rows,), generator=gen)
    target[torch.rand(rows, generator=gen) < 0.1] = -100
    target = target.cuda()
    weight = (0.5 + torch.rand(vocab, generator=gen)).cuda() if weighted else None
    stream = _lib.stream_of(x)
    ids = (_lib.dtype_id(dtype), 0 if weight is None else _lib.dtype_id(weight.dtype), _lib.dtype_id(out_dtype),
           _lib.dtype_id(out_dtype))

    loss_a = torch.empty((), dtype=out_dtype, device='cuda')
    grad_a = torch.empty(rows, vocab, dtype=out_dtype, device='cuda')
    ws_bytes = lib.at_cross_entropy_workspace_bytes(rows)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device='cuda')
    _lib.check(lib.at_cross_entropy_fwd_bwd(
        x.data_ptr(), target.data_ptr(), _lib.ptr(weight), loss_a.data_ptr(), grad_a.data_ptr(), ws.data_ptr(),
        ws_bytes, rows, vocab, vocab, vocab, -100, *ids, stream), 'at_cross_entropy_fwd_bwd')

    loss_b = torch.empty((), dtype=out_dtype, device='cuda')
    grad_b = torch.full((rows, vocab), float('nan'), dtype=out_dtype, device='cuda')
    def call_static():
        _lib.check(lib.at_cross_entropy_fwd_bwd_static(
            x.data_ptr(), target.data_ptr(), _lib.ptr(weight), loss_b.data_ptr(), grad_b.data_ptr(),
            rows, vocab, vocab, vocab, -100, *ids, stream), 'at_cross_entropy_fwd_bwd_static')
    call_static()      # the first call on a device looks up the address of the library's workspace
    torch.cuda.synchronize()
    # neither torch's caching allocator nor the device's free memory (what a hipMalloc inside the
    # library would take from) moves across a call
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    grad_b.fill_(float('nan'))
    call_static()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(loss_a, loss_b), (loss_a.item(), loss_b.item())
    assert torch.equal(grad_a, grad_b)
    assert not torch.isnan(loss_b).item()


def test_static_workspace_matches_caller_workspace_on_two_calls_in_a_row() -> None:
    lib = _lib.load()
    assert lib.at_cross_entropy_static_max_batch() == 65536
    # the second call of each pair is smaller than the one before it
    run_pair(lib, 4096, 1000, torch.float32, torch.float32, True, 11)
    run_pair(lib, 37, 129, torch.float32, torch.float32, False, 12)
    run_pair(lib, 2048, 50257, torch.float16, torch.float16, False, 13)
    run_pair(lib, 512, 4099, torch.float16, torch.float32, True, 14)
    run_pair(lib, 65536, 16, torch.bfloat16, torch.bfloat16, False, 15)
    run_pair(lib, 3, 8, torch.bfloat16, torch.float32, False, 16)


def test_static_workspace_rejects_batches_beyond_its_limit() -> None:
    lib = _lib.load()
    rows, vocab = 65537, 4
    x = torch.zeros(rows, vocab, device='cuda')
    target = torch.zeros(rows, dtype=torch.int64, device='cuda')
    loss = torch.empty((), device='cuda')
    rc = lib.at_cross_entropy_fwd_bwd_static(x.data_ptr(), target.data_ptr(), None, loss.data_ptr(), None,
                                             rows, vocab, vocab, vocab, -100, 0, 0, 0, 0, _lib.stream_of(x))
    assert rc == -5   # AT_ERR_WORKSPACE
    with pytest.raises(RuntimeError, match='workspace'):
        _lib.check(rc, 'at_cross_entropy_fwd_bwd_static')


def test_static_entry_point_is_capturable_in_a_graph() -> None:
    """
    After one eager call on the device (which looks up the workspace address; that first call
    belongs outside a capture) the entry point consists of kernel launches only: captured in a HIP
    graph and replayed several times with eager work in between, every replay gives the eager result.
    """
    lib = _lib.load()
    rows, vocab = 1024, 4099
    x = randn((rows, vocab), 21, torch.float16, 2.0).cuda()
    gen = torch.Generator().manual_seed(22)
    target = torch.randint(0, vocab, (rows,), generator=gen)
    target[torch.rand(rows, generator=gen) < 0.1] = -100
    target = target.cuda()
    loss = torch.empty((), dtype=torch.float16, device='cuda')
    grad = torch.empty(rows, vocab, dtype=torch.float16, device='cuda')
    f16 = _lib.dtype_id(torch.float16)

    def call() -> None:
        _lib.check(lib.at_cross_entropy_fwd_bwd_static(
            x.data_ptr(), target.data_ptr(), None, loss.data_ptr(), grad.data_ptr(), rows, vocab, vocab, vocab,
            -100, f16, 0, f16, f16, torch.cuda.current_stream().cuda_stream), 'at_cross_entropy_fwd_bwd_static')

    call()
    torch.cuda.synchronize()
    loss_eager, grad_eager = loss.clone(), grad.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for replay in range(3):
        grad.fill_(float('nan'))
        loss.fill_(float('nan'))
        (x.float().sum()).item()        # eager work and a synchronisation between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(loss, loss_eager), replay
        assert torch.equal(grad, grad_eager), replay
