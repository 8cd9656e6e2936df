"""
Forward / backward timing of the example blocks on one GPU with synthetic inputs, for the layers
of attorch_amd and for torch.nn with the same parameters: the role of benchmark_fw_and_bw in
attorch's examples/utils.py:13-36 (forward pass, then backward passes through one retained
graph, each a mean over repeated calls, optionally under automatic mixed precision), plus the
forward + backward step measured as one.  Prints one JSON line per block and backend with
ms_fwd, ms_bwd and ms_fwd_bwd.

    python -m examples.run_blocks [--dtype bf16|fp16|fp32] [--amp] [--amp-dtype fp16|bf16] [--iters N]
                                  [--channels-last]

--amp keeps parameters and inputs in float32 and runs the forward pass under torch.autocast, as
the reference's examples do by default; --dtype then only names the storage dtype of the non-AMP
runs and is ignored.  --channels-last hands the ResNet block its image in torch.channels_last
memory format: Conv2d and BatchNorm2d of attorch_amd then work on that layout without copies.
"""

import argparse
import json
import sys
from typing import Callable, Dict, Tuple

import torch

import attorch_amd.nn as fused_nn
from examples.blocks import BasicBlock, MLPClassifier, TinyGPT


def mean_ms(fn: Callable[[], None], iters: int, warmup: int = 3) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def benchmark_fw_and_bw(model: torch.nn.Module, run: Callable[[torch.nn.Module], torch.Tensor], amp: bool,
                        amp_dtype: torch.dtype, iters: int) -> Tuple[float, float, float]:
    """
    Mean time in ms of the forward pass, of the backward pass (repeated through one retained
    graph, as examples/utils.py:29-32 does) and of a whole forward + backward step.
    """
    def forward() -> torch.Tensor:
        with torch.autocast('cuda', dtype=amp_dtype, enabled=amp):
            return run(model)

    fw = mean_ms(forward, iters)
    output = forward()
    output_grad = torch.randn_like(output)
    bw = mean_ms(lambda: output.backward(output_grad, retain_graph=True), iters)
    del output

    def step() -> None:
        model.zero_grad(set_to_none=True)
        forward().backward(output_grad)
    return fw, bw, mean_ms(step, iters)


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawTextHelpFormatter)
    parser.add_argument('--dtype', default='bf16', choices=['bf16', 'fp16', 'fp32'])
    parser.add_argument('--amp', action='store_true',
                        help='float32 parameters and inputs, forward under torch.autocast')
    parser.add_argument('--amp-dtype', default='fp16', choices=['fp16', 'bf16'])
    parser.add_argument('--iters', type=int, default=20)
    parser.add_argument('--channels-last', action='store_true',
                        help='ResNet block input in torch.channels_last memory format')
    args = parser.parse_args()
    if not torch.cuda.is_available():
        print('examples.run_blocks: no HIP device visible.', file=sys.stderr)
        return 2
    names = {'bf16': torch.bfloat16, 'fp16': torch.float16, 'fp32': torch.float32}
    dtype = torch.float32 if args.amp else names[args.dtype]
    amp_dtype = names[args.amp_dtype]
    gen = torch.Generator().manual_seed(0)

    def make(cls, *a, **k) -> Dict[str, torch.nn.Module]:
        ours = cls(fused_nn, *a, **k).to('cuda', dtype)
        theirs = cls(torch.nn, *a, **k).to('cuda', dtype)
        theirs.load_from(ours)
        return {'attorch_amd': ours, 'torch': theirs}

    cases = []
    x = torch.randn(4096, 784, generator=gen).to('cuda', dtype)
    t = torch.randint(0, 10, (4096,), generator=gen).cuda()
    cases.append(('MLP 784-2048-2048-10, batch 4096', make(MLPClassifier, 784, 2048, 2, 10),
                  lambda m: m(x, t)))
    img = torch.randn(64, 64, 56, 56, generator=gen).to('cuda', dtype)
    if args.channels_last:
        img = img.contiguous(memory_format=torch.channels_last)
    img.requires_grad_(True)
    cases.append(('ResNet basic block 64->64, X[64,64,56,56]' + (' channels-last' if args.channels_last else ''),
                  make(BasicBlock, 64, 64),
                  lambda m: m(img)))   # the block's output itself: its random upstream gradient keeps its memory format
    tok = torch.randint(0, 8192, (8, 512), generator=gen).cuda()
    cases.append(('GPT block x2, dim 1024, 16 heads, vocab 8192, tokens [8,512]',
                  make(TinyGPT, 8192, 2, 1024, 16), lambda m: m(tok, return_loss=True)))

    for name, models, run in cases:
        for backend, model in models.items():
            fw, bw, both = benchmark_fw_and_bw(model, run, args.amp, amp_dtype, args.iters)
            print(json.dumps({'block': name, 'backend': backend,
                              'dtype': f'amp({args.amp_dtype})' if args.amp else args.dtype,
                              'ms_fwd': fw, 'ms_bwd': bw, 'ms_fwd_bwd': both}))
    return 0


if __name__ == '__main__':
    sys.exit(main())
