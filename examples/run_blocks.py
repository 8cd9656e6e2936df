"""
Forward + backward timing of the example blocks on one GPU with synthetic inputs, for the layers
of attorch_amd and for torch.nn with the same parameters (the role of benchmark_fw_and_bw in
attorch's examples/utils.py:13-36).  Prints one JSON line per block and backend.

    python -m examples.run_blocks [--dtype bf16|fp16|fp32] [--iters N]
"""

import argparse
import json
import sys

import torch

import attorch_amd.nn as fused_nn
from examples.blocks import BasicBlock, MLPClassifier, TinyGPT


def time_fwd_bwd(step, iters: int, warmup: int = 3) -> float:
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        step()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawTextHelpFormatter)
    parser.add_argument('--dtype', default='bf16', choices=['bf16', 'fp16', 'fp32'])
    parser.add_argument('--iters', type=int, default=20)
    args = parser.parse_args()
    if not torch.cuda.is_available():
        print('examples.run_blocks: no HIP device visible.', file=sys.stderr)
        return 2
    dtype = {'bf16': torch.bfloat16, 'fp16': torch.float16, 'fp32': torch.float32}[args.dtype]
    gen = torch.Generator().manual_seed(0)

    def make(cls, *a, **k):
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
    cases.append(('ResNet basic block 64->64, X[64,64,56,56]', make(BasicBlock, 64, 64),
                  lambda m: m(img.requires_grad_(True)).float().square().mean()))
    tok = torch.randint(0, 8192, (8, 512), generator=gen).cuda()
    cases.append(('GPT block x2, dim 1024, 16 heads, vocab 8192, tokens [8,512]',
                  make(TinyGPT, 8192, 2, 1024, 16), lambda m: m(tok, return_loss=True)))

    for name, models, run in cases:
        for backend, model in models.items():
            def step():
                model.zero_grad(set_to_none=True)
                run(model).backward()
            ms = time_fwd_bwd(step, args.iters)
            print(json.dumps({'block': name, 'backend': backend, 'dtype': args.dtype, 'ms_fwd_bwd': ms}))
    return 0


if __name__ == '__main__':
    sys.exit(main())
