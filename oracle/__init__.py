"""
CPU oracle for the attorch layer-kernel hot path.

TEST INFRASTRUCTURE ONLY.  This package restates, in plain PyTorch CPU tensor arithmetic
(fp32, or fp64 on request), the algorithms of the reference's kernels and autograd Functions.
Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import it; the
product package attorch_amd never does and has no CPU path.

Every function cites the reference lines it follows (paths relative to the reference root).
The restatement is pinned in tests/test_oracle_*.py against independent implementations:
torch.nn.functional + autograd (the oracle of the reference's own tests), the known-answer
activation boundary points of the reference's tests/test_act_layers.py:55-61, brute-force
loops on tiny inputs, and closed-form invariants.  Parity status: every function here is
pinned by at least one such check; none is "parity unpinned".
"""

from .acts import ACT_NAMES, act_forward, act_grad, parse_act_func
from .layers import (act_dropout_backward, act_dropout_forward, batch_norm_backward, batch_norm_forward, conv2d_backward, conv2d_forward,
                     cross_entropy_backward, cross_entropy_forward, glu_backward, glu_forward,
                     layer_norm_backward,
                     layer_norm_forward, linear_backward, linear_forward, nll_loss_backward,
                     nll_loss_forward, p_loss_backward, p_loss_forward, rms_norm_backward,
                     rms_norm_forward, softmax_backward, softmax_forward)
