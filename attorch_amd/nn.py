"""
Interface with PyTorch fallback (the role of attorch/nn.py:1-8): every name of torch.nn, with
the layers this package implements taking precedence, so model code written against
`attorch_amd.nn` runs on the gfx950 kernels wherever they exist and on torch elsewhere.
Unlike the reference, Conv1d / Conv2d stay this package's (its convolution is a matrix-core
kernel, not a fallback candidate); AvgPool1d / AvgPool2d are torch's.
"""

from torch.nn import *  # noqa: F401,F403
from attorch_amd import *  # noqa: F401,F403
from torch.nn import AvgPool1d, AvgPool2d  # noqa: F401
