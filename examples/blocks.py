"""
The callers on either side of the layer-kernel hot path, as small models with synthetic inputs:
an MLP classifier (Linear+ReLU -> Linear -> CrossEntropy), a ResNet basic block
(conv -> BN+ReLU -> conv -> BN + residual + ReLU) and a GPT-style transformer block with a
language-model head (LayerNorm -> attention -> Linear+GELU -> Linear -> CrossEntropy).  They
follow the structure of attorch's examples (examples/mnist/mlp.py:14-50,
examples/imagenette/resnet.py:14-104, examples/wikitext-2/gpt.py:15-135), with the datasets
replaced by random tensors.

Each model takes `backend`: the module namespace its layers come from, either `attorch_amd.nn`
or `torch.nn`.  Fused options that only the former has (act_func of Linear / BatchNorm2d,
pre_act_add of BatchNorm2d) are spelled out as separate torch layers for the latter, and
`load_from` copies the parameters of one variant into the other so the two can be compared.
"""

from typing import Optional

import torch
from torch import Tensor
from torch import nn
from torch.nn import functional as F


def _is_fused(backend) -> bool:
    return getattr(backend, '__name__', '') == 'attorch_amd.nn'


class FusedLinear(nn.Module):
    """Linear followed by an activation: one fused layer on attorch_amd, two layers on torch."""
    def __init__(self, backend, in_dim: int, out_dim: int, act: Optional[str]) -> None:
        super().__init__()
        self.fused = _is_fused(backend)
        torch_act = {'relu': nn.ReLU, 'gelu': nn.GELU, None: nn.Identity}[act]
        if self.fused:
            self.linear = backend.Linear(in_dim, out_dim, act_func=act)
            self.act = nn.Identity()
        else:
            self.linear = backend.Linear(in_dim, out_dim)
            self.act = torch_act()

    def forward(self, input: Tensor) -> Tensor:
        return self.act(self.linear(input))

    def load_from(self, other: 'FusedLinear') -> None:
        weight = other.linear.weight.detach()
        if self.fused != other.fused:       # [in, out] on one side, [out, in] on the other
            weight = weight.T
        with torch.no_grad():
            self.linear.weight.copy_(weight)
            self.linear.bias.copy_(other.linear.bias)


class MLPClassifier(nn.Module):
    """Linear+ReLU hidden layers, a Linear head and the mean cross-entropy loss."""
    def __init__(self, backend, in_dim: int = 784, hidden_dim: int = 128, depth: int = 1,
                 num_classes: int = 10) -> None:
        super().__init__()
        dims = [in_dim] + [hidden_dim] * depth
        self.hidden = nn.ModuleList(FusedLinear(backend, a, b, 'relu') for a, b in zip(dims, dims[1:]))
        self.head = FusedLinear(backend, hidden_dim, num_classes, None)
        self.loss_func = backend.CrossEntropyLoss()

    def forward(self, input: Tensor, target: Optional[Tensor] = None) -> Tensor:
        output = input.flatten(start_dim=1)
        for layer in self.hidden:
            output = layer(output)
        output = self.head(output)
        return output if target is None else self.loss_func(output, target)

    def load_from(self, other: 'MLPClassifier') -> None:
        for mine, theirs in zip(list(self.hidden) + [self.head], list(other.hidden) + [other.head]):
            mine.load_from(theirs)


class ConvBNAct(nn.Module):
    """3x3 (or 1x1) convolution, batch normalization, optional residual and ReLU."""
    def __init__(self, backend, in_dim: int, out_dim: int, kernel_size: int = 3, stride: int = 1,
                 relu: bool = True) -> None:
        super().__init__()
        self.fused = _is_fused(backend)
        self.relu = relu
        self.conv = backend.Conv2d(in_dim, out_dim, kernel_size, stride=stride, padding=kernel_size // 2,
                                   bias=False)
        if self.fused:
            self.bn = backend.BatchNorm2d(out_dim, act_func='relu' if relu else None)
        else:
            self.bn = backend.BatchNorm2d(out_dim)

    def forward(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        output = self.conv(input)
        if self.fused:
            return self.bn(output, residual)
        output = self.bn(output)
        if residual is not None:
            output = output + residual
        return F.relu(output) if self.relu else output

    def load_from(self, other: 'ConvBNAct') -> None:
        with torch.no_grad():
            self.conv.weight.copy_(other.conv.weight)
            self.bn.weight.copy_(other.bn.weight)
            self.bn.bias.copy_(other.bn.bias)


class BasicBlock(nn.Module):
    """ResNet basic block: conv-BN-ReLU, conv-BN, + identity (1x1 conv-BN when shapes change), ReLU."""
    def __init__(self, backend, in_dim: int, out_dim: int, stride: int = 1) -> None:
        super().__init__()
        self.first = ConvBNAct(backend, in_dim, out_dim, 3, stride)
        self.second = ConvBNAct(backend, out_dim, out_dim, 3)
        self.downsample = None
        if in_dim != out_dim or stride != 1:
            self.downsample = ConvBNAct(backend, in_dim, out_dim, 1, stride, relu=False)

    def forward(self, input: Tensor) -> Tensor:
        identity = input if self.downsample is None else self.downsample(input)
        return self.second(self.first(input), identity)

    def load_from(self, other: 'BasicBlock') -> None:
        self.first.load_from(other.first)
        self.second.load_from(other.second)
        if self.downsample is not None:
            self.downsample.load_from(other.downsample)


class TransformerBlock(nn.Module):
    """Pre-norm block: x + attention(LN(x)), then + MLP(LN(.)) with a fused Linear+GELU."""
    def __init__(self, backend, dim: int, num_heads: int) -> None:
        super().__init__()
        self.num_heads = num_heads
        self.ln1 = backend.LayerNorm(dim)
        self.qkv = FusedLinear(backend, dim, 3 * dim, None)
        self.proj = FusedLinear(backend, dim, dim, None)
        self.ln2 = backend.LayerNorm(dim)
        self.fc1 = FusedLinear(backend, dim, 4 * dim, 'gelu')
        self.fc2 = FusedLinear(backend, 4 * dim, dim, None)

    def attention(self, input: Tensor) -> Tensor:
        batch, seq, dim = input.shape
        qkv = self.qkv(input).view(batch, seq, 3, self.num_heads, dim // self.num_heads)
        q, k, v = qkv.permute(2, 0, 3, 1, 4)
        # the attention core is not on the layer-kernel path: torch's on both backends
        out = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.proj(out.transpose(1, 2).reshape(batch, seq, dim))

    def forward(self, input: Tensor) -> Tensor:
        output = input + self.attention(self.ln1(input))
        return output + self.fc2(self.fc1(self.ln2(output)))

    def load_from(self, other: 'TransformerBlock') -> None:
        for name in ('qkv', 'proj', 'fc1', 'fc2'):
            getattr(self, name).load_from(getattr(other, name))
        with torch.no_grad():
            for name in ('ln1', 'ln2'):
                getattr(self, name).weight.copy_(getattr(other, name).weight)
                getattr(self, name).bias.copy_(getattr(other, name).bias)


class TinyGPT(nn.Module):
    """Embeddings, transformer blocks, final LayerNorm, vocabulary head, next-token loss."""
    def __init__(self, backend, vocab_size: int, depth: int, dim: int, num_heads: int,
                 max_seq_len: int = 512) -> None:
        super().__init__()
        self.tok_embed = nn.Embedding(vocab_size, dim)
        self.pos_embed = nn.Embedding(max_seq_len, dim)
        self.blocks = nn.ModuleList(TransformerBlock(backend, dim, num_heads) for _ in range(depth))
        self.norm = backend.LayerNorm(dim)
        self.head = FusedLinear(backend, dim, vocab_size, None)
        self.loss_func = backend.CrossEntropyLoss()

    def forward(self, tokens: Tensor, return_loss: bool = False) -> Tensor:
        positions = torch.arange(tokens.shape[1], device=tokens.device)
        output = self.tok_embed(tokens) + self.pos_embed(positions)
        for block in self.blocks:
            output = block(output)
        logits = self.head(self.norm(output))
        if not return_loss:
            return logits
        return self.loss_func(logits[:, :-1].reshape(-1, logits.shape[-1]), tokens[:, 1:].reshape(-1))

    def load_from(self, other: 'TinyGPT') -> None:
        with torch.no_grad():
            self.tok_embed.weight.copy_(other.tok_embed.weight)
            self.pos_embed.weight.copy_(other.pos_embed.weight)
            self.norm.weight.copy_(other.norm.weight)
            self.norm.bias.copy_(other.norm.bias)
        for mine, theirs in zip(self.blocks, other.blocks):
            mine.load_from(theirs)
        self.head.load_from(other.head)
