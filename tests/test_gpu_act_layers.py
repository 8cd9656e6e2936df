"""
GPU parity tests of the standalone activation layers with fused dropout and of Dropout against
the CPU oracle; grids follow the reference's tests/test_act_layers.py and
tests/test_dropout_layer.py (every layer class, dropout on and off, fp32 and 16-bit inputs,
autocast, the piece boundaries, the drop rates).  The dropout mask is read off the device
result, as the reference's tests do; what the tests add is that the mask must be a pure
function of (seed, position): the same in forward and backward, in every dtype and for every
alignment of the buffers.
"""

import pytest
import torch

import attorch_amd
import oracle
from attorch_amd import _lib
from .helpers import DTYPES, assert_close, compute_dtype, randn

pytestmark = pytest.mark.gpu

LAYERS = [('Sigmoid', 'sigmoid', {}), ('LogSigmoid', 'logsigmoid', {}), ('Tanh', 'tanh', {}),
          ('ReLU', 'relu', {}), ('GELU', 'gelu', {}), ('GELU', 'geluapprox', {'approximate': 'tanh'}),
          ('SiLU', 'silu', {}), ('ReLU6', 'relu6', {}), ('Hardsigmoid', 'hardsigmoid', {}),
          ('Hardtanh', 'hardtanh', {}), ('Hardswish', 'hardswish', {}), ('SELU', 'selu', {}),
          ('Mish', 'mish', {}), ('Softplus', 'softplus', {}), ('Softsign', 'softsign', {}),
          ('Tanhshrink', 'tanhshrink', {}), ('LeakyReLU', 'leaky_relu_0.01', {}),
          ('ELU', 'elu_1.0', {}), ('CELU', 'celu_1.0', {}), ('Hardshrink', 'hardshrink_0.5', {}),
          ('Softshrink', 'softshrink_0.5', {}), ('LeakyReLU', 'leaky_relu_0.2', {'negative_slope': 0.2}),
          ('ELU', 'elu_0.7', {'alpha': 0.7}), ('Softshrink', 'softshrink_0.25', {'lambd': 0.25})]
SHAPES = [(96,), (4, 2000), (8, 1024), (2049, 2), (8, 960, 196), (1, 3, 7, 5, 3)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('cls, act_func, kwargs', LAYERS)
@pytest.mark.parametrize('drop_p', [0.0, 0.5])
def test_act_layers(cls, act_func, kwargs, shape, dtype, drop_p, monkeypatch) -> None:
    # The layer draws its seed with random.randint; pinning it lets the test ask the library for
    # the very mask it used (where an activation is exactly zero, e.g. hardswish at -3, the
    # output alone cannot tell a dropped element from a kept one, but the gradient can).
    monkeypatch.setattr(attorch_amd.act_layers, 'randint', lambda lo, hi: 4711)
    x = randn(shape, 1, dtype, 2.0)
    dy = randn(shape, 2, dtype)
    name, param = oracle.parse_act_func(act_func)
    layer = getattr(attorch_amd, cls)(drop_p=drop_p, **kwargs)

    xd = x.cuda().requires_grad_(True)
    y = layer(xd)
    y.backward(dy.cuda())
    assert y.dtype is dtype and y.shape == x.shape

    cd = compute_dtype(dtype)
    dropped = None
    if drop_p > 0:
        dropped = _c_abi_mask(x.numel(), drop_p, 4711, torch.float32)[0].cpu().view(x.shape)
        assert torch.count_nonzero(y.detach().cpu()[dropped]) == 0
        if x.numel() >= 4096:
            assert abs(dropped.float().mean().item() - drop_p) < 0.05
    assert_close(y, oracle.act_dropout_forward(x, name, param, dropped, drop_p, compute=cd), dtype, 'output')
    assert_close(xd.grad, oracle.act_dropout_backward(dy, x, name, param, dropped, drop_p, compute=cd), dtype,
                 'input_grad')


@pytest.mark.parametrize('cls, kwargs, boundaries',
                         [('Hardshrink', {}, [-0.5, 0.5]), ('Softshrink', {}, [-0.5, 0.5]),
                          ('Hardswish', {}, [-3.0, 3.0]), ('Hardsigmoid', {}, [-3.0, 3.0]),
                          ('Hardtanh', {}, [-1.0, 1.0]), ('ReLU6', {}, [0.0, 6.0])])
def test_act_layers_at_piece_boundaries(cls, kwargs, boundaries) -> None:
    # tests/test_act_layers.py:55-78 of the reference: values and gradients at the joints
    ours = torch.tensor(boundaries, device='cuda', requires_grad=True)
    theirs = torch.tensor(boundaries, device='cuda', requires_grad=True)
    out = getattr(attorch_amd, cls)(**kwargs)(ours)
    ref = getattr(torch.nn, cls)(**kwargs)(theirs)
    torch.testing.assert_close(out, ref, rtol=1e-3, atol=1e-3)
    out.backward(torch.ones_like(out))
    ref.backward(torch.ones_like(ref))
    expected_grad = theirs.grad
    if cls == 'Hardswish':
        # The reference formula (act_kernels.py:328) gives x / 3 + 0.5 at both joints, as the
        # device kernel of the torch build its tests ran against; torch builds differ there
        # (this one and the CPU kernel give 0 and 1), so the joints are pinned to the formula.
        expected_grad = torch.tensor([-0.5, 1.5], device='cuda')
    torch.testing.assert_close(ours.grad, expected_grad, rtol=1e-3, atol=1e-3)


def test_act_layers_eval_autocast_and_options() -> None:
    x = randn((64, 300), 1).cuda().requires_grad_(True)
    layer = attorch_amd.GELU(drop_p=0.9)
    layer.eval()                                         # no dropout outside training
    torch.testing.assert_close(layer(x), torch.nn.functional.gelu(x), rtol=1e-4, atol=1e-5)
    with torch.autocast('cuda', dtype=torch.float16):    # dtype flows through (no cast policy)
        assert attorch_amd.ReLU()(x).dtype is torch.float32
        assert attorch_amd.ReLU()(x.half()).dtype is torch.float16
    with pytest.raises(RuntimeError):
        attorch_amd.GELU(approximate='erf')
    with pytest.raises(RuntimeError):
        attorch_amd.Hardtanh(min_val=-2.0)
    with pytest.warns(UserWarning):
        attorch_amd.ReLU(inplace=True)
    with pytest.raises(RuntimeError):
        attorch_amd.ActFuncAutoGrad.apply(x, 'swoosh', 0.0, True)


@pytest.mark.parametrize('shape', [(96,), (8, 1024), (2049, 2), (64, 960, 49)])
@pytest.mark.parametrize('drop_p', [0.0, 0.15, 0.3, 0.5, 0.75, 0.9, 1.0])
def test_dropout_layer(shape, drop_p) -> None:
    # tests/test_dropout_layer.py of the reference
    x = randn(shape, 1)
    x[x == 0] = 1.0            # an input that is zero already would read as dropped below
    x = x.cuda().requires_grad_(True)
    y = attorch_amd.Dropout(drop_p)(x)
    n_zeroed = (torch.count_nonzero(x) - torch.count_nonzero(y)).item()
    if drop_p == 0:
        assert n_zeroed == 0 and torch.equal(y, x)
    elif drop_p == 1:
        assert torch.count_nonzero(y).item() == 0
    else:
        dropped = (y.detach().cpu() == 0)
        assert_close(y, oracle.act_dropout_forward(x.detach().cpu(), None, None, dropped, drop_p),
                     torch.float32, 'output')
        if x.numel() >= 2048:
            assert abs(n_zeroed / x.numel() - drop_p) < 0.05
    dy = randn(shape, 2).cuda()
    y.backward(dy)
    expected = torch.where(y.detach() == 0, torch.zeros_like(dy), dy / (1 - drop_p)) if drop_p < 1 \
        else torch.zeros_like(dy)
    torch.testing.assert_close(x.grad, expected, rtol=1e-4, atol=1e-5)
    assert not attorch_amd.Dropout(0.5).eval()(x).eq(0).any()


def _c_abi_mask(n, drop_p, seed, dtype, offset_elems=0):
    """Forward of plain dropout on a tensor of ones through the C ABI; returns the dropped mask."""
    lib = _lib.load()
    base = torch.ones(n + offset_elems, dtype=dtype, device='cuda')
    x = base[offset_elems:]
    y = torch.empty(n + offset_elems, dtype=dtype, device='cuda')[offset_elems:]
    _lib.check(lib.at_act_dropout_fwd(x.data_ptr(), y.data_ptr(), n, 0, 0.0, drop_p, seed,
                                      _lib.dtype_id(dtype), _lib.stream_of(x)), 'fwd')
    return y == 0, y


def test_dropout_mask_is_a_function_of_seed_and_position() -> None:
    n = 1 << 20
    m32, y32 = _c_abi_mask(n + 5, 0.3, 1234, torch.float32)
    m16, _ = _c_abi_mask(n + 5, 0.3, 1234, torch.bfloat16)
    assert torch.equal(m32, m16)                                  # dtype (vector width) does not matter
    m_unaligned, _ = _c_abi_mask(n + 5, 0.3, 1234, torch.float32, offset_elems=1)
    assert torch.equal(m32, m_unaligned)                          # nor does the scalar path
    assert torch.equal(m32, _c_abi_mask(n + 5, 0.3, 1234, torch.float32)[0])   # repeatable
    other, _ = _c_abi_mask(n + 5, 0.3, 4321, torch.float32)
    assert 0.35 < (m32 != other).float().mean().item() < 0.49     # 2 p (1 - p) = 0.42 for independent masks
    assert abs(m32.float().mean().item() - 0.3) < 0.005
    torch.testing.assert_close(y32[~m32], torch.full_like(y32[~m32], 1 / 0.7))
    # backward draws the same mask
    lib = _lib.load()
    dy = torch.ones(n + 5, device='cuda')
    dx = torch.empty_like(dy)
    _lib.check(lib.at_act_dropout_bwd(dy.data_ptr(), None, dx.data_ptr(), n + 5, 0, 0.0, 0.3, 1234, 0,
                                      _lib.stream_of(dy)), 'bwd')
    assert torch.equal(dx == 0, m32)
    # neighbouring elements are not correlated: P(both dropped) = p^2
    both = (m32[:-1] & m32[1:]).float().mean().item()
    assert abs(both - 0.09) < 0.005


def test_act_dropout_argument_errors() -> None:
    lib = _lib.load()
    x = torch.ones(8, device='cuda')
    p, st = x.data_ptr(), _lib.stream_of(x)
    assert lib.at_act_dropout_fwd(None, p, 8, 0, 0.0, 0.0, 0, 0, st) == -1
    assert lib.at_act_dropout_fwd(p, p, 8, 99, 0.0, 0.0, 0, 0, st) == -4
    assert lib.at_act_dropout_fwd(p, p, 8, 0, 0.0, 1.5, 0, 0, st) == -2
    assert lib.at_act_dropout_fwd(p, p, 8, 0, 0.0, 0.0, 0, 7, st) == -3
    assert lib.at_act_dropout_bwd(p, None, p, 8, 4, 0.0, 0.0, 0, 0, st) == -1   # activation needs its input
    assert lib.at_act_dropout_fwd(p, p, 0, 0, 0.0, 0.0, 0, 0, st) == 0


def test_host_tensors_raise_instead_of_faulting() -> None:
    # a host pointer handed to a kernel is a memory fault; every layer checks all its tensors first
    x = torch.randn(8, 16, device='cuda', requires_grad=True)
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.Linear(16, 4, device='cpu')(x)
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.LayerNorm(16, device='cpu')(x)
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.RMSNorm(16, device='cpu')(x)
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.BatchNorm1d(16, device='cpu')(x)
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.Conv2d(16, 4, 1, device='cpu')(x.view(8, 16, 1, 1))
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.NLLLoss()(torch.log_softmax(x, dim=1), torch.zeros(8, dtype=torch.int64))
    with pytest.raises(RuntimeError, match='expected all tensors on'):
        attorch_amd.MSELoss()(x, torch.zeros(8, 16))
    y = attorch_amd.Softmax(dim=-1)(x)
    with pytest.raises(RuntimeError):                      # autograd's own device check comes first here
        torch.autograd.grad(y, x, torch.ones(8, 16))       # upstream gradient on the host
    with pytest.raises(RuntimeError, match='there is no CPU path'):
        attorch_amd.Softmax(dim=-1)(torch.zeros(2, 3))


def test_custom_bwd_restores_the_forward_autocast_state() -> None:
    """
    utils.custom_bwd must behave like torch.amp.custom_bwd(device_type='cuda'): backward sees the
    autocast state (and dtype) its forward ran in, whatever the state of the calling thread.
    """
    from torch.amp import custom_fwd
    from attorch_amd.utils import custom_bwd
    seen = []

    class Probe(torch.autograd.Function):
        @staticmethod
        @custom_fwd(device_type='cuda')
        def forward(ctx, x):
            return x * 2

        @staticmethod
        @custom_bwd
        def backward(ctx, g):
            seen.append((torch.is_autocast_enabled('cuda'), torch.get_autocast_dtype('cuda')))
            return g * 2

    x = torch.ones(3, requires_grad=True, device='cuda')
    Probe.apply(x).sum().backward()                       # no autocast anywhere
    with torch.autocast('cuda', dtype=torch.bfloat16):
        y = Probe.apply(x)
    y.sum().backward()                                    # forward under autocast, backward outside
    y = Probe.apply(x)
    with torch.autocast('cuda', dtype=torch.float16):
        y.sum().backward()                                # forward outside, backward called inside
    assert seen[0][0] is False
    assert seen[1] == (True, torch.bfloat16)
    assert seen[2][0] is False
    assert not torch.is_autocast_enabled('cuda')
