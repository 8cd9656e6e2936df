"""
Activation-function strings of the fused epilogues and their AT_ACT_* ids.
"""

from typing import Optional, Tuple

ACT_IDS = {
    None: 0, 'sigmoid': 1, 'logsigmoid': 2, 'tanh': 3, 'relu': 4, 'gelu': 5, 'geluapprox': 6,
    'silu': 7, 'relu6': 8, 'hardsigmoid': 9, 'hardtanh': 10, 'hardswish': 11, 'selu': 12,
    'mish': 13, 'softplus': 14, 'softsign': 15, 'tanhshrink': 16, 'leaky_relu': 17, 'elu': 18,
    'celu': 19, 'hardshrink': 20, 'softshrink': 21,
}
PARAMETRIZED = ('leaky_relu', 'elu', 'celu', 'hardshrink', 'softshrink')


def parse_act_func(act_func: Optional[str]) -> Tuple[Optional[str], Optional[float]]:
    """
    Splits an activation string 'name' or 'name_PARAM' into (name, PARAM).
    Same rule as attorch/linear_layer.py:65-69: a string containing '_' is split at its
    last underscore and the tail is parsed as the float parameter.

    Args:
        act_func: E.g. None, 'relu', 'leaky_relu_0.01'.

    Returns:
        Name and parameter (None when the string carries none).
    """
    param = None
    if act_func is not None and '_' in act_func:
        comps = act_func.split('_')
        act_func = '_'.join(comps[:-1])
        param = float(comps[-1])
    return act_func, param


def act_id(act_func: Optional[str], param: Optional[float]) -> int:
    """
    AT_ACT_* id of a parsed activation name.

    Raises:
        RuntimeError: Unknown name, or a parametrized activation without its parameter.
    """
    if act_func not in ACT_IDS:
        raise RuntimeError(f'Activation function {act_func} is invalid. '
                           f'Options are {[k for k in ACT_IDS if k]}')
    if act_func in PARAMETRIZED and param is None:
        raise RuntimeError(f'Activation function {act_func} needs a parameter, e.g. {act_func}_0.5')
    return ACT_IDS[act_func]
