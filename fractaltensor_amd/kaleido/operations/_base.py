"""Checks shared by the operations."""
from __future__ import annotations

import torch

from ..fractal_tensor import FractalTensor, Iterative
from ..tensor import Tensor


def require_tensor(x, name='input'):
    if not isinstance(x, Tensor):
        raise TypeError(f'{name} should be a kaleido Tensor, but {type(x).__name__} is given.')
    if x.data is None:
        raise RuntimeError(f'{name} is not initialized.')
    return x


def require_same_device(*xs):
    dev = xs[0].device
    for x in xs[1:]:
        if x.device != dev:
            raise RuntimeError(f'operands live on different devices: {dev} and {x.device}.')


def require_same_shape(x, y):
    if tuple(x.shape) != tuple(y.shape):
        raise ValueError(f'operands should have the same shape, got {list(x.shape)} and {list(y.shape)}.')


def require_iterative(xs):
    if not isinstance(xs, (FractalTensor, Iterative)):
        raise TypeError('Input should either a FractalTensor or a Iterative.')
    return xs


def wrap(t: torch.Tensor) -> Tensor:
    return Tensor.from_tensor(t)
