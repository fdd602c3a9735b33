"""Tensor-level operations: element-wise arithmetic, contractions, broadcasts,
reductions, constants, data movement and reshapes.

Names and argument meaning follow the reference's
kaleido/frontend/operations/tensor/** (elementwise.py:13-31, contraction.py:15-18,
broadcast.py:13-17, reduction.py:11-18, constants.py:17-23,
data_movements.py:16-20, reshape.py:8-12).  Each is one torch call on the
payload, on whatever device the payload lives.  Two reference quirks are not
reproduced: relu and dropout returning their input untouched
(elementwise.py:230,243); relu here is max(x, 0), dropout is the identity only
for drop_rate == 0.
"""
from __future__ import annotations

import builtins
from typing import Optional, Sequence

import torch

from ..tensor import Tensor
from ..types import (float32, int32, internal_type_to_torch_type, normalize_device, str_to_internal_type)
from . import dispatch
from ._base import require_same_device, require_same_shape, require_tensor, wrap

__all__ = [
    'add', 'sub', 'multiply', 'div', 'exp', 'log', 'pow', 'sin', 'cos', 'tanh', 'sqrt', 'abs', 'sigmoid',
    'cross_entropy', 'dropout', 'relu', 'maximum', 'mm', 'outer', 'scale', '_broadcast_div', '_broadcast_pow',
    'max', 'sum', 'mean', 'dot', 'softmax', 'layer_norm', 'zeros', 'ones', 'arange', 'rand', 'full', 'cat',
    'permute', 'reshape', 'squeeze', 'unsqueeze',
]


# ---- element-wise ------------------------------------------------------------

def _binary(fn, x, y):
    require_tensor(x, 'x'); require_tensor(y, 'y')
    require_same_device(x, y)
    if x.numel != 1 and y.numel != 1 and tuple(x.shape) != tuple(y.shape):
        # a [n, 1] column against an [n, m] matrix (the running max / sum of the
        # attention program) broadcasts; anything else is a shape error
        try:
            torch.broadcast_shapes(tuple(x.shape), tuple(y.shape))
        except RuntimeError:
            require_same_shape(x, y)
    return wrap(fn(x.data, y.data))


def add(x, y): return _binary(torch.add, x, y)
def sub(x, y): return _binary(torch.sub, x, y)
def multiply(x, y): return _binary(torch.mul, x, y)
def div(x, y): return _binary(torch.div, x, y)
def maximum(x, y): return _binary(torch.maximum, x, y)


def _unary(fn, x):
    return wrap(fn(require_tensor(x, 'x').data))


def exp(x): return _unary(torch.exp, x)
def log(x): return _unary(torch.log, x)
def sin(x): return _unary(torch.sin, x)
def cos(x): return _unary(torch.cos, x)
def tanh(x): return _unary(torch.tanh, x)
def sqrt(x): return _unary(torch.sqrt, x)
def abs(x): return _unary(torch.abs, x)
def sigmoid(x): return _unary(torch.sigmoid, x)
def relu(x): return _unary(torch.relu, x)


def pow(x, y: float):
    return wrap(torch.pow(require_tensor(x, 'x').data, float(y)))


def dropout(x, drop_rate: float = 0.5):
    return wrap(torch.nn.functional.dropout(require_tensor(x, 'x').data, p=drop_rate, training=drop_rate > 0))


def cross_entropy(x, y):
    """x: scores [N, C]; y: int class ids [N]."""
    require_tensor(x, 'x'); require_tensor(y, 'y')
    return wrap(torch.nn.functional.cross_entropy(x.data, y.data.reshape(-1).long()))


# ---- contractions and broadcasts ------------------------------------------------

def mm(x, y):
    routed = dispatch.try_mm(x, y)       # fp16 GPU tensors: (a @ b) @ c as one back-to-back GEMM; a large a @ b on ftk_gemm_f16
    if routed is not NotImplemented:
        return routed
    require_tensor(x, 'x'); require_tensor(y, 'y')
    require_same_device(x, y)
    if x.ndim != 2 or y.ndim != 2 or x.shape[1] != y.shape[0]:
        raise ValueError(f'mm expects [m,k] @ [k,n], got {list(x.shape)} and {list(y.shape)}.')
    return wrap(torch.matmul(x.data, y.data))


def outer(x, y):
    require_tensor(x, 'x'); require_tensor(y, 'y')
    require_same_device(x, y)
    return wrap(torch.outer(x.data.reshape(-1), y.data.reshape(-1)))


def scale(x, y):
    """x times the one-element tensor y."""
    require_tensor(x, 'x'); require_tensor(y, 'y')
    a, b = (x, y) if y.numel == 1 else (y, x)
    if b.numel != 1:
        raise ValueError('scale expects one operand with a single element.')
    return wrap(a.data * b.data.reshape(()))


def _broadcast_div(x, y):
    require_tensor(x, 'x'); require_tensor(y, 'y')
    return wrap(x.data / y.data)


def _broadcast_pow(x, y):
    require_tensor(x, 'x'); require_tensor(y, 'y')
    return wrap(torch.pow(x.data, y.data))


# ---- reductions -------------------------------------------------------------------

def max(x, dim: int = 0, keepdim: bool = False):
    return wrap(torch.max(require_tensor(x, 'x').data, dim=dim, keepdim=keepdim).values)


def sum(x, **kwargs):
    return wrap(torch.sum(require_tensor(x, 'x').data, **kwargs))


def mean(x, **kwargs):
    return wrap(torch.mean(require_tensor(x, 'x').data, **kwargs))


def dot(x, y):
    require_tensor(x, 'x'); require_tensor(y, 'y')
    return wrap(torch.dot(x.data.reshape(-1), y.data.reshape(-1)).reshape(1))


def softmax(x, dim: int = 0):
    return wrap(torch.softmax(require_tensor(x, 'x').data, dim=dim))


def layer_norm(x, w, b, eps: float = 1e-6):
    require_tensor(x, 'x'); require_tensor(w, 'w'); require_tensor(b, 'b')
    return wrap(torch.nn.functional.layer_norm(x.data, x.data.shape[-1:], w.data.reshape(-1), b.data.reshape(-1), eps))


# ---- constants -----------------------------------------------------------------------

def _torch_dtype(dtype):
    if isinstance(dtype, str):
        dtype = str_to_internal_type(dtype)
    return internal_type_to_torch_type(dtype)


def _torch_device(device):
    return 'cuda' if normalize_device(device) == 'cuda' else 'cpu'


def zeros(shape, dtype='float', device=None):
    return wrap(torch.zeros(*shape, dtype=_torch_dtype(dtype), device=_torch_device(device)))


def ones(shape, dtype='float', device=None):
    return wrap(torch.ones(*shape, dtype=_torch_dtype(dtype), device=_torch_device(device)))


def full(shape, fill_value, dtype='float', device=None):
    return wrap(torch.full(tuple(shape), fill_value, dtype=_torch_dtype(dtype), device=_torch_device(device)))


def rand(shape, dtype='float', device=None):
    return wrap(torch.rand(*shape, dtype=_torch_dtype(dtype), device=_torch_device(device)))


def arange(*args, dtype=int32, device='cpu'):
    return wrap(torch.arange(*args, dtype=_torch_dtype(dtype), device=_torch_device(device)))


# ---- data movement and reshapes ---------------------------------------------------------

def cat(xs: Sequence[Tensor], dim: int = 0):
    xs = list(xs)
    for x in xs:
        require_tensor(x, 'xs[i]')
    return wrap(torch.cat([x.data for x in xs], dim=dim))


def permute(x, axes):
    return wrap(require_tensor(x, 'x').data.permute(*axes))


def reshape(x, shape):
    return wrap(require_tensor(x, 'x').data.reshape(*shape))


def squeeze(x, dim: Optional[int] = None):
    t = require_tensor(x, 'x').data
    return wrap(t.squeeze() if dim is None else t.squeeze(dim))


def unsqueeze(x, dim: int):
    return wrap(require_tensor(x, 'x').data.unsqueeze(dim))
