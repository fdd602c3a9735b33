"""Conversions between Tensors and FractalTensors: stack, unbind, flatten,
slices, repeat, split (kaleido/frontend/operations/conversion.py:24-31)."""
from __future__ import annotations

import torch

from ..fractal_tensor import FractalTensor
from ..tensor import Tensor
from ._base import require_tensor, wrap

__all__ = ['stack', 'unbind', 'flatten', 'slices', 'repeat', 'split']


def stack(xs: FractalTensor, dim: int = 0) -> Tensor:
    """Depth-1 FractalTensor -> one Tensor with a new dimension `dim`."""
    if not isinstance(xs, FractalTensor) or xs.depth != 1:
        raise TypeError('stack expects a depth-1 FractalTensor.')
    t = xs.data.view(len(xs), *xs.element_shape)
    return wrap(t if dim == 0 else torch.movedim(t, 0, dim))


def unbind(x: Tensor, dim: int = 0) -> FractalTensor:
    return slices(x, dim)


def flatten(x: FractalTensor, dim: int = 0) -> Tensor:
    """All leaves concatenated along `dim`: a [numel * s_dim, ...] tensor (a view for dim 0)."""
    if not isinstance(x, FractalTensor):
        raise TypeError('flatten expects a FractalTensor.')
    es = x.element_shape
    if dim < 0 or dim >= len(es):
        raise ValueError('dim is out of range.')
    t = x.data.view(x.numel, *es)
    if dim == 0:
        return wrap(t.reshape(x.numel * es[0], *es[1:]))
    t = torch.movedim(t, 0, dim)  # [..., numel, s_dim, ...]
    shape = list(es)
    shape[dim] = es[dim] * x.numel
    return wrap(t.reshape(*shape))


def slices(x: Tensor, dim: int) -> FractalTensor:
    """Depth-1 FractalTensor over dimension `dim` of a Tensor.  Slices of a
    matrix keep rank 2: a row of a [n, m] tensor is a [1, m] tensor."""
    require_tensor(x, 'x')
    t = x.data
    if dim < 0:
        dim += t.dim()
    t = torch.movedim(t, dim, 0).contiguous()
    if t.dim() == 1:
        t = t.reshape(-1, 1)
    elif t.dim() == 2:
        t = t.reshape(t.shape[0], 1, t.shape[1])
    return FractalTensor.from_dense(t, 1)


def repeat(a, repeats: int) -> FractalTensor:
    """A Tensor repeated into a depth-1 FractalTensor; a FractalTensor repeated into one a level deeper."""
    if isinstance(a, Tensor):
        t = require_tensor(a, 'a').data
        return FractalTensor.from_dense(t.unsqueeze(0).repeat(repeats, *([1] * t.dim())), 1)
    if isinstance(a, FractalTensor):
        return FractalTensor.from_fractaltensors(*[a for _ in range(repeats)])
    raise TypeError('repeat expects a Tensor or a FractalTensor.')


def split(a, num: int, dim: int = -1):
    """Tensor -> depth-1 FractalTensor of `num` equal parts along `dim`;
    FractalTensor -> depth+1 FractalTensor of `num` equal runs of its items."""
    if isinstance(a, Tensor):
        parts = torch.chunk(require_tensor(a, 'a').data, num, dim=dim)
        if len(parts) != num or any(p.shape != parts[0].shape for p in parts):
            raise ValueError('the dimension does not divide into equal parts.')
        return FractalTensor.from_tensors(*[wrap(p.contiguous()) for p in parts])
    if isinstance(a, FractalTensor):
        n = len(a)
        if n % num:
            raise ValueError('the length does not divide into equal parts.')
        step = n // num
        return FractalTensor.from_fractaltensors(*[a[i * step:(i + 1) * step] for i in range(num)])
    raise TypeError('split expects a Tensor or a FractalTensor.')
