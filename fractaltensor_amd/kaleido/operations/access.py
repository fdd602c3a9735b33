"""Access operations over FractalTensors: index, zip, enumerate, product,
last, join (kaleido/frontend/operations/fractaltensor/access.py:18-29).

The windowed access patterns of the reference (slide, window, shifted_slide,
shifted_window: access.py:246-531) serve its convolution and sparse-attention
examples, which are outside the hot path built here; they raise
NotImplementedError.
"""
from __future__ import annotations

from ..fractal_tensor import FractalTensor, Iterative
from ..tensor import Tensor
from ._base import require_iterative

__all__ = ['index', 'zip', 'enumerate', 'product', 'last', 'join', 'slide', 'window', 'shifted_slide',
           'shifted_window']


def index(a, ids):
    """a[ids] with ids an int or a one-element int Tensor."""
    require_iterative(a)
    if isinstance(ids, Tensor):
        ids = int(ids.data.reshape(-1)[0].item())
    if not isinstance(ids, int):
        raise TypeError('ids should be an int or a one-element int Tensor.')
    return a[ids]


def zip(*inputs) -> Iterative:
    """Iterative whose i-th item is the list [inputs[0][i], inputs[1][i], ...].
    A single input comes back unchanged."""
    if len(inputs) == 0:
        raise ValueError('zip needs at least one input.')
    for x in inputs:
        require_iterative(x)
    if len(inputs) == 1:
        return inputs[0]
    n = len(inputs[0])
    for x in inputs[1:]:
        if len(x) != n:
            raise ValueError('inputs to zip should have the same length.')
    return Iterative(*[[x[i] for x in inputs] for i in range(n)])


def enumerate(*inputs) -> Iterative:
    """zip with a leading position index (a one-element int64 Tensor per item)."""
    if len(inputs) == 0:
        raise ValueError('enumerate needs at least one input.')
    n = len(require_iterative(inputs[0]))
    device = inputs[0].device if isinstance(inputs[0], FractalTensor) else 'cpu'
    ids = FractalTensor.from_pylist(list(range(n)), device=device)
    return zip(ids, *inputs)


def product(xs: FractalTensor, ys: FractalTensor):
    """Cartesian product as two depth+1 FractalTensors: xss[i][j] = xs[j], yss[i][j] = ys[i]."""
    if not isinstance(xs, FractalTensor) or not isinstance(ys, FractalTensor):
        raise TypeError('product expects two FractalTensors.')
    nx, ny = len(xs), len(ys)
    xss = FractalTensor.from_fractaltensors(*[xs for _ in range(ny)])
    rows = []
    for i in range(ny):
        item = ys[i]
        rows.append(FractalTensor.from_tensors(*[item] * nx) if isinstance(item, Tensor)
                    else FractalTensor.from_fractaltensors(*[item] * nx))
    yss = FractalTensor.from_fractaltensors(*rows)
    return xss, yss


def last(x):
    require_iterative(x)
    return x[len(x) - 1]


def join(x: FractalTensor, y: FractalTensor) -> FractalTensor:
    """Concatenation of two FractalTensors of the same type along the outermost level."""
    if not isinstance(x, FractalTensor) or not isinstance(y, FractalTensor):
        raise TypeError('join expects two FractalTensors.')
    if not x.is_equal_type(y):
        raise ValueError('FractalTensors to join must have the same type.')
    import torch
    out = FractalTensor(x._type.dtype)
    if x.depth == 1:
        out.indices = list(range(len(x) + len(y)))
    else:
        out.indices = list(x.indices) + list(y.indices)
    out._T = torch.cat([x.data, y.data])
    return out


def _windowed(name):
    def op(*args, **kwargs):
        raise NotImplementedError(f'{name} belongs to the convolution / sparse-attention access patterns, '
                                  'which this build does not cover.')
    op.__name__ = name
    return op


slide = _windowed('slide')
window = _windowed('window')
shifted_slide = _windowed('shifted_slide')
shifted_window = _windowed('shifted_window')
