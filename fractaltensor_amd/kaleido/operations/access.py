"""Access operations over FractalTensors: index, zip, enumerate, product,
last, join and the windowed access patterns slide, window, shifted_slide,
shifted_window (kaleido/frontend/operations/fractaltensor/access.py:18-29,
246-531) that the reference's convolution and sparse-attention examples use.

The windowed patterns are restated from the reference's source; none of its
tests holds an answer for them.  slide and shifted_slide (the two its examples
call) follow the source to the letter, oddities included and named below;
window follows its documented meaning where the source cannot mean what it does.
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
    out = Iterative(*[[x[i] for x in inputs] for i in range(n)])
    out.sources = tuple(inputs)   # what was zipped: lets a fused kernel take whole operands as the views they are
    return out


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


def _window_span(window_size: int, dilation: int) -> int:
    return (window_size - 1) * (dilation - 1) + window_size


def _pick(x: FractalTensor, ids) -> FractalTensor:
    items = [x[int(i)] for i in ids]
    if not items:
        raise IndexError('empty window')
    return FractalTensor.from_tensors(*items) if isinstance(items[0], Tensor) else FractalTensor.from_fractaltensors(*items)


def _copies(value, n: int) -> FractalTensor:
    import copy
    items = [copy.deepcopy(value) for _ in range(n)]
    return FractalTensor.from_tensors(*items) if isinstance(value, Tensor) else FractalTensor.from_fractaltensors(*items)


def slide(input: FractalTensor, window_size: int, stride: int, dilation: int, padding: int = None, padding_value=None):
    """Windows of `window_size` items, `dilation` apart, every `stride` positions over the input padded on both
    sides with `padding` copies of `padding_value`; depth grows by one (access.py:276-373).

    As in the source, one more window follows the regular ones: everything from the position after the last
    window's start to the end (access.py:346), so the result is ragged in general.
    """
    if window_size % 2 == 0:
        raise ValueError('Even number of window size is not implemented yet.')
    if not isinstance(input, FractalTensor):
        raise TypeError(f'Expected FractalTensor, got {type(input).__name__}.')
    if not isinstance(padding_value, (Tensor, FractalTensor)):
        raise TypeError(f'Expected Tensor or FractalTensor, got {type(padding_value).__name__}.')
    padded = input
    if padding:
        pad = _copies(padding_value, int(padding))
        padded = join(join(pad, input), pad)
    span = _window_span(window_size, dilation)
    starts = list(range(0, len(padded) - span + 1, stride))
    if not starts:
        raise ValueError('the window does not fit the padded input')
    slides = [_pick(padded, range(p, p + span, dilation)) for p in starts]
    slides.append(_pick(padded, range(starts[-1] + 1, len(padded), dilation)))
    return FractalTensor.from_fractaltensors(*slides)


def _unzip(input):
    """An Iterative of per-position tuples (what zip returns) as one FractalTensor per field (access.py:248-273)."""
    if isinstance(input, FractalTensor):
        return input
    if not isinstance(input, Iterative):
        raise TypeError(f'Expected FractalTensor or Iterative, got {type(input).__name__}')
    if len(input) == 0:
        raise ValueError('empty Iterative')
    fields = []
    for f in range(len(input[0])):
        items = [input[j][f] for j in range(len(input))]
        if isinstance(items[0], Tensor):
            fields.append(FractalTensor.from_tensors(*items))
        elif isinstance(items[0], FractalTensor):
            fields.append(FractalTensor.from_fractaltensors(*items))
        else:
            raise TypeError('fields of the Iterative should be Tensors or FractalTensors.')
    return fields


def shifted_slide(input, window_size: int, dilation: int = 1):
    """For every position the window centred on it, wrapping around at both ends; one result per field of a
    zipped input (access.py:376-431; the call of examples/sparse_attention/sparse_attention.py:51).

    The wrap is the source's: position x >= L maps to x - L, but x < 0 maps to x + L - 1 (access.py:384-390), one
    short of the circular x + L.  A FractalTensor input is walked item by item, each item being slid (what
    iterating the source's `xs` does), so it must be of depth 2 or more.
    """
    if window_size % 2 == 0:
        raise ValueError('Even number of window size is not implemented yet.')
    half = _window_span(window_size, dilation) // 2

    def one(x: FractalTensor) -> FractalTensor:
        if not isinstance(x, FractalTensor):
            raise TypeError(f'Expected FractalTensor, got {type(x).__name__}.')
        L = len(x)
        wrap = lambda i: i + L - 1 if i < 0 else (i - L if i >= L else i)
        return FractalTensor.from_fractaltensors(
            *[_pick(x, [wrap(i) for i in range(pos - half, pos + half + 1, dilation)]) for pos in range(L)])

    return [one(x) for x in _unzip(input)]


def _as_index(index, length: int) -> int:
    if isinstance(index, Tensor):
        if index.data.numel() != 1:
            raise ValueError('index should hold one element.')
        index = int(index.data.reshape(-1)[0].item())
    if index >= length:
        raise IndexError(f'{index} exceeds length of the input.')
    return int(index)


def window(index, input: FractalTensor, window_size: int, dilation: int, padding_value=None) -> FractalTensor:
    """The items in the window centred on item `index`, positions outside the input filled with copies of
    `padding_value` (the meaning access.py:436-446 documents).

    The source does not do that: it keeps only one side's padding when both are needed and starts every interior
    window at position 0 (access.py:463-481); no caller exists in the reference.  This follows the documentation.
    """
    if not isinstance(input, FractalTensor):
        raise TypeError(f'Expected FractalTensor, got {type(input).__name__}.')
    i = _as_index(index, len(input))
    half = _window_span(window_size, dilation) // 2
    L = len(input)
    picked = []
    import copy
    for p in range(i - half, i + half + 1, dilation):
        if 0 <= p < L:
            picked.append(input[p])
        else:
            if not isinstance(padding_value, (Tensor, FractalTensor)):
                raise TypeError('the window leaves the input and no padding_value is given.')
            picked.append(copy.deepcopy(padding_value))
    return FractalTensor.from_tensors(*picked) if isinstance(picked[0], Tensor) else FractalTensor.from_fractaltensors(*picked)


def shifted_window(index, input: FractalTensor, window_size: int, dilation: int) -> FractalTensor:
    """The items in the window centred on item `index`, wrapping around circularly (access.py:492-528)."""
    if not isinstance(input, FractalTensor):
        raise TypeError(f'Expected FractalTensor, got {type(input).__name__}.')
    i = _as_index(index, len(input))
    half = _window_span(window_size, dilation) // 2
    L = len(input)
    return _pick(input, [(p + L) % L for p in range(i - half, i + half + 1, dilation)])
