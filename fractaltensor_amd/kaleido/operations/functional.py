"""The parallel functions over FractalTensors: map, filter, dilated_map, scan,
fold, reduce.

Semantics of the reference (kaleido/frontend/operations/fractaltensor/functional/
aggregate.py:28-115, apply_to_each.py:28-180, base.py:63-109;
docs/fractaltensor_operations/parallel_functions_on_fractaltensor.md:46-203):

  map(f, xs)            [f(x) for x in xs]
  scan(f, xs, init)     s = f(s, x) for every x, all s kept; without an
                        initializer the first result is xs[0] itself
  fold / reduce         the last value of scan
  dilated_map(f, xs, d) f applied to the d interleaved subsequences xs[i::d],
                        results re-interleaved into the original order

A function returning a tuple of values yields one FractalTensor per field.
These are eager Python loops over torch payloads, on the CPU or the GPU: this
IS the reference's execution model.  On GPU operands fold, scan and map first
ask operations.dispatch whether the call is one of the hot-path programs (a
stack of LSTM layers, one layer as a scan over time, a map over samples of
either, blockwise attention); if so it runs as one fused kernel.
"""
from __future__ import annotations

from typing import Callable, List

from ..fractal_tensor import FractalTensor, Iterative
from ..tensor import Tensor
from . import dispatch
from ._base import require_iterative

__all__ = ['map', 'filter', 'dilated_map', 'scan', 'fold', 'reduce']


def _pack_field(values: List):
    v0 = values[0]
    if isinstance(v0, Tensor):
        return FractalTensor.from_tensors(*values)
    if isinstance(v0, FractalTensor):
        return FractalTensor.from_fractaltensors(*values)
    if isinstance(v0, int):
        return list(values)
    raise TypeError(f'Expected Tensor or FractalTensor, but {type(v0).__name__} is given.')


def pack_outputs(results: List):
    """List of per-item results -> FractalTensor (or a list of them, one per returned field)."""
    if not results:
        raise ValueError('nothing to pack: the input was empty.')
    r0 = results[0]
    if isinstance(r0, (Tensor, FractalTensor)):
        return _pack_field(results)
    if isinstance(r0, (tuple, list)):
        n = len(r0)
        if any(len(r) != n for r in results):
            raise RuntimeError('inconsistent behavior of calling lambda function.')
        return [_pack_field([r[i] for r in results]) for i in range(n)]
    if isinstance(r0, Iterative):
        # every item is a zip of n fields: one FractalTensor per field, a level deeper
        n = len(r0[0])
        if any(len(r[0]) != n for r in results):
            raise RuntimeError('inconsistent behavior of calling lambda function.')
        return [_pack_field([_pack_field([item[i] for item in r]) for r in results]) for i in range(n)]
    raise ValueError('Unsupported type of returned value.')


def map(func: Callable, xs, **kwargs):
    require_iterative(xs)
    routed = dispatch.try_map(func, xs, kwargs)      # blockwise attention on GPU operands: one kernel
    if routed is not NotImplemented:
        return routed
    return pack_outputs([func(x, **kwargs) for x in xs])


def filter(cond: Callable, xs, **kwargs):
    require_iterative(xs)
    kept = [x for x in xs if cond(x, **kwargs)]
    return pack_outputs(kept) if kept else None


def scan(func: Callable, xs, initializer=None, **kwargs):
    require_iterative(xs)
    routed = dispatch.try_scan(func, xs, initializer, kwargs)   # one LSTM layer over GPU sequences: one kernel
    if routed is not NotImplemented:
        return routed
    n = len(xs)
    results = []
    if initializer is None:
        if n == 0:
            raise ValueError('scan over an empty input needs an initializer.')
        state = xs[0]
        results.append(state)
        start = 1
    else:
        state = initializer
        start = 0
    for i in range(start, n):
        state = func(state, xs[i], **kwargs)
        results.append(state)
    return pack_outputs(results)


def fold(func: Callable, xs, initializer=None, **kwargs):
    require_iterative(xs)
    routed = dispatch.try_fold(func, xs, initializer, kwargs)   # a stack of LSTM layers on GPU operands: one kernel
    if routed is not NotImplemented:
        return routed
    outs = scan(func, xs, initializer, **kwargs)
    if isinstance(outs, list):
        return [o[len(o) - 1] for o in outs]
    return outs[len(outs) - 1]


def reduce(func: Callable, xs, initializer=None, **kwargs):
    return fold(func, xs, initializer, **kwargs)


def _dilate(xs: FractalTensor, dilation: int) -> FractalTensor:
    if not isinstance(xs, FractalTensor):
        raise TypeError('x should be a FractalTensor.')
    if dilation <= 0:
        raise ValueError('dilation should be greater than 0.')
    n = len(xs)
    if n <= dilation or dilation == 1:
        return FractalTensor.from_fractaltensors(xs)
    return FractalTensor.from_fractaltensors(*[xs[list(range(i, n, dilation))] for i in range(dilation)])


def _revert_dilate(groups: FractalTensor, dilation: int):
    if len(groups) == 1:
        return groups[0]
    items = []
    longest = len(groups[0])
    for i in range(longest):
        for j in range(len(groups)):
            if i < len(groups[j]):
                items.append(groups[j][i])
    return _pack_field(items)


def dilated_map(func: Callable, xs, dilation: int = 1, **kwargs):
    require_iterative(xs)
    if isinstance(dilation, Tensor):
        dilation = int(dilation.data.reshape(-1)[0].item())
    dispatch.note_dilation(dilation)
    outs = map(lambda group: func(group, **kwargs), _dilate(xs, dilation))
    if not isinstance(outs, list):
        outs = [outs]
    reverted = [_revert_dilate(o, dilation) for o in outs]
    return reverted[0] if len(reverted) == 1 else reverted
