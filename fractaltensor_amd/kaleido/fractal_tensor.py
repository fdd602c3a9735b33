"""kaleido.FractalTensor, Iterative and StaticList.

A FractalTensor is a nested, possibly ragged list of equally shaped tensors
kept in ONE flat contiguous buffer in lexicographic index order, plus a nested
index tree (kaleido/frontend/fractal_tensor.py:52-511,
docs/fractaltensor_operations/memory_layout_of_fractaltensor.md).  The public
surface follows the reference; two things are added because the fused GPU
kernels need them: `is_regular()` / `as_dense()` expose a non-ragged depth-k
FractalTensor as the dense [n1, ..., nk, *elem_shape] tensor it already is in
memory (zero copy), and `from_dense()` wraps a dense tensor the other way.
"""
from __future__ import annotations

from collections.abc import Sequence
from typing import List, Optional, Tuple, Union

import torch

from .tensor import Tensor, _Annotation
from .types import (FractalTensorStorage, Number, TensorStorage, int64, internal_type_to_torch_type,
                    normalize_device, pytype_to_internal_type, torch_type_to_internal_type)


def _count_leaves(node) -> int:
    if not isinstance(node, list):
        return 1
    if not node or not isinstance(node[0], list):
        return len(node)
    return sum(_count_leaves(c) for c in node)


def _nesting(node) -> int:
    d = 0
    while isinstance(node, list):
        d += 1
        node = node[0] if node else None
    return d


def _renumber(node):
    """Index tree with the same shape whose innermost lists count from 0."""
    if not node or not isinstance(node[0], list):
        return list(range(len(node)))
    return [_renumber(c) for c in node]


class FractalTensor(Sequence):
    def __init__(self, dtype: Union[Number, TensorStorage, FractalTensorStorage]):
        self._type = FractalTensorStorage(dtype)
        self._T: Optional[torch.Tensor] = None
        self._offsets = None  # leaf offset of every child of the root, built on demand

    def __class_getitem__(cls, item):
        return _Annotation(cls, item)

    # ---- type information ---------------------------------------------------
    @property
    def depth(self) -> int:
        return self._type.depth

    @property
    def element_type(self) -> TensorStorage:
        t = self._type.element_type()
        return t if isinstance(t, TensorStorage) else TensorStorage((1,), t, device='cpu')

    @property
    def element_shape(self) -> Tuple[int, ...]:
        return tuple(self.element_type.shape)

    @property
    def element_size(self) -> int:
        n = 1
        for s in self.element_shape:
            n *= s
        return n

    @property
    def device(self) -> str:
        if self._T is not None:
            return normalize_device(self._T.device.type)
        return self.element_type.device

    @property
    def length(self) -> int:
        return self._type.length

    @property
    def indices(self):
        return self._type.indices

    @indices.setter
    def indices(self, value: List):
        self._type.indices = value
        self._offsets = None

    @property
    def numel(self) -> int:
        """Number of leaf tensors."""
        if self.indices is None:
            raise RuntimeError('numel is data dependent. No data is given.')
        return _count_leaves(self.indices)

    @property
    def flatten_shape(self) -> Tuple[int, ...]:
        return (self.numel,) + self.element_shape

    @property
    def shape(self):
        raise ValueError('shape is undefined for a FractalTensor; see flatten_shape and element_shape.')

    @property
    def data(self) -> torch.Tensor:
        return self._T

    @data.setter
    def data(self, v: torch.Tensor):
        self._T = v.reshape(-1)

    def initialize(self, initializer, *args, **kwargs) -> None:
        self.data = initializer(*args, **kwargs)

    def is_equal_type(self, other) -> bool:
        return isinstance(other, FractalTensor) and self._type.is_equal_type(other._type)

    def width_by_depth(self, depth: int) -> List[int]:
        """How many children every sub-tree at `depth` has; the outermost level
        is depth == self.depth (or -1), the level just above the leaves is 1."""
        d = depth if depth >= 0 else self.depth + depth + 1
        if d > self.depth or d < 0:
            raise ValueError(f'depth exceed {self.depth}.')
        if d == 0:
            raise ValueError('width is not defined for depth 0.')
        if self.indices is None:
            raise RuntimeError('width_by_depth is data dependent. No data is given.')
        level = [self.indices]
        for _ in range(self.depth - d):
            level = [c for node in level for c in node]
        return [len(node) for node in level]

    # ---- dense view ---------------------------------------------------------
    def dense_shape(self) -> Optional[Tuple[int, ...]]:
        """(n1, ..., nk) when every level has a uniform width, else None."""
        if self.indices is None:
            return None
        dims = []
        for d in range(self.depth, 0, -1):
            w = self.width_by_depth(d)
            if len(set(w)) != 1:
                return None
            dims.append(w[0])
        return tuple(dims)

    def is_regular(self) -> bool:
        return self.dense_shape() is not None

    def as_dense(self) -> torch.Tensor:
        """The buffer as a dense [n1, ..., nk, *elem_shape] tensor (a view, no copy)."""
        dims = self.dense_shape()
        if dims is None:
            raise ValueError('a ragged FractalTensor has no dense view')
        if self._T is None:
            raise RuntimeError('FractalTensor is not initialized.')
        return self._T.view(*dims, *self.element_shape)

    @staticmethod
    def from_dense(t: torch.Tensor, depth: int) -> 'FractalTensor':
        """Wrap a dense tensor: its first `depth` dimensions become list levels."""
        if depth < 1 or depth >= t.dim() + 1:
            raise ValueError('depth must be between 1 and the rank of the tensor')
        t = t.contiguous()
        elem = TensorStorage(tuple(t.shape[depth:]) or (1,), torch_type_to_internal_type(t.dtype), device=t.device.type)
        typ = elem
        for _ in range(depth - 1):
            typ = FractalTensorStorage(typ)
        ft = FractalTensor(typ)

        def build(level):
            n = t.shape[level]
            if level == depth - 1:
                return list(range(n))
            return [build(level + 1) for _ in range(n)]

        ft.indices = build(0)
        ft._T = t.reshape(-1)
        return ft

    # ---- element access -------------------------------------------------------
    def _child_offsets(self) -> List[int]:
        if self._offsets is None:
            offs, acc = [0], 0
            for c in self.indices:
                acc += _count_leaves(c) if isinstance(c, list) else 1
                offs.append(acc)
            self._offsets = offs
        return self._offsets

    def index(self, idx: int):
        if self._T is None or self.indices is None:
            raise RuntimeError('FractalTensor is not initialized.')
        n = len(self.indices)
        if idx < 0:
            idx += n
        if idx < 0 or idx >= n:
            raise IndexError('FractalTensor index out of range')
        es = self.element_size
        offs = self._child_offsets()
        lo, hi = offs[idx] * es, offs[idx + 1] * es
        if self.depth == 1:
            return Tensor.from_tensor(self._T[lo:hi].view(*self.element_shape))
        child = FractalTensor(self._type.dtype.dtype)
        child.indices = _renumber(self.indices[idx])
        child._T = self._T[lo:hi]
        return child

    def first(self):
        return self.index(0)

    def last(self):
        return self.index(len(self) - 1)

    def join(self, other) -> 'FractalTensor':
        from . import operations as ops
        return ops.join(self, other)

    def _gather(self, ids) -> 'FractalTensor':
        items = [self.index(int(i)) for i in ids]
        if not items:
            raise IndexError('empty selection from a FractalTensor')
        if self.depth == 1:
            return FractalTensor.from_tensors(*items)
        return FractalTensor.from_fractaltensors(*items)

    def __getitem__(self, i):
        if isinstance(i, int):
            return self.index(i)
        if isinstance(i, slice):
            return self._gather(range(*i.indices(len(self))))
        if isinstance(i, (list, tuple)):
            return self._gather(i)
        if isinstance(i, Tensor):
            ids = i.data.reshape(-1).tolist()
            return self.index(int(ids[0])) if len(ids) == 1 else self._gather(ids)
        raise TypeError(f'unsupported index type {type(i)}')

    def __len__(self) -> int:
        if self.indices is None:
            raise RuntimeError('FractalTensor is not initialized.')
        return len(self.indices)

    def __iter__(self):
        for i in range(len(self)):
            yield self.index(i)

    def __add__(self, other: 'FractalTensor') -> 'FractalTensor':
        if not isinstance(other, FractalTensor) or other.numel != self.numel:
            raise ValueError('FractalTensors of different sizes cannot be added.')
        out = FractalTensor(self._type.dtype)
        out.indices = self.indices
        out._T = self._T + other._T
        return out

    def __str__(self):
        return f'FractalTensor(depth={self.depth}, length={self.length}, element={self.element_type!r})'

    __repr__ = __str__

    # ---- construction ---------------------------------------------------------
    @staticmethod
    def from_tensors(*xs: Tensor) -> 'FractalTensor':
        if not xs:
            raise ValueError('from_tensors needs at least one tensor')
        for x in xs:
            if not isinstance(x, Tensor):  # a ValueError, like the reference's (frontend/fractal_tensor.py:404-405)
                raise ValueError(f'Expected tensor, got {type(x).__name__}.')
            if tuple(x.shape) != tuple(xs[0].shape):
                raise ValueError('tensors in a FractalTensor must share one shape.')
        ft = FractalTensor(TensorStorage(xs[0].shape, xs[0].dtype, device=xs[0].device))
        ft.indices = list(range(len(xs)))
        ft._T = torch.stack([x.data for x in xs]).reshape(-1)
        return ft

    @staticmethod
    def from_fractaltensors(*arrays: 'FractalTensor') -> 'FractalTensor':
        if not arrays:
            raise ValueError('from_fractaltensors needs at least one FractalTensor')
        for a in arrays:
            if not isinstance(a, FractalTensor):
                raise TypeError('from_fractaltensors expects FractalTensors.')
            if not a._type.is_equal_type(arrays[0]._type):
                raise ValueError('FractalTensors to nest must have the same type.')
        ft = FractalTensor(arrays[0]._type)
        if all(a.indices is not None for a in arrays):
            ft.indices = [a.indices for a in arrays]
        if all(a._T is not None for a in arrays):
            ft._T = torch.cat([a._T for a in arrays])
        return ft

    @staticmethod
    def from_pylist(x: List, device: str = 'cpu') -> 'FractalTensor':
        """Nested Python list of ints -> FractalTensor of one-element int64 tensors."""
        if not isinstance(x, list):
            raise RuntimeError('x should be a python list.')
        depth = _nesting(x)
        probe = x
        while isinstance(probe, list):
            probe = probe[0]
        if not isinstance(probe, int):
            raise NotImplementedError()
        typ = TensorStorage((1,), pytype_to_internal_type(probe), device=device)
        for _ in range(depth - 1):
            typ = FractalTensorStorage(typ)
        ft = FractalTensor(typ)
        flat: List[int] = []

        def walk(node):
            if isinstance(node[0], list):
                return [walk(c) for c in node]
            flat.extend(node)
            return list(range(len(node)))

        ft.indices = walk(x)
        dev = 'cuda' if normalize_device(device) == 'cuda' else 'cpu'
        ft._T = torch.tensor(flat, dtype=torch.int64, device=dev)
        return ft


class Iterative(Sequence):
    """The result of zip: a sequence of per-position field lists."""

    def __init__(self, *xs):
        self._items = list(xs)
        self.sources = None   # set by zip: the sequences the items were taken from

    def __getitem__(self, i):
        return self._items[i]

    def __len__(self) -> int:
        return len(self._items)

    @property
    def length(self) -> int:
        return len(self._items)

    @staticmethod
    def make_iterative(*xs) -> 'Iterative':
        return Iterative(*xs)

    def unpack(self) -> Tuple:
        return tuple(self._items)

    def __str__(self):
        return f'Iterative(length={len(self)})'


class StaticList(Sequence):
    """Type-annotation helper (StaticList[float, '4']); carries no data path."""

    def __class_getitem__(cls, item):
        return _Annotation(cls, item)

    def __init__(self, *args, **kwargs):
        self._items = list(args)

    def __getitem__(self, i):
        return self._items[i]

    def __len__(self):
        return len(self._items)
