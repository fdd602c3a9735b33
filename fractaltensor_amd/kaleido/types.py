"""Element and container type descriptors of the kaleido frontend.

Mirrors the public names of the reference's kaleido/frontend/types.py
(Number / Int / Real / Bool, float32 / int32 / int64, TensorStorage,
FractalTensorStorage, the *_to_* conversion helpers) with the behaviour its
tests pin (kaleido/frontend/tests/test_type_equivalence.py:17-43).  float16 is
an addition: the fp16 GEMM and attention kernels need a name for it.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch


class Storage:
    """Base of all type descriptors."""

    def is_equal_type(self, other) -> bool:
        raise NotImplementedError


class Number(Storage):
    def __init__(self, byte: int, signed: int):
        if byte not in (16, 32, 64):
            raise ValueError('The byte should be 16, 32, or 64.')
        self.byte = byte
        self.signed = signed

    def is_equal_type(self, other) -> bool:
        return type(self) is type(other) and self.byte == other.byte and self.signed == other.signed

    @property
    def shape(self) -> Tuple[int, ...]:
        return (1,)

    def element_shape(self) -> Tuple[int, ...]:
        return (1,)

    def element_type(self):
        return type(self)

    def __repr__(self):
        return f"{'signed' if self.signed else 'unsigned'} {type(self).__name__}{self.byte}"


class Int(Number):
    def __init__(self, byte: int):
        super().__init__(byte, signed=1)


class Real(Number):
    def __init__(self, byte: int):
        super().__init__(byte, signed=1)

    @property
    def max(self) -> float:
        return torch.finfo(_TORCH_OF[('Real', self.byte)]).max


class Bool(Number):
    def __init__(self):
        super().__init__(byte=64, signed=0)


float16 = Real(16)
float32 = Real(32)
int32 = Int(32)
int64 = Int(64)

_TORCH_OF = {('Real', 16): torch.float16, ('Real', 32): torch.float32, ('Real', 64): torch.float64,
             ('Int', 32): torch.int32, ('Int', 64): torch.int64, ('Int', 16): torch.int16}
_INTERNAL_OF = {torch.float16: float16, torch.float32: float32, torch.int32: int32, torch.int64: int64}


def pytype_to_internal_type(x):
    if isinstance(x, bool):
        raise NotImplementedError()
    if isinstance(x, int):
        return int64
    if isinstance(x, float):
        return float32
    raise NotImplementedError()


def internal_type_to_torch_type(dtype: Number):
    key = (type(dtype).__name__, dtype.byte)
    if key not in _TORCH_OF:
        raise NotImplementedError()
    return _TORCH_OF[key]


def torch_type_to_internal_type(dtype: torch.dtype) -> Number:
    if dtype not in _INTERNAL_OF:
        raise NotImplementedError(f'no kaleido type for {dtype}')
    return _INTERNAL_OF[dtype]


def str_to_internal_type(dtype: str) -> Number:
    table = {'float': float32, 'int': int32, 'half': float16, 'float16': float16, 'float32': float32,
             'int32': int32, 'int64': int64}
    if dtype not in table:
        raise NotImplementedError()
    return table[dtype]


def normalize_device(device: Optional[str]) -> str:
    """'cpu' or 'cuda' (the reference knows exactly these two, kaleido/frontend/types.py:195-197)."""
    if device is None:
        return 'cpu'
    d = str(device)
    if d.startswith('cuda'):
        return 'cuda'
    if d == 'cpu':
        return 'cpu'
    raise ValueError(f'unknown device {device!r}')


def row_major_strides(shape: Sequence[int]) -> Tuple[int, ...]:
    strides, acc = [], 1
    for s in reversed(list(shape)):
        strides.append(acc)
        acc *= s
    return tuple(reversed(strides))


class TensorStorage(Storage):
    """Shape, element type, device and memory order of a dense tensor."""

    def __init__(self, shape, dtype: Number, device: Optional[str] = None, order: Optional[str] = None,
                 strides: Optional[Sequence[int]] = None):
        self._shape = list(shape)
        self._dtype = dtype
        self._device = normalize_device(device)
        self._order = order or 'row'
        if self._order not in ('row', 'col'):
            raise ValueError("order should be 'row' or 'col'.")
        if strides is not None:
            self._strides = tuple(strides)
        else:
            st = list(row_major_strides(self._shape))
            if self._order == 'col' and len(st) >= 2:
                # column-major in the last two dimensions
                st[-1], st[-2] = self._shape[-2], 1
            self._strides = tuple(st)

    @property
    def shape(self) -> List[int]:
        return self._shape

    @property
    def dtype(self) -> Number:
        return self._dtype

    @property
    def device(self) -> str:
        return self._device

    @property
    def strides(self) -> Tuple[int, ...]:
        return self._strides

    @property
    def ndim(self) -> int:
        return len(self._shape)

    @property
    def numel(self) -> int:
        n = 1
        for s in self._shape:
            n *= s
        return n

    def element_shape(self) -> Tuple[int, ...]:
        return tuple(self._shape)

    def element_type(self):
        return self

    def is_equal_type(self, other) -> bool:
        return (isinstance(other, TensorStorage) and self._dtype.is_equal_type(other._dtype)
                and list(self._shape) == list(other._shape))

    def __repr__(self):
        return f'Tensor[{self._shape}, {self._dtype}, {self._device}]'


class FractalTensorStorage(Storage):
    """Type of a FractalTensor: a list whose items have type `dtype` (a number,
    a tensor or another FractalTensor type)."""

    def __init__(self, dtype):
        if not isinstance(dtype, (Number, TensorStorage, FractalTensorStorage)):
            raise TypeError('dtype should be a Number, TensorStorage or FractalTensorStorage.')
        self._dtype = dtype
        self._indices = None
        self._length = -1

    @property
    def dtype(self):
        return self._dtype

    @property
    def depth(self) -> int:
        d, t = 1, self._dtype
        while isinstance(t, FractalTensorStorage):
            d += 1
            t = t._dtype
        return d

    @property
    def length(self) -> int:
        return self._length

    @property
    def indices(self):
        return self._indices

    @indices.setter
    def indices(self, value):
        def nesting(v):
            n = 0
            while isinstance(v, (list, tuple)):
                n += 1
                v = v[0] if len(v) else None
            return n

        if value is not None and nesting(value) != self.depth:
            raise ValueError(f'indices nest {nesting(value)} deep but the type has depth {self.depth}.')
        self._indices = value
        t, v = self, value
        while isinstance(t, FractalTensorStorage) and v is not None:
            t._length = len(v)
            v = v[0] if (len(v) and isinstance(v[0], (list, tuple))) else None
            t = t._dtype

    def element_type(self):
        t = self._dtype
        while isinstance(t, FractalTensorStorage):
            t = t._dtype
        return t

    def element_shape(self) -> Tuple[int, ...]:
        return tuple(self.element_type().element_shape())

    def is_equal_type(self, other) -> bool:
        return isinstance(other, FractalTensorStorage) and self._dtype.is_equal_type(other._dtype)

    def __repr__(self):
        return f'FractalTensor[{self._dtype!r}]'


class StaticListStorage(Storage):
    def __init__(self, dtype, length: int):
        self.dtype = dtype
        self.length = length
