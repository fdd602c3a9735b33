"""kaleido.Tensor: a dense tensor with a torch payload.

Same public surface as the reference's kaleido/frontend/tensor.py:29-337
(constructor arguments, properties, operator overloads, from_tensor / like /
initialize / view); the meta data is derived from the payload whenever there
is one instead of being patched after every operation.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

from .types import (Number, TensorStorage, float32, int64, internal_type_to_torch_type, normalize_device,
                    pytype_to_internal_type, row_major_strides, torch_type_to_internal_type)


class _Annotation:
    """What Tensor['512, 512', float, 'cpu'] evaluates to in a signature."""

    def __init__(self, origin, args):
        self.origin = origin
        self.args = args

    def __repr__(self):
        return f'{self.origin.__name__}[{self.args!r}]'


class Tensor:
    def __init__(self, shape: Sequence[int], dtype: Number, order: Optional[str] = None, device: Optional[str] = None,
                 strides: Optional[Sequence[int]] = None):
        self._type = TensorStorage(shape, dtype, device=device, order=order, strides=strides)
        self._payload: Optional[torch.Tensor] = None
        # (a, b): this tensor is a @ b, not formed yet.  The operator dispatch leaves an fp16 product on the GPU
        # pending so that a following `@ c` can run as one back-to-back GEMM; any other use forms it with torch.
        self._pending = None

    @property
    def _T(self) -> Optional[torch.Tensor]:
        if self._pending is not None:
            a, b = self._pending
            self._pending = None
            self._payload = torch.matmul(a, b)
        return self._payload

    @_T.setter
    def _T(self, v: Optional[torch.Tensor]):
        self._pending = None
        self._payload = v

    @staticmethod
    def pending_product(a: torch.Tensor, b: torch.Tensor) -> 'Tensor':
        """a @ b, formed on first use (of .data or anything that needs the payload).  a and b are kept by reference:
        writing into them before that use changes the product, as it would change any view."""
        t = Tensor((a.shape[0], b.shape[1]), torch_type_to_internal_type(a.dtype), device=a.device.type)
        t._pending = (a, b)
        return t

    def __class_getitem__(cls, item):
        return _Annotation(cls, item)

    # ---- meta -----------------------------------------------------------
    @property
    def shape(self) -> Tuple[int, ...]:
        if self._pending is not None:
            return (self._pending[0].shape[0], self._pending[1].shape[1])
        return tuple(self._payload.shape) if self._payload is not None else tuple(self._type.shape)

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def strides(self) -> Tuple[int, ...]:
        if self._T is not None and self._T.dim() == len(self._type.shape) and self._type._order == 'row':
            return row_major_strides(self.shape)
        return self._type.strides

    @property
    def element_type(self) -> TensorStorage:
        if self._T is not None:
            return TensorStorage(self.shape, self.dtype, device=self.device)
        return self._type

    @property
    def dtype(self) -> Number:
        ref = self._pending[0] if self._pending is not None else self._payload
        if ref is not None:
            try:
                return torch_type_to_internal_type(ref.dtype)
            except NotImplementedError:
                pass
        return self._type.dtype

    @property
    def device(self) -> str:
        ref = self._pending[0] if self._pending is not None else self._payload
        return normalize_device(ref.device.type) if ref is not None else self._type.device

    def size(self, n: int) -> int:
        return self.shape[n]

    @property
    def data(self) -> torch.Tensor:
        return self._T

    @data.setter
    def data(self, v: torch.Tensor):
        self._T = v

    def initialize(self, initializer, *args, **kwargs) -> None:
        self._T = initializer(*args, **kwargs)

    # ---- construction -----------------------------------------------------
    @staticmethod
    def from_tensor(v: torch.Tensor) -> 'Tensor':
        if not isinstance(v, torch.Tensor):
            raise TypeError('from_tensor expects a torch.Tensor.')
        t = Tensor(tuple(v.shape), torch_type_to_internal_type(v.dtype), device=v.device.type)
        t._T = v
        return t

    @staticmethod
    def like(x: 'Tensor') -> 'Tensor':
        return Tensor(x.shape, x.dtype, device=x.device)

    def view(self, shape) -> 'Tensor':
        return Tensor.from_tensor(self._T.view(*shape) if isinstance(shape, (list, tuple)) else self._T.view(shape))

    @property
    def T(self) -> 'Tensor':
        if self.ndim > 2:
            raise ValueError('T is defined for tensors of rank <= 2.')
        return Tensor.from_tensor(self._T.t() if self.ndim == 2 else self._T)

    def is_equal_shape(self, other) -> bool:
        return tuple(self.shape) == tuple(other.shape)

    def is_equal_type(self, other) -> bool:
        return isinstance(other, Tensor) and self.element_type.is_equal_type(other.element_type)

    # ---- arithmetic ---------------------------------------------------------
    def _lift(self, y):
        """Python scalars become one-element tensors on this tensor's device."""
        if isinstance(y, Tensor):
            return y
        if isinstance(y, (int, float)):
            dt = self._T.dtype if self._T is not None else internal_type_to_torch_type(pytype_to_internal_type(y))
            return Tensor.from_tensor(torch.tensor([y], dtype=dt, device=self._T.device if self._T is not None else 'cpu'))
        raise TypeError(f'unsupported operand type {type(y)}')

    def __add__(self, y):
        from . import operations as ops
        return ops.add(self, self._lift(y))

    __radd__ = __add__

    def __sub__(self, y):
        from . import operations as ops
        return ops.sub(self, self._lift(y))

    def __rsub__(self, y):
        from . import operations as ops
        return ops.sub(self._lift(y), self)

    def __mul__(self, y):
        from . import operations as ops
        y = self._lift(y)
        return ops.scale(self, y) if (y.numel == 1 and self.numel != 1) else ops.multiply(self, y)

    __rmul__ = __mul__

    def __matmul__(self, y):
        from . import operations as ops
        return ops.mm(self, y)

    def __rmatmul__(self, y):
        from . import operations as ops
        return ops.mm(y, self)

    def __truediv__(self, y):
        from . import operations as ops
        return ops.div(self, self._lift(y))

    def __rtruediv__(self, y):
        from . import operations as ops
        return ops._broadcast_div(self._lift(y), self)

    def __pow__(self, y):
        from . import operations as ops
        return ops.pow(self, float(y)) if isinstance(y, (int, float)) else ops._broadcast_pow(self, y)

    def __neg__(self):
        return Tensor.from_tensor(-self._T)

    def __mod__(self, y):
        return self._T % (y._T if isinstance(y, Tensor) else y)

    def _scalar(self):
        v = self._T.reshape(-1)[0].item()
        return v

    def __eq__(self, y):
        if isinstance(y, (int, float)):
            return self._scalar() == y
        if isinstance(y, Tensor):
            return bool(torch.equal(self._T, y._T))
        return NotImplemented

    def __ne__(self, y):
        r = self.__eq__(y)
        return r if r is NotImplemented else not r

    def __gt__(self, y):
        return self._scalar() > (y._scalar() if isinstance(y, Tensor) else y)

    def __ge__(self, y):
        return self._scalar() >= (y._scalar() if isinstance(y, Tensor) else y)

    def __lt__(self, y):
        return self._scalar() < (y._scalar() if isinstance(y, Tensor) else y)

    def __le__(self, y):
        return self._scalar() <= (y._scalar() if isinstance(y, Tensor) else y)

    __hash__ = object.__hash__

    def __str__(self):
        return f'Tensor(shape={list(self.shape)}, dtype={self.dtype}, device={self.device})'

    __repr__ = __str__


class Parameter(Tensor):
    """A learnable tensor.  The reference's Parameter.update is a stub
    (kaleido/frontend/tensor.py:336-337); so is this one: the project is forward-only."""

    def update(self, func) -> None:
        raise NotImplementedError('parameter updates are not part of the forward-only hot path')
