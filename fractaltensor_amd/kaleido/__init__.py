"""kaleido: the operator API of microsoft/FractalTensor's Python frontend
(kaleido/__init__.py:10-14), re-implemented on torch payloads, with the three
hot-path programs available as fused MI355X kernels in `operations.fused`.

    import fractaltensor_amd.kaleido as kaleido
    from fractaltensor_amd.kaleido import Tensor, FractalTensor, operations as ops
"""
from . import operations
from .fractal_tensor import FractalTensor, Iterative, StaticList
from .program import Context, PlotProgram, function, params
from .tensor import Parameter, Tensor
from .types import (Bool, FractalTensorStorage, Int, Number, Real, StaticListStorage, Storage, TensorStorage,
                    float16, float32, int32, int64, internal_type_to_torch_type, pytype_to_internal_type,
                    str_to_internal_type)
