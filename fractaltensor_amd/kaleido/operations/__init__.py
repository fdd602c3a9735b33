"""kaleido.operations: the reference's operator namespace
(kaleido/frontend/operations/__init__.py:8-18) plus `fused`, the GPU fast paths,
and `dispatch`, which routes unchanged operator programs to them."""
from . import dispatch, fused
from .access import *
from .conversion import *
from .functional import *
from .tensor_ops import *
