"""`import kaleido`: the package name the reference's programs use (kaleido/__init__.py:10-14).

The implementation lives in fractaltensor_amd.kaleido; this module puts it, and the
module paths the reference's examples and tests import from, under the name
`kaleido`, as the SAME module objects (one operator namespace, one dispatch cache):

    import kaleido
    from kaleido import Tensor, FractalTensor, operations as ops
    from kaleido.parser.plot import PlotProgram          # examples/stacked_rnn/stacked_rnn.py:9
    from kaleido.frontend.types import Bool, Int, Real   # kaleido/frontend/tests/test_type_equivalence.py
"""
import sys
import types

import fractaltensor_amd.kaleido as _impl

_prefix = _impl.__name__
for _name, _module in list(sys.modules.items()):
    if _name == _prefix or _name.startswith(_prefix + '.'):
        sys.modules['kaleido' + _name[len(_prefix):]] = _module


def _namespace(name: str, **members):
    m = types.ModuleType(name, f'{name}: names of the reference layout, served by fractaltensor_amd.kaleido.')
    m.__dict__.update(members)
    sys.modules[name] = m
    return m


# kaleido.frontend.{operations, fractal_tensor, tensor, types} and kaleido.parser(.plot) of the reference layout
_frontend = _namespace('kaleido.frontend', operations=_impl.operations, fractal_tensor=_impl.fractal_tensor,
                       tensor=_impl.tensor, types=_impl.types)
for _sub in ('operations', 'fractal_tensor', 'tensor', 'types'):
    sys.modules['kaleido.frontend.' + _sub] = getattr(_impl, _sub)
_plot = _namespace('kaleido.parser.plot', PlotProgram=_impl.program.PlotProgram)
_parser = _namespace('kaleido.parser', Context=_impl.program.Context, function=_impl.program.function,
                     params=_impl.program.params, plot=_plot)
_impl.frontend = _frontend
_impl.parser = _parser


# kaleido._core: the name of the reference's native binding (kaleido/__init__.py:20-26, kaleido/core/init.cc:16-22)
# is the C-ABI binding here.  It loads libftkernels.so when first touched, not when kaleido is imported, so that
# host-only programs run where the library has not been built.
class _LazyCore(types.ModuleType):
    def __getattr__(self, name):
        import fractaltensor_amd._core as core
        sys.modules['kaleido._core'] = core
        _impl._core = core
        return getattr(core, name)


_impl._core = _LazyCore('kaleido._core', 'kaleido._core: the C-ABI binding fractaltensor_amd._core, loaded on first use.')
sys.modules['kaleido._core'] = _impl._core

sys.modules['kaleido'] = _impl
