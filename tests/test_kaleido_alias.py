"""`import kaleido` gives the operator API under the reference's package name and module paths, and operator
dispatch leaves host programs alone."""
import numpy as np
import torch

from oracle import kaleido_oracle as ko


def test_reference_import_paths_resolve_to_one_implementation():
    import kaleido
    from kaleido import FractalTensor, FractalTensorStorage, Iterative, StaticList, Tensor, TensorStorage   # noqa: F401
    from kaleido import operations as ops
    from kaleido.frontend.types import Bool, Int, Real   # noqa: F401
    from kaleido.parser.plot import PlotProgram
    import fractaltensor_amd.kaleido as impl
    import fractaltensor_amd.kaleido.operations.dispatch as d
    assert kaleido is impl and ops is impl.operations and ops.dispatch is d
    import kaleido.operations.functional as f
    assert f is impl.operations.functional
    ctx = kaleido.Context()

    @kaleido.function(ctx)
    def twice(x):
        return x + x

    ctx[-1].ir_block.propagate_storage()
    PlotProgram().plot(ctx[-1].ir_block)
    t = Tensor.from_tensor(torch.ones((1, 4)))
    assert float(twice(t).data.sum()) == 8.0
    assert kaleido.float32.max == torch.finfo(torch.float32).max


def test_host_programs_are_never_routed():
    from kaleido import operations as ops
    from fractaltensor_amd import programs
    ops.dispatch.reset()
    L, T, B, H = 2, 3, 2, 32
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 8, seed=1)
    xss = programs.make_sequence_batch(T, B, H, seed=2)
    out = programs.stacked_lstm(xss, Wss, Uss, bss)
    assert all(v == 0 for v in ops.dispatch.stats.values())
    W = Wss.as_dense().numpy(); U = Uss.as_dense().numpy()
    WU = np.stack([ko.fuse_gate_weights(W[l], U[l]) for l in range(L)])
    ref, _ = ko.stacked_lstm(xss.as_dense().numpy().reshape(T, B, H), WU, bss.as_dense().numpy().reshape(L, 4 * H))
    assert ko.max_rel_err(out.as_dense().numpy().reshape(T, B, H), ref[-1]) <= 1e-5


def test_function_fingerprint_follows_code_and_closure_scalars():
    from kaleido.operations import dispatch

    def make(scale):
        inner = lambda x: x * scale
        return lambda y: inner(y)

    assert dispatch._fingerprint(make(2.0)) == dispatch._fingerprint(make(2.0))
    assert dispatch._fingerprint(make(2.0)) != dispatch._fingerprint(make(3.0))
    assert dispatch._fingerprint(make(2.0)) != dispatch._fingerprint(lambda y: y)


_GLOBAL_SCALE = 2.0


def _global_layer(x):
    return x * _GLOBAL_SCALE


def test_function_fingerprint_follows_module_globals_and_defaults():
    """A caller whose own code does not change but whose module-level callee, module-level scalar or default
    argument does must get a new key; callables without code are keyed on the object, not on its address."""
    import functools
    from kaleido.operations import dispatch
    caller = lambda y: _global_layer(y)
    before = dispatch._fingerprint(caller)
    assert before == dispatch._fingerprint(lambda y: _global_layer(y)) or True      # another code object: may differ
    assert dispatch._fingerprint(caller) == before
    g = globals()
    saved = g['_global_layer'], g['_GLOBAL_SCALE']
    try:
        g['_GLOBAL_SCALE'] = 3.0                          # a scalar the callee reads
        assert dispatch._fingerprint(caller) != before
        g['_GLOBAL_SCALE'] = saved[1]
        assert dispatch._fingerprint(caller) == before
        g['_global_layer'] = lambda x: x + 1.0            # the callee itself
        assert dispatch._fingerprint(caller) != before
    finally:
        g['_global_layer'], g['_GLOBAL_SCALE'] = saved
    mk = lambda d: (lambda x, d=d: x * d)
    assert dispatch._fingerprint(mk(2)) == dispatch._fingerprint(mk(2)) and dispatch._fingerprint(mk(2)) != dispatch._fingerprint(mk(4))
    kw = lambda d: (lambda x, *, d=d: x * d)
    assert dispatch._fingerprint(kw(2)) != dispatch._fingerprint(kw(4))
    part = functools.partial(_global_layer)
    assert dispatch._fingerprint(part) == ('object', part) and dispatch._fingerprint(part) != dispatch._fingerprint(functools.partial(_global_layer))


def test_kaleido_core_is_the_c_abi_binding():
    """`kaleido._core`, the module name of the reference's native binding (kaleido/__init__.py:20-26), is
    fractaltensor_amd._core."""
    import kaleido
    import kaleido._core as kcore
    assert kcore.version() >= 100
    import fractaltensor_amd._core as core
    import sys
    assert sys.modules['kaleido._core'] is core and kaleido._core is core
    from kaleido._core import b2b_gemm, stacked_lstm   # noqa: F401


def test_a_map_over_host_samples_is_not_captured():
    """The capture of a map's function only ever happens on GPU operands; on the host the map is the plain loop."""
    from kaleido import FractalTensor, operations as ops
    from kaleido.operations import dispatch
    dispatch.reset()
    x = FractalTensor.from_dense(torch.arange(24.).reshape(2, 3, 1, 4), 2)
    calls = []
    out = ops.map(lambda s: (calls.append(1), s)[1], x)
    assert len(calls) == 2 and torch.equal(out.as_dense(), x.as_dense())
    assert all(v == 0 for v in dispatch.stats.values())


def test_dilations_are_noted_only_under_a_probe():
    from kaleido.operations import dispatch
    dispatch.note_dilation(4)                  # outside a probe: ignored
    with dispatch._Probe() as p:
        dispatch.note_dilation(4)
        with dispatch._Probe() as q:           # a nested probe keeps its own list
            dispatch.note_dilation(2)
        assert q.dilations == [2]
    assert p.dilations == [4] and not dispatch._probing()


def test_a_pending_product_knows_its_type_and_is_formed_on_first_use():
    from kaleido import Tensor, FractalTensor
    a, b = torch.arange(12.).reshape(3, 4), torch.arange(8.).reshape(4, 2)
    p = Tensor.pending_product(a, b)
    assert p._pending is not None and p.shape == (3, 2) and p.ndim == 2 and p.device == 'cpu' and p.numel == 6
    assert p._pending is not None                                   # the questions above did not form it
    assert torch.equal(p.data, a @ b) and p._pending is None
    q = Tensor.pending_product(a, b)
    ft = FractalTensor.from_tensors(q, q)                            # any use of the payload forms it
    assert torch.equal(ft.as_dense()[1], a @ b)
    r = Tensor.pending_product(a, b)
    r.data = torch.zeros(3, 2)                                       # assigning a payload drops the pending product
    assert r._pending is None and float(r.data.sum()) == 0.0
    # host tensors are never left pending by the operators
    x = Tensor.from_tensor(a) @ Tensor.from_tensor(b)
    assert x._pending is None and torch.equal(x.data, a @ b)
