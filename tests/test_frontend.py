"""The kaleido-compatible frontend on the CPU: the known answers the reference's own
frontend tests hold, restated, and the eager model programs against the oracle."""
import itertools
import operator
import random

import numpy as np
import pytest
import torch

import fractaltensor_amd.kaleido as kaleido
from fractaltensor_amd import programs
from fractaltensor_amd.kaleido import FractalTensor, Iterative, Tensor, TensorStorage, FractalTensorStorage
from fractaltensor_amd.kaleido import operations as ops
from oracle import kaleido_oracle as ko


# ---- containers (kaleido/frontend/tests/test_fractaltensor_creation.py) ----------------

@pytest.mark.parametrize('shape', [[13], [3, 7], [7, 11, 3], [3, 7, 2, 11, 5]])
def test_row_major_strides(shape):                      # :14-46
    t = Tensor(shape, kaleido.float32, device='cpu')
    n = int(np.prod(shape))
    t.initialize(torch.arange, n, dtype=torch.float32)
    t.data = t.data.view(shape)
    assert t.data.ndim == t.ndim
    rnd = random.Random(1)
    idx = [rnd.randint(0, s - 1) for s in shape]
    off = sum(i * s for i, s in zip(idx, t.strides))
    assert t.data.reshape(-1)[off] == off


def test_from_tensors_keeps_shapes():                   # :55-70
    ts = []
    for _ in range(5):
        t = Tensor([3, 7, 5], kaleido.float32, device='cpu')
        t.initialize(torch.rand, *t.shape)
        ts.append(t)
    ft = FractalTensor.from_tensors(*ts)
    assert ft.depth == 1 and len(ft) == 5
    for i, t in enumerate(ft):
        assert tuple(t.shape) == (3, 7, 5) and torch.equal(t.data, ts[i].data)


def test_constructors_reject_what_the_reference_rejects():   # frontend/fractal_tensor.py:398-405, 435-455
    with pytest.raises(ValueError):
        FractalTensor.from_tensors()                        # "input should be a non-empty list."
    with pytest.raises(ValueError):
        FractalTensor.from_tensors(3)                       # "Expected tensor, got int."
    with pytest.raises(IndexError):
        FractalTensor.from_pylist([])                       # the reference's walk deletes from an empty list


def test_nested_from_uninitialised_children():          # :72-106
    mk = lambda: FractalTensor(TensorStorage((3, 4), kaleido.float32, device='cpu', order='row'))
    x = FractalTensor.from_fractaltensors(mk(), mk(), mk())
    y = FractalTensor.from_fractaltensors(mk(), mk())
    z = FractalTensor.from_fractaltensors(x, y)
    z.indices = [[list(range(7)), list(range(11)), list(range(2))], [list(range(9)), list(range(1))]]
    assert z.depth == 3 and z.numel == 30 and z.flatten_shape == (30, 3, 4)
    z.initialize(torch.rand, *z.flatten_shape)
    assert tuple(z[0][1][10].shape) == (3, 4)
    assert torch.equal(z[1][0][0].data, z.data.view(30, 3, 4)[20])


def test_from_pylist_flat():                            # :108-116
    x = FractalTensor.from_pylist(list(range(13)))
    assert x.depth == 1
    for i in range(len(x)):
        assert x[i].data == i


def test_from_pylist_ragged_depth3():                   # :118-140
    rnd = random.Random(12345)
    data, start = [], 0
    for _ in range(rnd.randint(1, 23)):
        row = []
        for _ in range(rnd.randint(1, 23)):
            end = start + rnd.randint(1, 23)
            row.append(list(range(start, end)))
            start = end
        data.append(row)
    x = FractalTensor.from_pylist(data)
    assert x.depth == 3
    v = 0
    for i in range(len(x)):
        for j in range(len(x[i])):
            for k in range(len(x[i][j])):
                assert x[i][j][k].data[0] == v
                v += 1


def test_width_by_depth_literals():                     # :142-172
    x = FractalTensor.from_pylist([[0, 1, 2], [3, 4], [5, 6, 7, 8]])
    assert x.depth == 2
    assert x.width_by_depth(-1) == [3]
    assert x.width_by_depth(-2) == [3, 2, 4]
    with pytest.raises(ValueError):
        x.width_by_depth(-3)
    x = FractalTensor.from_pylist([[[0, 1], [2, 3, 4], [5]], [[6, 7, 8, 9]], [[10]]])
    assert x.depth == 3
    assert x.width_by_depth(-1) == [3]
    assert x.width_by_depth(-2) == [3, 1, 1]
    assert x.width_by_depth(-3) == [2, 3, 1, 4, 1]
    with pytest.raises(ValueError):
        x.width_by_depth(-4)


def test_type_equivalence():                            # tests/test_type_equivalence.py:17-43
    from fractaltensor_amd.kaleido import Real, Int, Bool
    assert not Real(64).is_equal_type(Int(32))
    assert not Real(64).is_equal_type(Real(32))
    assert not Bool().is_equal_type(Real(16))
    assert Real(64).is_equal_type(Real(64)) and Int(16).is_equal_type(Int(16))
    x = TensorStorage((2, 64), kaleido.float32, device='cpu')
    assert x.is_equal_type(x)
    assert not x.is_equal_type(TensorStorage((1, 3), kaleido.float32, 'cpu'))
    y = FractalTensorStorage(TensorStorage((2, 64), kaleido.float32, device='cpu'))
    assert y.is_equal_type(FractalTensorStorage(TensorStorage((2, 64), kaleido.float32, device='cpu')))
    assert not y.is_equal_type(FractalTensorStorage(TensorStorage((4, 7), kaleido.float32, device='cpu')))


def test_dense_view_is_zero_copy_and_ragged_has_none():
    t = torch.arange(2 * 3 * 4 * 5, dtype=torch.float32).view(2, 3, 4, 5)
    ft = FractalTensor.from_dense(t, 2)
    assert ft.depth == 2 and ft.dense_shape() == (2, 3) and ft.element_shape == (4, 5)
    assert ft.as_dense().data_ptr() == ft.data.data_ptr()
    assert torch.equal(ft[1][2].data, t[1, 2])
    ragged = FractalTensor.from_pylist([[0, 1, 2], [3, 4]])
    assert not ragged.is_regular()
    with pytest.raises(ValueError):
        ragged.as_dense()


# ---- parallel functions (operations/tests/test_aggregate.py, test_apply_to_each.py) -------

def _ints(n=17, seed=12345):
    rnd = random.Random(seed)
    data = [rnd.randint(0, 193) for _ in range(n)]
    return data, FractalTensor.from_pylist(data)


def test_scan_is_accumulate():                          # test_aggregate.py:27-47
    data, xs = _ints()
    ys = ops.scan(lambda s, x: ops.add(s, x), xs)
    assert isinstance(ys, FractalTensor) and len(ys) == len(xs)
    assert [y.data.item() for y in ys] == list(itertools.accumulate(data, operator.add))
    init = Tensor((1,), kaleido.int32)
    init.data = torch.LongTensor([5])
    ys = ops.scan(lambda s, x: ops.add(s, x), xs, init)
    expected = list(itertools.accumulate([5] + data, operator.add))
    assert [y.data.item() for y in ys] == expected[1:]
    assert ops.fold(lambda s, x: ops.add(s, x), xs, init).data.item() == expected[-1]
    assert ops.reduce(lambda s, x: ops.add(s, x), xs, init).data.item() == expected[-1]


def test_scan_with_two_outputs():                       # test_aggregate.py:49-57
    data, xs = _ints()
    init = Tensor((1,), kaleido.int32)
    init.data = torch.LongTensor([5])
    ys, zs = ops.scan(lambda s, x: (x, x), xs, init)
    for x, y, z in ops.zip(xs, ys, zs):
        assert y.data.item() == x.data.item() == z.data.item()


def test_functional_rejects_python_lists():             # test_apply_to_each.py:19-29
    for fn in (ops.map, ops.fold, ops.scan, ops.reduce, ops.filter, ops.dilated_map):
        with pytest.raises(TypeError):
            fn(lambda x: x, [1, 2, 3])


def test_nested_map_and_multiple_outputs():             # test_apply_to_each.py:31-54
    xss = FractalTensor.from_pylist([[0, 1, 2], [3, 4], [5, 6, 7, 8]])
    yss = ops.map(lambda xs: ops.map(lambda x: x, xs), xss)
    a, b = ops.map(lambda xs: ops.map(lambda x: (x, x), xs), xss)
    for i, row in enumerate(xss):
        for j, x in enumerate(row):
            assert x.data == yss[i][j].data == a[i][j].data == b[i][j].data


def test_map_over_zip():                                # test_apply_to_each.py:56-77
    xs1 = FractalTensor.from_pylist(list(range(7)))
    xs2 = FractalTensor.from_pylist(list(range(7, 14)))
    ys, zs = ops.map(lambda p: (p[0], p[1]), ops.zip(xs1, xs2))
    for y, z, x1, x2 in ops.zip(ys, zs, xs1, xs2):
        assert y.data.eq(x1.data).all() and z.data.eq(x2.data).all()


def test_map_returning_iterative():                     # test_apply_to_each.py:79-91
    xss = FractalTensor.from_pylist([[0, 1, 2], [3, 4], [5, 6, 7, 8]])

    def f(xs):
        v1, v2 = ops.map(lambda x: (x, x), xs)
        return ops.zip(v1, v2)

    yss, zss = ops.map(f, xss)
    for i, ys in enumerate(yss):
        for j, _ in enumerate(ys):
            assert yss[i][j].data.item() == zss[i][j].data.item() == xss[i][j].data.item()


def test_filter():
    xs = FractalTensor.from_pylist(list(range(10)))
    even = ops.filter(lambda x: x.data.item() % 2 == 0, xs)
    assert [e.data.item() for e in even] == [0, 2, 4, 6, 8]
    assert ops.filter(lambda x: False, xs) is None


# ---- access and conversion (test_zip.py, test_product.py, test_join.py, test_flatten.py, test_constants.py)

def test_zip_and_nested_zip():                          # test_zip.py:22-36
    xs1 = FractalTensor.from_pylist(list(range(7)))
    xs2 = FractalTensor.from_pylist(list(range(7, 14)))
    z = ops.zip(xs1, xs2)
    assert isinstance(z, Iterative)
    for a, b in z:
        assert b.data - a.data == 7
    for ab, c in ops.zip(ops.zip(xs1, xs2), xs1):
        a, b = ab
        assert b.data - a.data == 7 and b.data - c.data == 7
    assert ops.zip(xs1) is xs1
    with pytest.raises(ValueError):
        ops.zip(xs1, FractalTensor.from_pylist([1, 2]))


def test_product():                                     # test_product.py:21-29
    x = FractalTensor.from_pylist(list(range(11)))
    y = FractalTensor.from_pylist(list(range(7)))
    xss, yss = ops.product(x, y)
    assert isinstance(xss, FractalTensor) and isinstance(yss, FractalTensor)
    for i, (xs, ys) in enumerate(ops.zip(xss, yss)):
        for j, (a, b) in enumerate(ops.zip(xs, ys)):
            assert a.data.item() == j and b.data.item() == i


def _rand_ft(depth, length, rnd):
    elem = TensorStorage([3, 7], kaleido.float32, device='cpu')
    if depth == 1:
        ft = FractalTensor(elem)
        ft.indices = list(range(length))
    else:
        ft = FractalTensor(FractalTensorStorage(elem))
        ft.indices = [list(range(rnd.randint(5, 17))) for _ in range(length)]
    ft.initialize(torch.rand, *ft.flatten_shape)
    return ft


def test_join():                                        # test_join.py:36-54
    rnd = random.Random(12345)
    for depth, (n1, n2) in ((1, (19, 3)), (2, (11, 7))):
        a, b = _rand_ft(depth, n1, rnd), _rand_ft(depth, n2, rnd)
        c = ops.join(a, b)
        assert isinstance(c, FractalTensor) and c.depth == a.depth
        assert len(c) == len(a) + len(b) and c.numel == a.numel + b.numel
        assert torch.equal(c[len(a)].data if depth == 1 else c[len(a)][0].data, b[0].data if depth == 1 else b[0][0].data)


@pytest.mark.parametrize('dim', [0, 1])
def test_flatten_shapes(dim):                           # test_flatten.py:39-59
    rnd = random.Random(5)
    x = _rand_ft(2, 5, rnd)
    count = x.numel
    y = ops.flatten(x, dim)
    assert isinstance(y, Tensor)
    expect = [3, 7]
    expect[dim] *= count
    assert list(y.shape) == expect
    if dim == 0:
        assert torch.equal(y.data[3:6], x[0][1].data)


# ---- windowed access (operations/fractaltensor/access.py:246-531; no reference test holds an answer) ------

def _vals(ft):
    return [int(t.data.item()) for t in ft]


def _minus_one():
    pv = FractalTensor.from_pylist([0])[0]
    pv.data = pv.data * 0 - 1
    return pv


def test_slide_windows_and_the_tail_window():
    x = FractalTensor.from_pylist(list(range(9)))
    s = ops.slide(x, 3, 1, 1, padding=1, padding_value=_minus_one())
    assert s.depth == 2
    got = [_vals(w) for w in s]
    # padded = [-1, 0..8, -1]; nine regular windows, as torch's unfold gives them ...
    padded = torch.tensor([-1] + list(range(9)) + [-1])
    assert got[:9] == padded.unfold(0, 3, 1).tolist()
    # ... and the source's one more: from the position after the last start to the end (access.py:346)
    assert got[9] == [8, -1]
    s = ops.slide(x, 3, 2, 2, padding=0, padding_value=_minus_one())
    assert [_vals(w) for w in s] == [[0, 2, 4], [2, 4, 6], [4, 6, 8], [5, 7]]
    with pytest.raises(ValueError):
        ops.slide(x, 4, 1, 1, padding=1, padding_value=_minus_one())
    with pytest.raises(TypeError):
        ops.slide(x, 3, 1, 1, padding=1, padding_value=None)
    with pytest.raises(TypeError):
        ops.slide([1, 2, 3], 3, 1, 1, padding=1, padding_value=_minus_one())


def test_shifted_slide_wraps_as_the_source_does():
    ks = FractalTensor.from_pylist(list(range(6)))
    vs = FractalTensor.from_pylist(list(range(10, 16)))
    wk, wv = ops.shifted_slide(ops.zip(ks, vs), window_size=3)
    # interior positions: the plain centred window; right end: circular; left end: x < 0 -> x + L - 1
    # (access.py:384-390), i.e. position 0 sees item 4, not item 5
    assert [_vals(w) for w in wk] == [[4, 0, 1], [0, 1, 2], [1, 2, 3], [2, 3, 4], [3, 4, 5], [4, 5, 0]]
    assert [_vals(w) for w in wv] == [[14, 10, 11], [10, 11, 12], [11, 12, 13], [12, 13, 14], [13, 14, 15], [14, 15, 10]]
    # window 5, dilation 2 (the call of examples/sparse_attention/sparse_attention.py:51): span 9, every other item
    xs = FractalTensor.from_pylist(list(range(12)))
    w, _ = ops.shifted_slide(ops.zip(xs, xs), window_size=5, dilation=2)
    assert _vals(w[6]) == [2, 4, 6, 8, 10] and _vals(w[11]) == [7, 9, 11, 1, 3] and _vals(w[0]) == [7, 9, 0, 2, 4]
    # a FractalTensor input is walked item by item, each item slid (what the source's loop over `xs` does)
    nested = FractalTensor.from_pylist([[0, 1, 2, 3], [4, 5, 6, 7, 8]])
    per_item = ops.shifted_slide(nested, window_size=3)
    assert [_vals(win) for win in per_item[1]] == [[7, 4, 5], [4, 5, 6], [5, 6, 7], [6, 7, 8], [7, 8, 4]]
    with pytest.raises(TypeError):
        ops.shifted_slide(xs, window_size=3)
    with pytest.raises(ValueError):
        ops.shifted_slide(ops.zip(ks, vs), window_size=4)


def test_window_and_shifted_window():
    x = FractalTensor.from_pylist(list(range(9)))
    pv = _minus_one()
    assert _vals(ops.window(0, x, 3, 1, pv)) == [-1, 0, 1]
    assert _vals(ops.window(8, x, 5, 1, pv)) == [6, 7, 8, -1, -1]
    assert _vals(ops.window(4, x, 3, 2, pv)) == [2, 4, 6]
    assert _vals(ops.window(1, x, 3, 2, pv)) == [-1, 1, 3]
    for i in range(2, 7):                                   # interior: a plain slice
        assert _vals(ops.window(i, x, 5, 1, pv)) == list(range(i - 2, i + 3))
        assert _vals(ops.shifted_window(i, x, 5, 1)) == list(range(i - 2, i + 3))
    assert _vals(ops.shifted_window(0, x, 3, 1)) == [8, 0, 1]
    assert _vals(ops.shifted_window(8, x, 5, 1)) == [6, 7, 8, 0, 1]
    idx = Tensor((1,), kaleido.int32)
    idx.data = torch.LongTensor([7])
    assert _vals(ops.shifted_window(idx, x, 3, 1)) == [6, 7, 8]
    with pytest.raises(IndexError):
        ops.window(9, x, 3, 1, pv)
    with pytest.raises(TypeError):
        ops.shifted_window(0, [1, 2], 3, 1)


def test_windowed_attention_program_over_shifted_slide():
    """The windowed part of the reference's sparse attention (examples/sparse_attention/sparse_attention.py:25-38,
    51-53): every token attends to the window shifted_slide gives it; against a direct softmax(q K_w^T) V_w."""
    torch.manual_seed(3)
    S, D, W = 10, 8, 3
    mk = lambda: FractalTensor.from_tensors(*[Tensor.from_tensor(torch.randn(1, D)) for _ in range(S)])
    q, k, v = mk(), mk(), mk()
    wk, wv = ops.shifted_slide(ops.zip(k, v), window_size=W)

    def attn(x):
        qt, ks, vs = x
        return ops.softmax(qt @ ops.flatten(ks).T, dim=1) @ ops.flatten(vs)

    out = ops.map(attn, ops.zip(q, wk, wv))
    K = torch.cat([t.data for t in k]); V = torch.cat([t.data for t in v])
    for pos in range(S):
        ids = [(i + S - 1 if i < 0 else (i - S if i >= S else i)) for i in range(pos - 1, pos + 2)]
        ref = torch.softmax(q[pos].data @ K[ids].T, dim=1) @ V[ids]
        assert torch.allclose(out[pos].data, ref, atol=1e-6)


def test_eager_windowed_attention_with_random_positions_matches_oracle():
    """shifted_slide + sparse_attn over every token (examples/sparse_attention/sparse_attention.py:25-38, 51-53,
    69-71) through the frontend, against the numpy restatement; the restatement's window positions against a
    hand-worked case (S = 4, window 3: token 0 sees [2, 0, 1] -- the source's wrap lands one short of circular --
    token 3 sees [2, 3, 0]) and its arithmetic against torch on explicit index lists."""
    assert ko.window_positions(0, 4, 3, 1) == [2, 0, 1]
    assert ko.window_positions(3, 4, 3, 1) == [2, 3, 0]
    assert ko.window_positions(5, 12, 5, 2) == [1, 3, 5, 7, 9]
    assert ko.window_positions(1, 12, 5, 2) == [8, 10, 1, 3, 5]        # -3 -> 8, -1 -> 10
    torch.manual_seed(0)
    S, D, W, dl, R = 12, 8, 5, 2, 3
    mk = lambda: FractalTensor.from_dense(torch.randn(S, 1, D), 1)
    q, k, v = mk(), mk(), mk()
    ids = torch.randint(0, S, (S, 1, R))
    dense = lambda t: t.as_dense().numpy().reshape(1, S, D)
    out = programs.windowed_attention(q, k, v, W, dl, FractalTensor.from_dense(ids, 1))
    ref = ko.windowed_attention(dense(q), dense(k), dense(v), W, dl, ids.numpy().reshape(1, S, R))
    np.testing.assert_allclose(out.as_dense().numpy().reshape(S, D), ref[0], rtol=1e-5, atol=1e-6)
    out = programs.windowed_attention(q, k, v, 3)
    ref3 = ko.windowed_attention(dense(q), dense(k), dense(v), 3)
    np.testing.assert_allclose(out.as_dense().numpy().reshape(S, D), ref3[0], rtol=1e-5, atol=1e-6)
    Q, K, V = (torch.from_numpy(dense(t)[0]).double() for t in (q, k, v))
    for t in (0, 1, 6, 11):
        P = ko.window_positions(t, S, W, dl) + ids[t, 0].tolist()
        direct = torch.softmax(Q[t] @ K[P].T, dim=0) @ V[P]
        np.testing.assert_allclose(ref[0, t], direct.numpy(), rtol=1e-12)


def test_arange_slices_and_constants():                 # test_constants.py:16-34
    for args in ((11,), (5, 7), (5, 24, 3)):
        ft = ops.slices(ops.arange(*args), dim=0)
        assert isinstance(ft, FractalTensor)
        assert isinstance(ft.element_type.dtype, kaleido.Int)
        assert [x.data.item() for x in ft] == list(range(*args))
    z = ops.zeros(shape=(3, 7), dtype='float', device='cpu')
    o = ops.ones(shape=(3, 7), dtype='float', device='cpu')
    assert z.data.sum() == 0 and o.data.sum() == 21
    rows = ops.slices(Tensor.from_tensor(torch.arange(12.).view(3, 4)), dim=0)
    assert rows[1].shape == (1, 4)      # a row of a matrix stays a row vector
    rep = ops.repeat(ops.zeros(shape=(1, 8), device='cpu'), 5)
    assert rep.depth == 1 and len(rep) == 5 and rep.element_shape == (1, 8)


def test_tensor_operators():
    a = Tensor.from_tensor(torch.tensor([[1., 2.], [3., 4.]]))
    b = Tensor.from_tensor(torch.tensor([[5., 6.], [7., 8.]]))
    assert torch.equal((a + b).data, a.data + b.data)
    assert torch.equal((a - b).data, a.data - b.data)
    assert torch.equal((a * b).data, a.data * b.data)
    assert torch.equal((a @ b).data, a.data @ b.data)
    assert torch.equal((a / b).data, a.data / b.data)
    assert torch.equal((a * 2.0).data, a.data * 2)
    assert torch.equal(a.T.data, a.data.t())
    with pytest.raises(ValueError):
        ops.add(a, Tensor.from_tensor(torch.zeros(3, 3)))
    with pytest.raises(TypeError):
        ops.add(a, 3)


def test_decorators_are_pass_through():
    ctx = kaleido.Context()

    @kaleido.function(ctx)
    def f(x: Tensor['1, 4', float, 'cpu']) -> Tensor['1, 4', float, 'cpu']:
        return x + x

    out = f(Tensor.from_tensor(torch.ones(1, 4)))
    assert out.data.sum() == 8
    ctx[-1].ir_block.propagate_storage()
    kaleido.PlotProgram().plot(ctx[-1].ir_block)


# ---- eager model programs against the oracle -----------------------------------------------

def _np_params(Wss, Uss, bss):
    W = Wss.as_dense().numpy(); U = Uss.as_dense().numpy(); b = bss.as_dense().numpy()
    L, _, H, _ = W.shape
    WU = np.stack([ko.fuse_gate_weights(W[l], U[l]) for l in range(L)])
    return WU, b.reshape(L, 4 * H)


def test_eager_stacked_lstm_matches_oracle():
    L, T, B, H = 2, 4, 3, 16
    Wss, Uss, bss = programs.make_lstm_params(L, H, 0.3, seed=1)
    xss = programs.make_sequence_batch(T, B, H, seed=2)
    out = programs.stacked_lstm(xss, Wss, Uss, bss)
    assert out.depth == 2 and out.dense_shape() == (T, B)
    WU, bias = _np_params(Wss, Uss, bss)
    hs, _ = ko.stacked_lstm(xss.as_dense().numpy().reshape(T, B, H), WU, bias, dtype=np.float32)
    np.testing.assert_allclose(out.as_dense().numpy().reshape(T, B, H), hs[-1], atol=2e-6)


def test_eager_dilated_lstm_matches_oracle():
    L, T, B, H = 3, 9, 2, 8
    Wss, Uss, bss = programs.make_lstm_params(L, H, 0.3, seed=3)
    xss = programs.make_sequence_batch(T, B, H, seed=4)
    out = programs.dilated_lstm(xss, Wss, Uss, bss)
    WU, bias = _np_params(Wss, Uss, bss)
    hs, _ = ko.stacked_lstm(xss.as_dense().numpy().reshape(T, B, H), WU, bias, dilations=[1, 2, 4], dtype=np.float32)
    np.testing.assert_allclose(out.as_dense().numpy().reshape(T, B, H), hs[-1], atol=2e-6)


def test_eager_flash_attention_matches_oracle():
    B, Hd, S, blk, D = 1, 2, 32, 8, 16
    q, k, v = (programs.make_attention_input(B, Hd, S, blk, D, seed=s) for s in (5, 6, 7))
    scale = D ** -0.5
    out = programs.flash_attention(q, k, v, scale)
    assert out.depth == 3 and out.dense_shape() == (B, Hd, S // blk)
    dense = lambda ft: ft.as_dense().numpy().reshape(B, Hd, S, D)
    ref = ko.attention(dense(q), dense(k), dense(v), scale, dtype=np.float32)
    np.testing.assert_allclose(dense(out), ref, atol=2e-6)


def test_eager_grid_rnn_matches_oracle():
    """The reference's fourth model program (examples/grid_rnn/grid_rnn.py) through the frontend: nested scans
    with tuple state over zip(product(src, trg)), folded over the blocks, against the numpy statement of the
    recurrence; and a hand check of the first block's corner, which has no neighbours."""
    H, S, Tg, depth = 8, 4, 3, 2
    torch.manual_seed(11)
    mk = lambda n: FractalTensor.from_tensors(*[Tensor.from_tensor(torch.randn(1, H)) for _ in range(n)])
    src, trg = mk(S), mk(Tg)
    params = programs.make_grid_params(depth, H, seed=5)
    hx, hy = programs.grid_rnn(src, trg, params, H)
    assert hx.depth == 2 and len(hx) == Tg and len(hx[0]) == S
    np_params = [tuple(tuple(t.data.numpy() for t in cell) for cell in block) for block in params]
    s_np = np.stack([t.data.numpy()[0] for t in src]); t_np = np.stack([t.data.numpy()[0] for t in trg])
    rx, ry = ko.grid_rnn(s_np, t_np, np_params)
    for i in range(Tg):
        for j in range(S):
            np.testing.assert_allclose(hx[i][j].data.numpy()[0], rx[i, j], rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(hy[i][j].data.numpy()[0], ry[i, j], rtol=1e-5, atol=1e-6)
    # one block, corner (0, 0): no state, so h_x = tanh(src[0] @ h2h_x + b_x), h_y = tanh(trg[0] @ h2h_y + b_y)
    one = programs.make_grid_params(1, H, seed=6)
    cx, cy = ko.grid_rnn(s_np, t_np, [tuple(tuple(t.data.numpy() for t in cell) for cell in one[0])])
    (i2hx, h2hx, bx), (i2hy, h2hy, by) = one[0]
    np.testing.assert_allclose(cx[0, 0], np.tanh(s_np[0] @ h2hx.data.numpy() + bx.data.numpy()[0]), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(cy[0, 0], np.tanh(t_np[0] @ h2hy.data.numpy() + by.data.numpy()[0]), rtol=1e-5, atol=1e-6)
    # and position (1, 2) from its two neighbours
    s12 = np.concatenate([cx[0, 2], cy[1, 1]])
    np.testing.assert_allclose(cx[1, 2], np.tanh(s12 @ i2hx.data.numpy() + s_np[2] @ h2hx.data.numpy() + bx.data.numpy()[0]), rtol=1e-5, atol=1e-6)


def test_batched_grid_oracle_agrees_with_the_per_sample_one_and_with_a_path_product():
    """The array-layout oracle used for the GPU kernel, pinned two ways: (1) with crossed inputs, a bias row per
    block and one sample per batch row it is the per-sample recurrence above, sample by sample; (2) with the
    second axis of length one and Ux's lower half unused it is a plain stacked tanh RNN along the first axis,
    written here directly."""
    H, S, Tg, D, B = 8, 4, 3, 2, 3
    rng = np.random.default_rng(3)
    params = programs.make_grid_params(D, H, seed=9)
    npar = [tuple(tuple(t.data.numpy().astype(np.float64) for t in cell) for cell in block) for block in params]
    Wx = np.stack([b[0][1] for b in npar]); Ux = np.stack([b[0][0] for b in npar]); bx = np.stack([b[0][2] for b in npar])
    Wy = np.stack([b[1][1] for b in npar]); Uy = np.stack([b[1][0] for b in npar]); by = np.stack([b[1][2] for b in npar])
    src = rng.standard_normal((S, B, H)); trg = rng.standard_normal((Tg, B, H))
    hsss = ko.grid_rnn_batched(src, trg, Wx, Ux, bx, Wy, Uy, by, crossed=True)
    assert hsss.shape == (D, Tg, S, 2, B, H)
    for b in range(B):
        rx, ry = ko.grid_rnn(src[:, b], trg[:, b], npar)
        np.testing.assert_allclose(hsss[-1, :, :, 0, b], rx, rtol=1e-12, atol=1e-14)
        np.testing.assert_allclose(hsss[-1, :, :, 1, b], ry, rtol=1e-12, atol=1e-14)
    # (2) L2 = 1: state_y is always zero, so h_x(d, i) = tanh(in @ Wx + h_x(d, i-1) @ Ux[:H] + b)
    xs = rng.standard_normal((5, B, H)); ys = rng.standard_normal((1, B, H))
    bB = rng.standard_normal((D, B, H))                         # a bias row per batch row, as in the benchmark
    got = ko.grid_rnn_batched(xs, ys, Wx, Ux, bB, Wy, Uy, bB, crossed=False)
    inp = xs
    for d in range(D):
        h = np.zeros((B, H)); outs = []
        for i in range(5):
            h = np.tanh(inp[i] @ Wx[d] + h @ Ux[d][:H] + bB[d])
            outs.append(h)
        inp = np.stack(outs)
        np.testing.assert_allclose(got[d, :, 0, 0], inp, rtol=1e-12, atol=1e-14)


def test_fused_paths_refuse_cpu_inputs():
    Wss, Uss, bss = programs.make_lstm_params(1, 32, 0.1, seed=1)
    xss = programs.make_sequence_batch(2, 2, 32, seed=2)
    with pytest.raises(RuntimeError, match='GPU only'):
        ops.fused.stacked_lstm(xss, Wss, Uss, bss)
    q = programs.make_attention_input(1, 1, 64, 64, 64, seed=1)
    with pytest.raises(RuntimeError, match='GPU only'):
        ops.fused.flash_attention(q, q, q)
