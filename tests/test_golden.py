"""The known answers that the reference's own tests and docstrings hold (tests/golden/reference_kats.json: data
only, with the file and lines each is taken from) against the oracle and the kaleido-compatible frontend."""
import json
import os
import random

import numpy as np
import pytest
import torch

import fractaltensor_amd.kaleido as kaleido
from fractaltensor_amd.kaleido import FractalTensor, FractalTensorStorage, Tensor, TensorStorage
from fractaltensor_amd.kaleido import operations as ops
from oracle import kaleido_oracle as ko

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'reference_kats.json')) as _f:
    KATS = json.load(_f)


def test_fixture_is_what_its_script_writes(tmp_path):
    import importlib.util
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
    spec = importlib.util.spec_from_file_location('make_reference_kats', os.path.join(here, 'make_reference_kats.py'))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    random.seed(12345)
    data = [random.randint(0, 193) for _ in range(17)]
    assert KATS['scan_add']['data'] == data
    assert all('source' in v for k, v in KATS.items() if k != '_about')


@pytest.mark.parametrize('case', KATS['dilate']['cases'], ids=lambda c: f"d{c['dilation']}")
def test_dilate_known_answers(case):
    x, d = case['x'], case['dilation']
    # the oracle's index form
    groups = ko.dilate_indices(len(x), d)
    assert [[x[i] for i in g] for g in groups] == case['expected']
    order = ko.revert_dilate_indices(groups)
    assert [groups[g][p] for g, p in order] == list(range(len(x)))
    # the frontend: dilated_map of the identity over each sub-sequence gives the sequence back in order,
    # and the sub-sequences it sees are the expected ones
    seen = []

    def body(sub):
        seen.append([int(t.data.item()) for t in sub])
        return ops.map(lambda t: t, sub)

    ys = ops.dilated_map(body, FractalTensor.from_pylist(x), dilation=d)
    assert seen == case['expected']
    assert [int(t.data.item()) for t in ys] == x


def test_scan_known_answers():
    k = KATS['scan_add']
    xs = FractalTensor.from_pylist(k['data'])
    ys = ops.scan(lambda s, x: ops.add(s, x), xs)
    assert [y.data.item() for y in ys] == k['expected']
    init = Tensor((1,), kaleido.int32)
    init.data = torch.LongTensor([k['initializer']])
    ys = ops.scan(lambda s, x: ops.add(s, x), xs, init)
    assert [y.data.item() for y in ys] == k['expected_with_initializer']
    assert ops.fold(lambda s, x: ops.add(s, x), xs, init).data.item() == k['expected_with_initializer'][-1]
    k2 = KATS['scan_two_outputs']
    xs = FractalTensor.from_pylist(k2['data'])
    init.data = torch.LongTensor([k2['initializer']])
    ys, zs = ops.scan(lambda s, x: (x, x), xs, init)
    assert [y.data.item() for y in ys] == k2['data'] == [z.data.item() for z in zs]


def test_product_known_answers():
    k = KATS['product']
    xss, yss = ops.product(FractalTensor.from_pylist(k['x']), FractalTensor.from_pylist(k['y']))
    assert len(xss) == len(k['y'])
    for i, (xs, ys) in enumerate(ops.zip(xss, yss)):
        assert [a.data.item() for a in xs] == k['x']
        assert [b.data.item() for b in ys] == [k['y'][i]] * len(k['x'])


@pytest.mark.parametrize('case', KATS['width_by_depth']['cases'], ids=lambda c: f"depth{c['depth']}")
def test_width_by_depth_known_answers(case):
    x = FractalTensor.from_pylist(case['data'])
    assert x.depth == case['depth']
    for d, w in case['widths'].items():
        assert x.width_by_depth(int(d)) == w
    with pytest.raises(ValueError):
        x.width_by_depth(case['raises'])


@pytest.mark.parametrize('case', KATS['join']['cases'], ids=lambda c: f"depth{c['depth']}")
def test_join_known_answers(case):
    rnd = random.Random(12345)

    def make(depth, length):
        elem = TensorStorage([3, 7], kaleido.float32, device='cpu')
        if depth == 1:
            ft = FractalTensor(elem)
            ft.indices = list(range(length))
        else:
            ft = FractalTensor(FractalTensorStorage(elem))
            ft.indices = [list(range(rnd.randint(5, 17))) for _ in range(length)]
        ft.initialize(torch.rand, *ft.flatten_shape)
        return ft

    a, b = make(case['depth'], case['len_x']), make(case['depth'], case['len_y'])
    c = ops.join(a, b)
    assert c.depth == case['depth'] and len(c) == case['len_x'] + case['len_y'] and c.numel == a.numel + b.numel


@pytest.mark.parametrize('cols', KATS['softmax_widths']['widths'])
def test_softmax_oracle_at_the_reference_widths(cols):
    x = np.random.default_rng(cols).standard_normal((5, cols)).astype(np.float32)
    y = ko.online_softmax_rows(x, chunk=64)
    np.testing.assert_allclose(y.sum(axis=1), 1.0, rtol=1e-12)
    np.testing.assert_allclose(y, torch.softmax(torch.tensor(x, dtype=torch.float64), dim=1).numpy(), rtol=1e-12, atol=0)
