"""Writes tests/golden/reference_kats.json: the known answers that the reference's own tests and docstrings hold
for the path, as data (inputs and expected outputs), each with the file and lines it is taken from.

Nothing of the reference is imported or run: the literals below are copied from its docstrings and test
assertions, and the one random input (test_aggregate.py seeds Python's generator with 12345) is regenerated
with the same seed."""
import itertools
import json
import operator
import os
import random


def main():
    random.seed(12345)                                             # test_aggregate.py:20
    data = [random.randint(0, 193) for _ in range(17)]             # MAX = 193, N = 17 (:16-17)
    kats = {
        '_about': "Known answers that the reference's own tests and docstrings hold for the path, as data: inputs and "
                  'expected outputs. Written by tests/golden/make_reference_kats.py from the literals cited per entry; '
                  'nothing of the reference was imported or run.',
        'dilate': {
            'source': 'kaleido/frontend/operations/fractaltensor/functional/apply_to_each.py:92-121 (docstring examples of '
                      'DilatedMap._dilate)',
            'cases': [
                {'x': list(range(9)), 'dilation': 2, 'expected': [[0, 2, 4, 6, 8], [1, 3, 5, 7]]},
                {'x': list(range(9)), 'dilation': 3, 'expected': [[0, 3, 6], [1, 4, 7], [2, 5, 8]]},
                {'x': list(range(9)), 'dilation': 5, 'expected': [[0, 5], [1, 6], [2, 7], [3, 8], [4]]}]},
        'scan_add': {
            'source': 'kaleido/frontend/operations/tests/test_aggregate.py:16-47 (random.seed(12345); 17 ints in [0, 193]; '
                      'scan(add) == itertools.accumulate, also with initializer 5)',
            'data': data,
            'expected': list(itertools.accumulate(data, operator.add)),
            'initializer': 5,
            'expected_with_initializer': list(itertools.accumulate([5] + data, operator.add))[1:]},
        'scan_two_outputs': {
            'source': 'kaleido/frontend/operations/tests/test_aggregate.py:49-57 (scan(lambda s, x: (x, x), xs, init): both '
                      'outputs repeat the input)',
            'data': data, 'initializer': 5},
        'product': {
            'source': 'kaleido/frontend/operations/tests/test_product.py:16-30 (x = 0..10, y = 0..6: xss[i][j] = j, '
                      'yss[i][j] = i)',
            'x': list(range(11)), 'y': list(range(7))},
        'width_by_depth': {
            'source': 'kaleido/frontend/tests/test_fractaltensor_creation.py:142-172',
            'cases': [
                {'data': [[0, 1, 2], [3, 4], [5, 6, 7, 8]], 'depth': 2, 'widths': {'-1': [3], '-2': [3, 2, 4]}, 'raises': -3},
                {'data': [[[0, 1], [2, 3, 4], [5]], [[6, 7, 8, 9]], [[10]]], 'depth': 3,
                 'widths': {'-1': [3], '-2': [3, 1, 1], '-3': [2, 3, 1, 4, 1]}, 'raises': -4}]},
        'join': {
            'source': 'kaleido/frontend/operations/tests/test_join.py:36-54 (lengths and element counts add; depth kept)',
            'cases': [{'depth': 1, 'len_x': 19, 'len_y': 3}, {'depth': 2, 'len_x': 11, 'len_y': 7}]},
        'softmax_widths': {
            'source': 'kaleido/core/operators/tests/test_softmax.cc:77-87 (row softmax compared at widths 7, 517, 1027; rows '
                      'sum to 1)',
            'widths': [7, 517, 1027]},
    }
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'reference_kats.json'), 'w') as f:
        json.dump(kats, f, indent=1)


if __name__ == '__main__':
    main()
