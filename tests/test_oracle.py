"""Pins the CPU oracle against independent statements of the same maths.

Nothing here re-types the oracle's own formula: every check is a closed form,
a library routine (torch.nn.LSTM, torch softmax / SDPA), a literal from the
reference's docstrings or tests, brute force, or an invariant.
"""
import itertools

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import kaleido_oracle as ko

RNG = np.random.default_rng(1234)


def _rand_lstm(L, T, B, H, scale=0.1, bias=True):
    xs = RNG.standard_normal((T, B, H))
    WUs = RNG.uniform(-scale, scale, (L, 2 * H, 4 * H))
    bs = RNG.uniform(-scale, scale, (L, 4 * H)) if bias else None
    return xs, WUs, bs


# ----------------------------------------------------------------- LSTM cell

def test_cell_zero_weights_closed_form():
    B, H = 3, 8
    x = RNG.standard_normal((B, H))
    hp = RNG.standard_normal((B, H))
    cp = RNG.standard_normal((B, H))
    h, c = ko.lstm_cell(x, hp, cp, np.zeros((2 * H, 4 * H)))
    # all gates 0.5, candidate tanh(0)=0
    np.testing.assert_allclose(c, 0.5 * cp, rtol=0, atol=1e-15)
    np.testing.assert_allclose(h, 0.5 * np.tanh(0.5 * cp), rtol=0, atol=1e-15)


def test_cell_saturated_gates_pick_the_right_blocks():
    """Bias drives one gate at a time: catches a wrong gate order (i,f,o,g)."""
    B, H = 2, 4
    x = np.zeros((B, H)); hp = np.zeros((B, H))
    cp = RNG.standard_normal((B, H))
    W0 = np.zeros((2 * H, 4 * H))
    big = 50.0
    # forget gate open, input gate shut: c carries, h = o * tanh(c) with o = 0.5
    b = np.zeros(4 * H); b[H:2 * H] = big; b[0:H] = -big
    h, c = ko.lstm_cell(x, hp, cp, W0, b)
    np.testing.assert_allclose(c, cp, atol=1e-12)
    np.testing.assert_allclose(h, 0.5 * np.tanh(cp), atol=1e-12)
    # input gate open, forget shut, candidate saturated to +1: c = 1
    b = np.zeros(4 * H); b[0:H] = big; b[H:2 * H] = -big; b[3 * H:] = big
    h, c = ko.lstm_cell(x, hp, cp, W0, b)
    np.testing.assert_allclose(c, np.ones((B, H)), atol=1e-12)
    # output gate open on top of that: h = tanh(1)
    b[2 * H:3 * H] = big
    h, c = ko.lstm_cell(x, hp, cp, W0, b)
    np.testing.assert_allclose(h, np.tanh(np.ones((B, H))), atol=1e-12)


def _torch_lstm_from_fused(WUs, bs, H):
    """torch.nn.LSTM carrying the same parameters (torch gate order i,f,g,o)."""
    L = len(WUs)
    net = torch.nn.LSTM(H, H, num_layers=L, bias=True).double()
    perm = np.concatenate([np.arange(0, H), np.arange(H, 2 * H), np.arange(3 * H, 4 * H), np.arange(2 * H, 3 * H)])
    with torch.no_grad():
        for l in range(L):
            W = WUs[l][:H, :][:, perm]   # [I, 4H] in torch order
            U = WUs[l][H:, :][:, perm]
            getattr(net, f'weight_ih_l{l}').copy_(torch.from_numpy(W.T.copy()))
            getattr(net, f'weight_hh_l{l}').copy_(torch.from_numpy(U.T.copy()))
            b = np.zeros(4 * H) if bs is None else bs[l][perm]
            getattr(net, f'bias_ih_l{l}').copy_(torch.from_numpy(b))
            getattr(net, f'bias_hh_l{l}').zero_()
    return net


@pytest.mark.parametrize('L,T,B,H', [(1, 5, 3, 8), (3, 7, 4, 16)])
def test_stacked_lstm_matches_torch_nn_lstm(L, T, B, H):
    xs, WUs, bs = _rand_lstm(L, T, B, H, scale=0.3)
    hsss, csss = ko.stacked_lstm(xs, WUs, bs)
    net = _torch_lstm_from_fused(WUs, bs, H)
    out, (hn, cn) = net(torch.from_numpy(xs))
    np.testing.assert_allclose(hsss[-1], out.detach().numpy(), atol=1e-12)
    np.testing.assert_allclose(hsss[:, -1], hn.detach().numpy(), atol=1e-12)
    np.testing.assert_allclose(csss[:, -1], cn.detach().numpy(), atol=1e-12)


def test_per_gate_form_equals_fused_form():
    B, H = 5, 12
    ws = [RNG.uniform(-.3, .3, (H, H)) for _ in range(4)]
    us = [RNG.uniform(-.3, .3, (H, H)) for _ in range(4)]
    bs = [RNG.uniform(-.3, .3, (1, H)) for _ in range(4)]
    x, hp, cp = (RNG.standard_normal((B, H)) for _ in range(3))
    h1, c1 = ko.lstm_cell_per_gate(x, hp, cp, ws, us, bs)
    h2, c2 = ko.lstm_cell(x, hp, cp, ko.fuse_gate_weights(ws, us), np.concatenate(bs, axis=1)[0])
    np.testing.assert_allclose(h1, h2, atol=1e-13)
    np.testing.assert_allclose(c1, c2, atol=1e-13)


# ------------------------------------------------------------------ wavefront

@pytest.mark.parametrize('L,T', list(itertools.product(range(1, 6), range(1, 7))))
def test_wavefront_covers_every_cell_once_in_dependency_order(L, T):
    seen = {}
    for s, stage in enumerate(ko.wavefront_diagonals(L, T)):
        for cell in stage:
            assert cell not in seen
            seen[cell] = s
    assert set(seen) == set(itertools.product(range(L), range(T)))
    for (l, t), s in seen.items():
        if l > 0:
            assert seen[(l - 1, t)] < s
        if t > 0:
            assert seen[(l, t - 1)] < s


def test_wavefront_order_is_bit_identical_to_layer_major():
    xs, WUs, bs = _rand_lstm(4, 6, 3, 8)
    a = ko.stacked_lstm(xs, WUs, bs, dtype=np.float32)
    b = ko.stacked_lstm_wavefront(xs, WUs, bs, dtype=np.float32)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


# -------------------------------------------------------------------- dilated

def test_dilate_docstring_examples():
    # kaleido/frontend/operations/fractaltensor/functional/apply_to_each.py:92-121
    assert ko.dilate_indices(9, 2) == [[0, 2, 4, 6, 8], [1, 3, 5, 7]]
    assert ko.dilate_indices(9, 3) == [[0, 3, 6], [1, 4, 7], [2, 5, 8]]
    assert ko.dilate_indices(9, 5) == [[0, 5], [1, 6], [2, 7], [3, 8], [4]]
    assert ko.dilate_indices(4, 1) == [[0, 1, 2, 3]]
    assert ko.dilate_indices(3, 8) == [[0, 1, 2]]
    with pytest.raises(ValueError):
        ko.dilate_indices(3, 0)


@pytest.mark.parametrize('n,d', [(9, 2), (9, 3), (9, 5), (16, 4), (7, 7), (5, 1)])
def test_revert_dilate_round_trip(n, d):
    groups = ko.dilate_indices(n, d)
    order = ko.revert_dilate_indices(groups)
    assert [groups[j][i] for (j, i) in order] == list(range(n))


def test_dilated_recurrence_equals_interleaved_scans():
    L, T, B, H = 3, 11, 2, 8
    xs, WUs, bs = _rand_lstm(L, T, B, H, scale=0.3)
    dil = [1, 2, 4]
    a = ko.stacked_lstm(xs, WUs, bs, dilations=dil)
    b = ko.dilated_lstm_interleaved(xs, WUs, bs, dilations=dil)
    np.testing.assert_allclose(a[0], b[0], atol=1e-14)
    np.testing.assert_allclose(a[1], b[1], atol=1e-14)


def test_dilation_larger_than_sequence_is_a_plain_scan():
    # apply_to_each.py:129: len(x) <= dilation returns the sequence whole
    xs, WUs, bs = _rand_lstm(1, 4, 2, 8)
    a = ko.dilated_lstm_interleaved(xs, WUs, bs, dilations=[8])
    b = ko.stacked_lstm(xs, WUs, bs)
    np.testing.assert_allclose(a[0], b[0], atol=1e-14)


# ------------------------------------------------------------------- B2B GEMM

def test_b2b_identity_and_permutation():
    M, K = 6, 4
    A = RNG.standard_normal((M, K))
    eye = np.eye(K)
    np.testing.assert_array_equal(ko.b2b_gemm(A, eye, eye), A)
    perm = np.eye(K)[[2, 0, 3, 1]]            # B[k,n] = perm  => stored [N,K] = perm.T
    D = ko.b2b_gemm(A, perm.T, eye)
    np.testing.assert_array_equal(D, A @ perm)
    # non-square, checks the [N,K] / [P,N] storage convention
    N, P = 5, 3
    Bm = RNG.standard_normal((K, N)); Cm = RNG.standard_normal((N, P))
    np.testing.assert_allclose(ko.b2b_gemm(A, Bm.T.copy(), Cm.T.copy()), (A @ Bm) @ Cm, atol=1e-13)


def test_b2b_c_oracle_matches_float64():
    G, M, N, K, P = 2, 48, 64, 32, 16
    A = (RNG.standard_normal((G, M, K)) / np.sqrt(K)).astype(np.float16)
    Bn = (RNG.standard_normal((G, N, K)) / np.sqrt(K)).astype(np.float16)
    Cp = (RNG.standard_normal((G, P, N)) / np.sqrt(N)).astype(np.float16)
    D = c_oracle.b2b_gemm(A, Bn, Cp, round_intermediate=False)
    for g in range(G):
        ref = ko.b2b_gemm(A[g], Bn[g], Cp[g])
        assert ko.max_rel_err(D[g], ref) < 1e-5
    Dr = c_oracle.b2b_gemm(A, Bn, Cp, round_intermediate=True)
    for g in range(G):
        ref = ko.b2b_gemm(A[g], Bn[g], Cp[g], round_intermediate=True, dtype=np.float32)
        assert ko.max_rel_err(Dr[g], ref) < 1e-5


def test_c_half_conversions_match_numpy():
    lib = c_oracle.lib()
    vals = np.concatenate([RNG.standard_normal(2000) * s for s in (1e-7, 1e-4, 1.0, 300.0, 7e4)]).astype(np.float32)
    for v in vals:
        assert lib.orc_float_to_half(float(v)) == int(np.float32(v).astype(np.float16).view(np.uint16))
    for bits in list(range(0, 0x7c00, 37)) + [0x8001, 0x83ff, 0xfbff, 0x7c00, 0xfc00]:
        assert lib.orc_half_to_float(bits) == float(np.uint16(bits).view(np.float16))


# ------------------------------------------------------ softmax and attention

@pytest.mark.parametrize('cols', [7, 517, 1027])   # kaleido/core/operators/tests/test_softmax.cc:77-87
def test_online_softmax_matches_torch(cols):
    x = RNG.standard_normal((5, cols)) * 4
    ref = torch.softmax(torch.from_numpy(x), dim=-1).numpy()
    for chunk in (1, 3, 64):
        y = ko.online_softmax_rows(x, chunk=chunk)
        np.testing.assert_allclose(y, ref, atol=1e-15)
        np.testing.assert_allclose(y.sum(-1), 1.0, atol=1e-12)
    yc = c_oracle.online_softmax(x.astype(np.float32))
    np.testing.assert_allclose(yc, ref, rtol=2e-5, atol=1e-7)  # fp32 running sum
    np.testing.assert_allclose(ko.softmax_rows(x), ref, atol=1e-15)


def test_md_merge_is_associative_and_matches_direct():
    x = RNG.standard_normal((3, 40)) * 5
    parts = [x[:, :7], x[:, 7:19], x[:, 19:]]
    md = [(p.max(1), np.exp(p - p.max(1, keepdims=True)).sum(1)) for p in parts]
    left = ko.md_merge(*ko.md_merge(*md[0], *md[1]), *md[2])
    right = ko.md_merge(*md[0], *ko.md_merge(*md[1], *md[2]))
    np.testing.assert_allclose(left[0], right[0]); np.testing.assert_allclose(left[1], right[1], rtol=1e-13)
    np.testing.assert_allclose(left[0], x.max(1))
    np.testing.assert_allclose(left[1], np.exp(x - x.max(1, keepdims=True)).sum(1), rtol=1e-13)


def test_attention_matches_torch_sdpa():
    B, Hd, S, D = 2, 3, 37, 16
    Q, K, V = (RNG.standard_normal((B, Hd, S, D)) for _ in range(3))
    scale = 1.0 / np.sqrt(D)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(Q), torch.from_numpy(K), torch.from_numpy(V), scale=scale).numpy()
    np.testing.assert_allclose(ko.attention(Q, K, V, scale), ref, atol=1e-12)


@pytest.mark.parametrize('bq,bkv', [(64, 64), (16, 8), (5, 7), (100, 100)])
def test_blockwise_attention_is_partition_invariant(bq, bkv):
    S, D = 50, 8
    Q, K, V = (RNG.standard_normal((S, D)) for _ in range(3))
    ref = ko.attention(Q, K, V, 0.3)
    np.testing.assert_allclose(ko.flash_attention_blockwise(Q, K, V, 0.3, bq, bkv), ref, atol=1e-12)


def test_uniform_keys_give_mean_of_values():
    S, D = 24, 8
    Q = RNG.standard_normal((S, D)); V = RNG.standard_normal((S, D))
    K = np.tile(RNG.standard_normal((1, D)), (S, 1))
    out = ko.flash_attention_blockwise(Q, K, V, 1.0, 8, 8)
    np.testing.assert_allclose(out, np.tile(V.mean(0), (S, 1)), atol=1e-12)


def test_c_flash_attention_matches_closed_form():
    BH, S, D = 3, 70, 32
    Q, K, V = ((RNG.standard_normal((BH, S, D))).astype(np.float16) for _ in range(3))
    scale = 1.0 / np.sqrt(D)
    out = c_oracle.flash_attention(Q, K, V, scale, block_kv=16)
    ref = ko.attention(Q, K, V, scale)
    assert ko.max_rel_err(out, ref) < 1e-5


# ----------------------------------------------------- C LSTM vs numpy oracle

def test_c_lstm_matches_numpy_oracle():
    L, T, B, H = 3, 6, 5, 16
    xs, WUs, bs = _rand_lstm(L, T, B, H, scale=0.3)
    for dil in (None, [1, 2, 4]):
        hc, cc = c_oracle.stacked_lstm(xs, WUs, bs, dil)
        hr, cr = ko.stacked_lstm(xs, WUs, bs, dilations=dil)
        assert ko.max_rel_err(hc, hr) < 1e-5 and ko.max_rel_err(cc, cr) < 1e-5
    x, hp, cp = (RNG.standard_normal((B, H)) for _ in range(3))
    h, c = c_oracle.lstm_cell(x, hp, cp, WUs[0], None)
    hr, cr = ko.lstm_cell(x, hp, cp, WUs[0])
    assert ko.max_rel_err(h, hr) < 1e-6 and ko.max_rel_err(c, cr) < 1e-6


# ------------------------------------------------------------ fp16-storage LSTM

def test_f16_stack_rounds_every_state_it_writes_and_reads_the_rounded_values():
    """Pins oracle.stacked_lstm_f16 without retyping it: one step is the (already pinned) float64 cell on the
    fp16 inputs, rounded once; a second step must start from the ROUNDED first state; a second layer must read
    the ROUNDED hidden sequence of the first."""
    rng = np.random.default_rng(0)
    B, H = 5, 32
    xs = rng.standard_normal((2, B, H)).astype(np.float16)
    WU = rng.uniform(-0.3, 0.3, (2, 2 * H, 4 * H)).astype(np.float16)
    bs = rng.uniform(-0.3, 0.3, (2, 4 * H))
    hs, cs = ko.stacked_lstm_f16(xs, WU, bs)
    assert hs.dtype == np.float16 and cs.dtype == np.float16 and hs.shape == (2, 2, B, H)
    z = np.zeros((B, H))
    W0, W1 = WU[0].astype(np.float64), WU[1].astype(np.float64)
    h00, c00 = ko.lstm_cell(xs[0].astype(np.float64), z, z, W0, bs[0])
    assert np.array_equal(hs[0, 0], h00.astype(np.float16)) and np.array_equal(cs[0, 0], c00.astype(np.float16))
    h01, c01 = ko.lstm_cell(xs[1].astype(np.float64), hs[0, 0].astype(np.float64), cs[0, 0].astype(np.float64), W0, bs[0])
    assert np.array_equal(hs[0, 1], h01.astype(np.float16)) and np.array_equal(cs[0, 1], c01.astype(np.float16))
    # ... and not from the unrounded one: that gives a different (if close) answer somewhere
    h01u, _ = ko.lstm_cell(xs[1].astype(np.float64), h00, c00, W0, bs[0])
    assert not np.array_equal(h01u.astype(np.float16), hs[0, 1])
    h10, c10 = ko.lstm_cell(hs[0, 0].astype(np.float64), z, z, W1, bs[1])
    assert np.array_equal(hs[1, 0], h10.astype(np.float16)) and np.array_equal(cs[1, 0], c10.astype(np.float16))


def test_f16_stack_stays_within_rounding_of_the_float64_stack():
    rng = np.random.default_rng(1)
    L, T, B, H = 3, 10, 4, 64
    xs = rng.standard_normal((T, B, H)).astype(np.float16)
    WU = rng.uniform(-1 / 8, 1 / 8, (L, 2 * H, 4 * H)).astype(np.float16)
    for dil in (None, [1, 2, 4]):
        h16, c16 = ko.stacked_lstm_f16(xs, WU, None, dil)
        h64, c64 = ko.stacked_lstm(xs.astype(np.float64), WU.astype(np.float64), None, dil)
        assert ko.max_rel_err(h16.astype(np.float64), h64) < 5e-3       # a few fp16 ulps (2^-11) accumulated
        assert ko.max_rel_err(c16.astype(np.float64), c64) < 5e-3
        assert ko.max_rel_err(h16.astype(np.float64), h64) > 1e-5       # but it does round
