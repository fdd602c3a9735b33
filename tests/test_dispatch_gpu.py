"""Operator programs, unchanged, on GPU FractalTensors: fold / scan / map route them to one fused launch.

Two sets of programs: the ones of fractaltensor_amd/programs.py, and programs written here the way the reference's
examples are written (`import kaleido`, decorated cell functions, per-gate map over zip(ws, us, bs), fold over
zip / enumerate of the stacked parameters: examples/stacked_rnn/stacked_rnn.py:12-79,
examples/dilated_rnn/dilated_rnn.py:16-41, examples/flash_attention/flash_attention.py:14-91).  Every routed result
is checked against the oracle, and against the eager loop where that is affordable."""
import numpy as np
import pytest
import torch

import kaleido
from kaleido import FractalTensor, Tensor
from kaleido import operations as ops

from fractaltensor_amd import programs
from oracle import kaleido_oracle as ko

pytestmark = pytest.mark.gpu
dispatch = ops.dispatch


@pytest.fixture(autouse=True)
def fresh_dispatch():
    before = (dispatch.enabled, dispatch.allow_half_attention)
    dispatch.reset()
    dispatch.enabled = True
    dispatch.allow_half_attention = False
    yield
    dispatch.reset()
    dispatch.enabled, dispatch.allow_half_attention = before


def _np_params(Wss, Uss, bss):
    W = Wss.as_dense().float().cpu().numpy(); U = Uss.as_dense().float().cpu().numpy(); b = bss.as_dense().float().cpu().numpy()
    L, _, H, _ = W.shape
    return np.stack([ko.fuse_gate_weights(W[l], U[l]) for l in range(L)]), b.reshape(L, 4 * H)


def _core():
    import fractaltensor_amd._core as core
    return core


# ---- programs in the reference's style ---------------------------------------------------------------------------

ctx = kaleido.Context()


@kaleido.function(ctx)
def gate_f(w, u, b, x, s):
    return x @ w + s @ u + b


@kaleido.function(ctx)
def lstm_cell(h_prev, c_prev, input, ws, us, bs):
    prev_gate = ops.map(lambda x: gate_f(*x, input, h_prev), ops.zip(ws, us, bs))
    gate = ops.map(lambda x: ops.sigmoid(x), prev_gate[:3])
    c = gate[1] * c_prev + gate[0] * ops.tanh(prev_gate[3])
    h = gate[2] * ops.tanh(c)
    return h, c


def batched_cell(hs_prev, cs_prev, xs, ws, us, bs):
    hs, cs = ops.map(lambda x: lstm_cell(*x, ws, us, bs), ops.zip(hs_prev[0:xs.length], cs_prev[0:xs.length], xs))
    return hs, cs


def lstm_layer(xss, ws, us, bs):
    hidden = xss.element_shape[-1]
    init = ops.repeat(ops.zeros(shape=(1, hidden), device=xss.device), xss[0].length)
    hss, css = ops.scan(lambda state, x: batched_cell(*state, x, ws, us, bs), xss, initializer=(init, init))
    return hss


def stacked_lstm(embs, Wss, Uss, bss):
    return ops.fold(lambda s, param: lstm_layer(s, *param), ops.zip(Wss, Uss, bss), initializer=embs)


def dilated_layer(state, itr, Ws, Us, bs):
    hidden = state.element_shape[-1]
    zeros = ops.zeros(shape=(1, hidden), device=state.device, dtype='float')
    h, _ = ops.dilated_map(lambda xs: ops.scan(lambda s, x: lstm_cell(*s, x, Ws, Us, bs), xs, initializer=(zeros, zeros)),
                           state, dilation=2 ** int(itr.data.item()))
    return h


def dilated_model(embs, Wss, Uss, bss):
    """Batch-major: every sample's sequence through the whole dilated stack."""
    itrs = ops.enumerate(Wss, Uss, bss)
    return ops.map(lambda xs: ops.fold(lambda s, x: dilated_layer(s, *x), itrs, initializer=xs), embs)


def attn_func(prev_maxes, prev_sums, prev_out, query, key, value):
    attn_weights = query @ key.T
    cur_maxes = ops.max(attn_weights, dim=-1, keepdim=True)
    exp_weights = ops.exp(attn_weights - cur_maxes)
    exp_values = exp_weights @ value
    cur_sums = ops.sum(exp_weights, dim=-1, keepdim=True)
    new_maxes = ops.maximum(cur_maxes, prev_maxes)
    renorm_prev = ops.exp(prev_maxes - new_maxes)
    renorm_cur = ops.exp(cur_maxes - new_maxes)
    new_sums = renorm_prev * prev_sums + renorm_cur * cur_sums
    o = (prev_out * prev_sums * renorm_prev + renorm_cur * exp_values) / new_sums
    return new_maxes, new_sums, o


def per_block_func(query, ks, vs):
    rows, dim = query.shape
    init_sum = ops.zeros(shape=(rows, 1), device=query.device)
    init_max = ops.full(shape=(rows, 1), fill_value=-kaleido.float32.max, device=query.device)
    init_o = ops.zeros(shape=(rows, dim), device=query.device)
    _, _, o = ops.reduce(lambda state, kvs: attn_func(*state, query, *kvs), ops.zip(ks, vs),
                         initializer=(init_max, init_sum, init_o))
    return o


def per_head_func(qs, ks, vs):
    return ops.map(lambda q: per_block_func(q, ks, vs), qs)


def flash_attention(qsss, ksss, vsss):
    return ops.map(lambda xss: ops.map(lambda xs: per_head_func(*xs), ops.zip(*xss)), ops.zip(qsss, ksss, vsss))


# ---- stacked LSTM -------------------------------------------------------------------------------------------------

def test_programs_stacked_lstm_is_routed_to_one_launch():
    core = _core()
    L, T, B, H = 3, 5, 33, 256
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 16, seed=1, device='cuda')
    xss = programs.make_sequence_batch(T, B, H, seed=2, device='cuda')
    out = programs.stacked_lstm(xss, Wss, Uss, bss)                       # cold: one probe of layer 0, then the launch
    assert dispatch.stats['stacked_lstm'] == 1 and dispatch.stats['probes'] == 1 and dispatch.stats['declined'] == 0
    assert isinstance(out, FractalTensor) and out.depth == 2 and out.dense_shape() == (T, B) and out.element_shape == (1, H)
    WU, bias = _np_params(Wss, Uss, bss)
    ref, _ = ko.stacked_lstm(xss.as_dense().cpu().numpy().reshape(T, B, H), WU, bias)
    assert ko.max_rel_err(out.as_dense().cpu().numpy().reshape(T, B, H), ref[-1]) <= 1e-4
    before = dict(core.launch_counts)
    out2 = programs.stacked_lstm(xss, Wss, Uss, bss)                      # warm: exactly one fused call, nothing else
    assert core.launch_counts['stacked_lstm'] == before['stacked_lstm'] + 1
    assert dispatch.stats['probes'] == 1 and dispatch.stats['stacked_lstm'] == 2
    assert torch.equal(out2.as_dense(), out.as_dense())


def test_reference_style_stacked_lstm_on_a_ragged_time_major_batch():
    """Sequences of lengths 6, 4, 4, 2 as the time-major batch examples/utils/data_utils.py:42-66 builds; routed with
    per-step row counts, equal to the eager loop and to the oracle run per sequence."""
    L, H = 2, 64
    lens = [6, 4, 4, 2]
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 8, seed=3, device='cuda')
    g = torch.Generator().manual_seed(4)
    seqs = [torch.randn((n, H), generator=g) for n in lens]
    steps = []
    for t in range(max(lens)):
        rows = [s[t] for s in seqs if len(s) > t]
        steps.append(FractalTensor.from_dense(torch.stack(rows).reshape(len(rows), 1, H).cuda(), 1))
    embs = FractalTensor.from_fractaltensors(*steps)
    routed = stacked_lstm(embs, Wss, Uss, bss)
    assert dispatch.stats['stacked_lstm'] == 1 and dispatch.stats['declined'] == 0
    dispatch.enabled = False
    eager = stacked_lstm(embs, Wss, Uss, bss)
    dispatch.enabled = True
    assert routed.indices == eager.indices
    assert ko.max_rel_err(routed.data.cpu().numpy(), eager.data.cpu().numpy()) <= 1e-4
    WU, bias = _np_params(Wss, Uss, bss)
    for b, s in enumerate(seqs):
        ref, _ = ko.stacked_lstm(s.numpy().reshape(len(s), 1, H), WU, bias)
        got = np.stack([routed[t][b].data.cpu().numpy().reshape(H) for t in range(len(s))])
        assert ko.max_rel_err(got, ref[-1][:, 0]) <= 1e-4


def test_fp16_stacked_lstm_program_goes_to_the_fp16_kernel():
    """A program whose tensors are all fp16 (its zero state included) is routed to the fp16-storage kernel."""
    core = _core()
    L, T, B, H = 2, 4, 8, 128
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 8, seed=5, device='cuda')
    half = lambda ft, d: FractalTensor.from_dense(ft.as_dense().half(), d)
    xss = programs.make_sequence_batch(T, B, H, seed=6, device='cuda')

    def layer_f16(seq, ws, us, bs):
        zero = ops.repeat(ops.zeros(shape=(1, H), dtype='half', device=seq.device), seq[0].length)
        hss, _ = ops.scan(lambda state, xs: programs.batched_cell(state[0], state[1], xs, ws, us, bs), seq, initializer=(zero, zero))
        return hss

    out = ops.fold(lambda seq, p: layer_f16(seq, *p), ops.zip(half(Wss, 2), half(Uss, 2), half(bss, 2)), initializer=half(xss, 2))
    assert dispatch.stats['stacked_lstm'] == 1 and core.launch_counts.get('stacked_lstm_f16', 0) >= 1
    assert out.data.dtype == torch.float16
    WU, bias = _np_params(half(Wss, 2), half(Uss, 2), half(bss, 2))
    ref, _ = ko.stacked_lstm(xss.as_dense().half().float().cpu().numpy().reshape(T, B, H), WU, bias)
    assert ko.max_rel_err(out.as_dense().float().cpu().numpy().reshape(T, B, H), ref[-1]) <= 1e-2


def test_a_fold_that_is_no_lstm_stays_eager():
    """Same operand structure, different arithmetic (the layer's output doubled): the probe sees the difference."""
    L, T, B, H = 2, 3, 2, 32
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 8, seed=7, device='cuda')
    xss = programs.make_sequence_batch(T, B, H, seed=8, device='cuda')

    def doubled(seq, p):
        hss = programs.lstm_layer(seq, p[0], p[1], p[2])
        return FractalTensor.from_dense(hss.as_dense() * 2, 2)

    out = ops.fold(doubled, ops.zip(Wss, Uss, bss), initializer=xss)
    assert dispatch.stats['declined'] == 1 and dispatch.stats['stacked_lstm'] == 0
    WU, bias = _np_params(Wss, Uss, bss)
    x = xss.as_dense().cpu().numpy().reshape(T, B, H)
    h0, _ = ko.stacked_lstm(x, WU[:1], bias[:1])
    h1, _ = ko.stacked_lstm(2 * h0[-1], WU[1:], bias[1:])
    assert ko.max_rel_err(out.as_dense().cpu().numpy().reshape(T, B, H), 2 * h1[-1]) <= 1e-4
    # the fold ran as the eager loop; the scan over time inside every layer is an LSTM layer and was routed on its own
    assert dispatch.stats['probes'] == 2 and dispatch.stats['lstm_scan'] == L
    ops.fold(doubled, ops.zip(Wss, Uss, bss), initializer=xss)          # both verdicts are remembered: no further probe
    assert dispatch.stats['probes'] == 2 and dispatch.stats['lstm_scan'] == 2 * L


# ---- dilated LSTM -------------------------------------------------------------------------------------------------

@pytest.mark.parametrize('L,T,B,H', [(3, 9, 2, 32), (4, 20, 5, 256)])
def test_programs_dilated_lstm_is_routed_with_the_dilations_it_asks_for(L, T, B, H):
    core = _core()
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 16, seed=9, device='cuda')
    xss = programs.make_sequence_batch(T, B, H, seed=10, device='cuda')
    out = programs.dilated_lstm(xss, Wss, Uss, bss)
    assert dispatch.stats['dilated_lstm'] == 1 and dispatch.stats['declined'] == 0
    WU, bias = _np_params(Wss, Uss, bss)
    ref, _ = ko.stacked_lstm(xss.as_dense().cpu().numpy().reshape(T, B, H), WU, bias, dilations=[2 ** k for k in range(L)])
    assert ko.max_rel_err(out.as_dense().cpu().numpy().reshape(T, B, H), ref[-1]) <= 1e-4
    before = core.launch_counts['stacked_lstm']
    programs.dilated_lstm(xss, Wss, Uss, bss)
    assert core.launch_counts['stacked_lstm'] == before + 1 and dispatch.stats['probes'] == 1


def test_reference_style_dilated_model_runs_the_samples_together():
    """Batch-major samples of different lengths, each folded through the dilated stack on its own
    (dilated_rnn.py:33-41).  A sample no longer than a layer's dilation is scanned in order by that layer (the one
    group _dilate then makes), so samples go down together as far as the dilations treat them alike: lengths 9 and 6
    in one ragged launch, length 3 (which the third layer's dilation of 4 leaves as one group) in another."""
    core = _core()
    L, H = 3, 32
    lens = [9, 6, 3]
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 8, seed=11, device='cuda')
    g = torch.Generator().manual_seed(12)
    seqs = [torch.randn((n, 1, H), generator=g) for n in lens]
    embs = FractalTensor.from_fractaltensors(*[FractalTensor.from_dense(s.cuda(), 1) for s in seqs])
    out = dilated_model(embs, Wss, Uss, bss)
    assert dispatch.stats['dilated_lstm'] == 2 and dispatch.stats['declined'] == 0
    assert out.depth == 2 and [len(o) for o in out.indices] == lens
    WU, bias = _np_params(Wss, Uss, bss)
    for b, s in enumerate(seqs):
        n = lens[b]
        dil = [d if n > d else 1 for d in (1, 2, 4)]
        ref, _ = ko.stacked_lstm(s.numpy().reshape(n, 1, H), WU, bias, dilations=dil)
        assert ko.max_rel_err(out[b].as_dense().cpu().numpy().reshape(n, H), ref[-1][:, 0]) <= 1e-4
    before = core.launch_counts['stacked_lstm']
    dilated_model(embs, Wss, Uss, bss)                                   # warm: two launches, no probe
    assert core.launch_counts['stacked_lstm'] == before + 2 and dispatch.stats['probes'] == 1
    dispatch.enabled = False
    eager = dilated_model(embs, Wss, Uss, bss)
    assert ko.max_rel_err(out.data.cpu().numpy(), eager.data.cpu().numpy()) <= 1e-4


def test_reference_style_dilated_model_is_one_launch_for_samples_of_one_length():
    """The program form of BASELINE configs[4] (an outer map over samples of a fold over dilated layers) at a
    reduced size: every sample in ONE launch, not one launch per sample."""
    core = _core()
    L, T, B, H = 4, 20, 37, 256
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 16, seed=13, device='cuda')
    x = torch.randn((B, T, 1, H), generator=torch.Generator().manual_seed(14))
    embs = FractalTensor.from_dense(x.cuda(), 2)
    out = dilated_model(embs, Wss, Uss, bss)
    assert dispatch.stats['dilated_lstm'] == 1 and dispatch.stats['declined'] == 0
    assert out.depth == 2 and out.dense_shape() == (B, T)
    WU, bias = _np_params(Wss, Uss, bss)
    ref, _ = ko.stacked_lstm(x.numpy().reshape(B, T, H).transpose(1, 0, 2), WU, bias, dilations=[1, 2, 4, 8])
    got = out.as_dense().cpu().numpy().reshape(B, T, H).transpose(1, 0, 2)
    assert ko.max_rel_err(got, ref[-1]) <= 1e-4
    before = dict(core.launch_counts)
    hits = dispatch.stats['weight_cache_hits']
    out2 = dilated_model(embs, Wss, Uss, bss)
    assert core.launch_counts['stacked_lstm'] == before['stacked_lstm'] + 1
    assert dispatch.stats['weight_cache_hits'] == hits + 1               # the packed weights were not built again
    assert torch.equal(out2.as_dense(), out.as_dense())


# ---- batch-major programs and single layers ---------------------------------------------------------------------------

def sample_scan(xs, ws, us, bs):
    """One sample's sequence through one layer (the batch-major form, examples/stacked_rnn/stacked_lstm1.py:40-51)."""
    z = ops.zeros(shape=(1, xs.element_shape[-1]), device=xs.device)
    hs, cs = ops.scan(lambda state, x: lstm_cell(*state, x, ws, us, bs), xs, initializer=(z, z))
    return hs, cs


def batch_major_layer(xss, Ws, Us, bs):
    hss, css = ops.map(lambda xs: sample_scan(xs, Ws, Us, bs), xss)
    return hss


def batch_major_stack(embs, Wss, Uss, bss):
    return ops.fold(lambda s, param: batch_major_layer(s, *param), ops.zip(Wss, Uss, bss), initializer=embs)


@pytest.mark.parametrize('lens', [[5] * 6, [7, 3, 5, 5, 1, 7]])
def test_batch_major_stack_is_one_launch(lens):
    """fold over layers of a map over samples of a scan over time: the probe finds that the depth-2 operand is
    [B][T], the batch is turned time-major on the device (sorted by length and padded when the lengths differ) and
    the stack runs as one launch."""
    core = _core()
    L, H = 3, 64
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 8, seed=70, device='cuda')
    g = torch.Generator().manual_seed(71)
    seqs = [torch.randn((n, 1, H), generator=g) for n in lens]
    embs = FractalTensor.from_fractaltensors(*[FractalTensor.from_dense(s.cuda(), 1) for s in seqs])
    out = batch_major_stack(embs, Wss, Uss, bss)
    assert dispatch.stats['stacked_lstm'] == 1 and dispatch.stats['declined'] == 0 and dispatch.stats['probes'] == 1
    assert out.depth == 2 and [len(o) for o in out.indices] == lens and out.element_shape == (1, H)
    WU, bias = _np_params(Wss, Uss, bss)
    for b, s in enumerate(seqs):
        ref, _ = ko.stacked_lstm(s.numpy().reshape(lens[b], 1, H), WU, bias)
        assert ko.max_rel_err(out[b].as_dense().cpu().numpy().reshape(lens[b], H), ref[-1][:, 0]) <= 1e-4
    before = core.launch_counts['stacked_lstm']
    batch_major_stack(embs, Wss, Uss, bss)
    assert core.launch_counts['stacked_lstm'] == before + 1 and dispatch.stats['probes'] == 1
    dispatch.enabled = False
    eager = batch_major_stack(embs, Wss, Uss, bss)
    assert eager.indices == out.indices
    assert ko.max_rel_err(out.data.cpu().numpy(), eager.data.cpu().numpy()) <= 1e-4


def test_batch_major_layer_on_its_own_is_one_launch():
    """A map over samples of one scan each, called without the fold around it: hs and cs of every sample from one launch."""
    core = _core()
    H, lens = 32, [4, 6, 2]
    Wss, Uss, bss = programs.make_lstm_params(1, H, 1 / 4, seed=72, device='cuda')
    g = torch.Generator().manual_seed(73)
    seqs = [torch.randn((n, 1, H), generator=g) for n in lens]
    xss = FractalTensor.from_fractaltensors(*[FractalTensor.from_dense(s.cuda(), 1) for s in seqs])
    before = core.launch_counts.get('stacked_lstm', 0)
    hss, css = ops.map(lambda xs: sample_scan(xs, Wss[0], Uss[0], bss[0]), xss)
    assert dispatch.stats['lstm_scan'] == 1 and core.launch_counts['stacked_lstm'] > before
    WU, bias = _np_params(Wss, Uss, bss)
    for b, s in enumerate(seqs):
        h, c = ko.stacked_lstm(s.numpy().reshape(lens[b], 1, H), WU, bias)
        assert ko.max_rel_err(hss[b].as_dense().cpu().numpy().reshape(lens[b], H), h[0][:, 0]) <= 1e-4
        assert ko.max_rel_err(css[b].as_dense().cpu().numpy().reshape(lens[b], H), c[0][:, 0]) <= 1e-4
    warm = core.launch_counts['stacked_lstm']
    ops.map(lambda xs: sample_scan(xs, Wss[0], Uss[0], bss[0]), xss)
    assert core.launch_counts['stacked_lstm'] == warm + 1


def test_single_layer_scan_of_config1_is_one_launch():
    """BASELINE configs[0] as its program: one layer written as a scan over time of a map over the batch
    (examples/stacked_rnn/stacked_rnn.py:54-65), called on its own, B 64, T 16, H 256."""
    core = _core()
    T, B, H = 16, 64, 256
    Wss, Uss, bss = programs.make_lstm_params(1, H, 0.1, seed=1234, device='cuda', bias=False)
    xss = programs.make_sequence_batch(T, B, H, seed=1234, device='cuda')
    hss = lstm_layer(xss, Wss[0], Uss[0], bss[0])
    assert dispatch.stats['lstm_scan'] == 1 and dispatch.stats['probes'] == 1 and dispatch.stats['declined'] == 0
    assert hss.depth == 2 and hss.dense_shape() == (T, B) and hss.element_shape == (1, H)
    WU, bias = _np_params(Wss, Uss, bss)
    ref, _ = ko.stacked_lstm(xss.as_dense().cpu().numpy().reshape(T, B, H), WU, bias)
    assert ko.max_rel_err(hss.as_dense().cpu().numpy().reshape(T, B, H), ref[0]) <= 1e-4
    before = dict(core.launch_counts)
    lstm_layer(xss, Wss[0], Uss[0], bss[0])
    assert core.launch_counts['stacked_lstm'] == before['stacked_lstm'] + 1 and dispatch.stats['probes'] == 1


def test_scan_returns_both_states_and_takes_ragged_steps_and_a_given_state():
    H = 64
    Wss, Uss, bss = programs.make_lstm_params(1, H, 1 / 8, seed=74, device='cuda')
    ws, us, bs = Wss[0], Uss[0], bss[0]
    WU, bias = _np_params(Wss, Uss, bss)
    step = lambda state, x: batched_cell(*state, x, ws, us, bs)
    # ragged time-major steps (4, 4, 2, 1 rows)
    g = torch.Generator().manual_seed(75)
    sizes = [4, 4, 2, 1]
    steps = [torch.randn((n, 1, H), generator=g) for n in sizes]
    xss = FractalTensor.from_fractaltensors(*[FractalTensor.from_dense(t.cuda(), 1) for t in steps])
    zero = ops.repeat(ops.zeros(shape=(1, H), device='cuda'), sizes[0])
    hss, css = ops.scan(step, xss, initializer=(zero, zero))
    assert dispatch.stats['lstm_scan'] == 1 and [len(o) for o in hss.indices] == sizes
    for b in range(sizes[0]):
        n = sum(1 for v in sizes if v > b)
        x = np.stack([steps[t][b, 0].numpy() for t in range(n)]).reshape(n, 1, H)
        h, c = ko.stacked_lstm(x, WU, bias)
        got_h = np.stack([hss[t][b].data.cpu().numpy().reshape(H) for t in range(n)])
        got_c = np.stack([css[t][b].data.cpu().numpy().reshape(H) for t in range(n)])
        assert ko.max_rel_err(got_h, h[0][:, 0]) <= 1e-4 and ko.max_rel_err(got_c, c[0][:, 0]) <= 1e-4
    # a layer that goes on from a given state: equal to the eager loop
    T, B = 5, 3
    xs2 = programs.make_sequence_batch(T, B, H, seed=76, device='cuda')
    h0 = FractalTensor.from_dense((torch.rand((B, 1, H), generator=g) - 0.5).cuda(), 1)
    c0 = FractalTensor.from_dense((torch.rand((B, 1, H), generator=g) - 0.5).cuda(), 1)
    routed = ops.scan(step, xs2, initializer=(h0, c0))
    assert dispatch.stats['lstm_scan'] == 2
    dispatch.enabled = False
    eager = ops.scan(step, xs2, initializer=(h0, c0))
    for r, e in zip(routed, eager):
        assert ko.max_rel_err(r.as_dense().cpu().numpy(), e.as_dense().cpu().numpy()) <= 1e-4


def test_a_scan_that_is_no_lstm_cell_stays_eager():
    H, T, B = 32, 3, 2
    Wss, Uss, bss = programs.make_lstm_params(1, H, 1 / 8, seed=77, device='cuda')
    ws, us, bs = Wss[0], Uss[0], bss[0]
    xss = programs.make_sequence_batch(T, B, H, seed=78, device='cuda')
    zero = ops.repeat(ops.zeros(shape=(1, H), device='cuda'), B)

    def clipped(state, x):          # the cell state clipped to +-0.05: same operands, other arithmetic
        hs, cs = batched_cell(*state, x, ws, us, bs)
        return hs, FractalTensor.from_dense(cs.as_dense().clamp(-0.05, 0.05), 1)

    hss, css = ops.scan(clipped, xss, initializer=(zero, zero))
    assert dispatch.stats['declined'] == 1 and dispatch.stats['lstm_scan'] == 0
    assert float(css.as_dense().abs().max()) <= 0.05 + 1e-7


def test_weights_changed_in_place_are_packed_again():
    L, T, B, H = 2, 4, 3, 32
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 4, seed=79, device='cuda')
    xss = programs.make_sequence_batch(T, B, H, seed=80, device='cuda')
    programs.stacked_lstm(xss, Wss, Uss, bss)
    programs.stacked_lstm(xss, Wss, Uss, bss)
    assert dispatch.stats['weight_cache_hits'] == 1
    Wss.data.mul_(0.5)                                   # an in-place update of the parameters, as an optimizer makes
    out = programs.stacked_lstm(xss, Wss, Uss, bss)
    assert dispatch.stats['weight_cache_hits'] == 1
    WU, bias = _np_params(Wss, Uss, bss)
    ref, _ = ko.stacked_lstm(xss.as_dense().cpu().numpy().reshape(T, B, H), WU, bias)
    assert ko.max_rel_err(out.as_dense().cpu().numpy().reshape(T, B, H), ref[-1]) <= 1e-4


def _scaled_layer(seq, ws, us, bs):
    return programs.lstm_layer(seq, ws, us, bs)


def test_a_layer_function_redefined_at_module_level_is_probed_again():
    """The fold's lambda reaches its layer function through a module global.  When that global is rebound to a
    function that computes something else, the verdict of the old one must not be reused."""
    L, T, B, H = 2, 3, 2, 32
    Wss, Uss, bss = programs.make_lstm_params(L, H, 1 / 8, seed=81, device='cuda')
    xss = programs.make_sequence_batch(T, B, H, seed=82, device='cuda')
    run = lambda: ops.fold(lambda s, p: _scaled_layer(s, *p), ops.zip(Wss, Uss, bss), initializer=xss)
    first = run()
    assert dispatch.stats['stacked_lstm'] == 1 and dispatch.stats['probes'] == 1
    original = globals()['_scaled_layer']

    def halved(seq, ws, us, bs):
        return FractalTensor.from_dense(programs.lstm_layer(seq, ws, us, bs).as_dense() * 0.5, 2)

    globals()['_scaled_layer'] = halved
    try:
        second = run()
    finally:
        globals()['_scaled_layer'] = original
    assert dispatch.stats['stacked_lstm'] == 1 and dispatch.stats['declined'] == 1      # probed anew, found different, run eagerly
    assert float((second.as_dense() - first.as_dense()).abs().max()) > 1e-3


# ---- attention ----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize('D,scale', [(128, 128 ** -0.5), (64, 1.0), (64, 0.2), (32, 32 ** -0.5)])   # 32: the reference example's head dimension
def test_programs_flash_attention_is_routed_with_its_scale(D, scale):
    core = _core()
    B, Hd, S, blk = 2, 2, 256, 64
    qsss, ksss, vsss = (programs.make_attention_input(B, Hd, S, blk, D, seed=20 + i, device='cuda', dtype=torch.float16) for i in range(3))
    out = programs.flash_attention(qsss, ksss, vsss, scale)
    assert dispatch.stats['flash_attention'] == 1 and dispatch.stats['declined'] == 0
    assert out.depth == 3 and out.dense_shape() == (B, Hd, S // blk) and out.element_shape == (blk, D)
    to4 = lambda t: t.as_dense().reshape(B, Hd, S, D).float().cpu().numpy()
    ref = ko.attention(to4(qsss), to4(ksss), to4(vsss), scale, dtype=np.float32)
    assert ko.max_rel_err(to4(out), ref) <= 1e-2
    before = core.launch_counts['flash_attention']
    programs.flash_attention(qsss, ksss, vsss, scale)
    assert core.launch_counts['flash_attention'] == before + 1 and dispatch.stats['probes'] == 1
    programs.flash_attention(qsss, ksss, vsss, scale * 0.5)               # another scale in the closure: probed anew
    assert dispatch.stats['probes'] == 2


def test_reference_style_flash_attention_without_a_scale():
    B, Hd, S, blk, D = 1, 2, 128, 64, 64
    qsss, ksss, vsss = (programs.make_attention_input(B, Hd, S, blk, D, seed=30 + i, device='cuda', dtype=torch.float16) for i in range(3))
    scaled = FractalTensor.from_dense(qsss.as_dense() * 0.25, 3)           # keeps the unscaled scores in fp16's comfortable range
    out = flash_attention(scaled, ksss, vsss)
    assert dispatch.stats['flash_attention'] == 1
    to4 = lambda t: t.as_dense().reshape(B, Hd, S, D).float().cpu().numpy()
    ref = ko.attention(to4(scaled), to4(ksss), to4(vsss), 1.0, dtype=np.float32)
    assert ko.max_rel_err(to4(out), ref) <= 1e-2


def test_reference_example_sizes_of_flash_attention():
    """The example's own configuration (examples/flash_attention/flash_attention.py:96-110): batch 2, 8 heads, 1024
    tokens in blocks of 64, head dimension 32, fp32 data, no scale.  Routed by default, to the fp32 kernel: the
    result is within 1e-4 of float64."""
    core = _core()
    B, Hd, S, blk, D = 2, 8, 1024, 64, 32
    qsss, ksss, vsss = (programs.make_attention_input(B, Hd, S, blk, D, seed=60 + i, device='cuda') for i in range(3))
    scaled = FractalTensor.from_dense(qsss.as_dense() * 0.25, 3)
    before = core.launch_counts.get('flash_attention_f32', 0)
    out = flash_attention(scaled, ksss, vsss)
    assert dispatch.stats['flash_attention'] == 1 and out.data.dtype == torch.float32
    assert core.launch_counts['flash_attention_f32'] == before + 2      # the probe's reference and the program
    to4 = lambda t: t.as_dense().reshape(B, Hd, S, D).double().cpu().numpy()
    ref = ko.attention(to4(scaled), to4(ksss), to4(vsss), 1.0)
    assert ko.max_rel_err(to4(out), ref) <= 1e-4
    flash_attention(scaled, ksss, vsss)                                  # warm: one launch, no probe
    assert core.launch_counts['flash_attention_f32'] == before + 3 and dispatch.stats['probes'] == 1


def test_fp32_attention_program_goes_to_the_fp32_kernel_unless_half_is_allowed():
    core = _core()
    B, Hd, S, blk, D = 1, 1, 128, 64, 64
    qsss, ksss, vsss = (programs.make_attention_input(B, Hd, S, blk, D, seed=40 + i, device='cuda') for i in range(3))
    dispatch.enabled = False
    eager = programs.flash_attention(qsss, ksss, vsss, D ** -0.5)
    dispatch.enabled = True
    routed = programs.flash_attention(qsss, ksss, vsss, D ** -0.5)
    assert dispatch.stats['flash_attention'] == 1 and routed.data.dtype == torch.float32
    assert core.launch_counts.get('flash_attention_f32', 0) >= 1
    assert ko.max_rel_err(routed.data.cpu().numpy(), eager.data.cpu().numpy()) <= 1e-4
    dispatch.allow_half_attention = True
    half_before = core.launch_counts.get('flash_attention', 0)
    lowered = programs.flash_attention(qsss, ksss, vsss, D ** -0.5)
    assert core.launch_counts.get('flash_attention', 0) == half_before + 1 and lowered.data.dtype == torch.float32
    assert ko.max_rel_err(lowered.data.cpu().numpy(), eager.data.cpu().numpy()) <= 1e-2


# ---- (a @ b) @ c -----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize('M,K,N,P', [
    (4096, 128, 128, 128),     # one problem of BASELINE configs[1]: b and c go down row-major as they are
    (8192, 64, 256, 64),       # a shape of the reference's own benchmark: the wide-N kernel
    (200, 96, 64, 160),        # ragged rows, the general kernel
])
def test_chained_matmul_runs_as_one_back_to_back_gemm(M, K, N, P):
    core = _core()
    rng = np.random.default_rng(50)
    a, b, c = ((rng.standard_normal(s) / np.sqrt(s[0])).astype(np.float16) for s in ((M, K), (K, N), (N, P)))
    a[:] = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float16)
    ta, tb, tc = (Tensor.from_tensor(torch.from_numpy(x).cuda()) for x in (a, b, c))
    before = core.launch_counts.get('b2b_gemm', 0) + core.launch_counts.get('b2b_gemm_rowmajor', 0)
    d = (ta @ tb) @ tc
    assert dispatch.stats['b2b_gemm'] == 1
    assert core.launch_counts.get('b2b_gemm', 0) + core.launch_counts.get('b2b_gemm_rowmajor', 0) == before + 1
    assert d.shape == (M, P) and d.data.dtype == torch.float16
    ref = ko.b2b_gemm(a, np.ascontiguousarray(b.T), np.ascontiguousarray(c.T))
    assert ko.max_rel_err(d.data.float().cpu().numpy(), ref) <= 1e-2
    dispatch.enabled = False
    eager = (ta @ tb) @ tc
    assert ko.max_rel_err(d.data.float().cpu().numpy(), eager.data.float().cpu().numpy()) <= 1e-2


def test_chained_matmul_beyond_the_fused_kernels_runs_as_two_products():
    """N = 4096: more than the general back-to-back kernel holds of the intermediate product.  The chain must run as
    the two torch products it always was, not raise."""
    core = _core()
    assert core.b2b_gemm_supported(2048, 128, 128) and not core.b2b_gemm_supported(4096, 128, 128)
    rng = np.random.default_rng(52)
    M, K, N, P = 64, 128, 4096, 64
    a, b, c = (torch.from_numpy((rng.standard_normal(s) / np.sqrt(s[0])).astype(np.float16)).cuda() for s in ((M, K), (K, N), (N, P)))
    p = Tensor.from_tensor(a) @ Tensor.from_tensor(b)
    assert p._pending is None                                            # never left pending
    d = p @ Tensor.from_tensor(c)
    assert dispatch.stats['b2b_gemm'] == 0 and torch.equal(d.data, (a @ b) @ c)
    # N = 2048 with K = 128: past the fused kernels' LDS, inside the general kernel's reach
    b2, c2 = b[:, :2048].contiguous(), c[:2048].contiguous()
    d2 = (Tensor.from_tensor(a) @ Tensor.from_tensor(b2)) @ Tensor.from_tensor(c2)
    assert dispatch.stats['b2b_gemm'] == 1
    ref = ko.b2b_gemm(a.cpu().numpy(), np.ascontiguousarray(b2.cpu().numpy().T), np.ascontiguousarray(c2.cpu().numpy().T))
    assert ko.max_rel_err(d2.data.float().cpu().numpy(), ref) <= 1e-2


def test_a_large_plain_product_runs_on_the_library_kernel():
    """ops.mm on fp16 GPU operands: the library's product kernel when there is a 256 x 256 tile for every compute unit
    (N % 256 == 0, K % 32 == 0), torch's otherwise; the same values either way."""
    core = _core()
    rng = np.random.default_rng(53)
    M, K, N = 4000, 160, 4096                       # 16 x 16 tiles, the last row block ragged
    a = torch.from_numpy((rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float16)).cuda()
    b = torch.from_numpy(rng.standard_normal((K, N)).astype(np.float16)).cuda()
    before = core.launch_counts.get('gemm', 0)
    d = Tensor.from_tensor(a) @ Tensor.from_tensor(b)
    assert dispatch.stats['gemm'] == 1 and core.launch_counts.get('gemm', 0) == before + 1
    ref = a.double() @ b.double()
    assert d.shape == (M, N) and d.data.dtype == torch.float16
    assert float((d.data.double() - ref).abs().max() / ref.abs().max()) <= 1e-3
    assert float((d.data == ref.half()).float().mean()) > 0.98        # fp32 sums of exact products, rounded once
    # few tiles, a width that is no multiple of 256, fp32 operands: torch's product, bit for bit
    for aa, bb in ((a[:512].contiguous(), b), (a, b[:, :4000].contiguous()), (a.float(), b.float())):
        d = Tensor.from_tensor(aa) @ Tensor.from_tensor(bb)
        assert dispatch.stats['gemm'] == 1 and torch.equal(d.data, aa @ bb)


def test_a_pending_product_is_formed_by_any_other_use():
    rng = np.random.default_rng(51)
    a, b = (torch.from_numpy((rng.standard_normal(s) / 8).astype(np.float16)).cuda() for s in ((64, 64), (64, 96)))
    p = Tensor.from_tensor(a) @ Tensor.from_tensor(b)
    assert p._pending is not None and p.shape == (64, 96) and p.device == 'cuda'       # nothing has run yet
    s = p + p                                                                           # a use: the product is formed by torch
    assert p._pending is None and torch.equal(p.data, a @ b) and torch.equal(s.data, (a @ b) * 2)
    # products the fused kernels do not take are never left pending: fp32 operands, a transposed view, a single row
    q = Tensor.from_tensor(a.float()) @ Tensor.from_tensor(b.float())
    assert q._pending is None
    q = Tensor.from_tensor(a) @ Tensor.from_tensor(a).T
    assert q._pending is None and torch.equal(q.data, a @ a.t())
    q = Tensor.from_tensor(a[:1].contiguous()) @ Tensor.from_tensor(b)
    assert q._pending is None
    # a second factor the kernels do not take: the chain falls back to two torch products
    c = torch.from_numpy((rng.standard_normal((96, 40)) / 8).astype(np.float16)).cuda()
    d = (Tensor.from_tensor(a) @ Tensor.from_tensor(b)) @ Tensor.from_tensor(c)
    assert dispatch.stats['b2b_gemm'] == 0 and torch.equal(d.data, (a @ b) @ c)
