"""numpy restatement of the FractalTensor hot-path algorithms (CPU oracle).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; never by the shipped package.

Every function cites the reference file:line whose algorithm it restates
(paths relative to the reference checkout).  Arithmetic runs in the dtype of
the ``dtype`` argument (float64 by default, float32 to mirror torch CPU).

Pinning status (what checks each function independently of its own formula;
the checks live in ``tests/test_oracle.py``):

* lstm_cell / lstm_cell_per_gate / lstm_layer / stacked_lstm: pinned by
  torch.nn.LSTM after permuting gate blocks (i,f,o,g)->(i,f,g,o), by the
  zero-weight closed form c=0.5*c_prev, h=0.5*tanh(c), by the saturated
  forget-gate carry case, and by per-gate == fused-gate equivalence.
* wavefront_diagonals / stacked_lstm_wavefront: pinned by brute force over
  all small (L, T): every cell exactly once, dependencies satisfied, result
  bit-identical to layer-major order.
* dilate_indices / revert_dilate_indices / dilated_lstm: pinned by the three
  literal examples in the reference docstring and by equivalence between the
  recurrence form and d independent interleaved scans.
* b2b_gemm: pinned by identity / permutation matrices and float64 matmul.
* attention / flash_attention_blockwise / md_merge / online_softmax: pinned
  by torch softmax / scaled_dot_product_attention, rows summing to one,
  block-partition invariance, uniform-key => mean(V).
* grid_rnn / grid_rnn_batched (checks in ``tests/test_frontend.py``): pinned by
  the corner position and one interior position worked by hand from their
  neighbours, by the eager nested-scan program built from the frontend's own
  operators, by equality of the two layouts sample by sample, and by the grid
  of width one, which is a plain stacked tanh RNN written directly.
* window_positions / windowed_attention (``tests/test_frontend.py``): pinned by
  hand-worked windows including both wrapped ends, by torch softmax on
  explicit index lists, and by the eager shifted_slide + sparse_attn program.
  The reference holds no expected output for either model; the windowed
  access operators themselves (slide, window, ...) are "parity unpinned" in
  the sense that only their source and documentation fix them.
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------
# error metrics used by every parity test
# --------------------------------------------------------------------------


def max_rel_err(got, ref) -> float:
    """max|got-ref| / max|ref| (normalised maximum error)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    denom = float(np.max(np.abs(ref)))
    if denom == 0.0:
        return float(np.max(np.abs(got)))
    return float(np.max(np.abs(got - ref)) / denom)


def max_elem_rel_err(got, ref, floor) -> float:
    """max over elements of |got-ref| / max(|ref|, floor)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)))


# --------------------------------------------------------------------------
# LSTM
# --------------------------------------------------------------------------


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def lstm_cell(x, h_prev, c_prev, WU, bias=None, dtype=np.float64):
    """One batched LSTM cell with the fused gate GEMM.

    g = [x, h_prev] @ WU + bias with column blocks [i | f | o | c~];
    i, f, o = sigmoid; c~ = tanh; c = f*c_prev + i*c~; h = o*tanh(c).

    Follows examples/stacked_rnn/stacked_rnn.py:13-36 (gate_f + lstm_cell,
    gate order i, f, o, candidate) in the batched fused form of
    benchmarks/rnn/baselines/stacked_lstm/pt_model/rnn.py:94-108.

    x [B, I], h_prev/c_prev [B, H], WU [I+H, 4H], bias [4H] or None.
    """
    x = np.asarray(x, dtype=dtype)
    h_prev = np.asarray(h_prev, dtype=dtype)
    c_prev = np.asarray(c_prev, dtype=dtype)
    WU = np.asarray(WU, dtype=dtype)
    H = h_prev.shape[1]
    g = np.concatenate([x, h_prev], axis=1) @ WU
    if bias is not None:
        g = g + np.asarray(bias, dtype=dtype)[None, :]
    i = sigmoid(g[:, 0 * H:1 * H])
    f = sigmoid(g[:, 1 * H:2 * H])
    o = sigmoid(g[:, 2 * H:3 * H])
    cand = np.tanh(g[:, 3 * H:4 * H])
    c = f * c_prev + i * cand
    h = o * np.tanh(c)
    return h.astype(dtype), c.astype(dtype)


def lstm_cell_per_gate(x, h_prev, c_prev, ws, us, bs, dtype=np.float64):
    """The reference's literal per-gate form: four separate x@w + h@u + b.

    examples/stacked_rnn/stacked_rnn.py:13-19 (gate_f) and :31-35.
    ws/us: sequences of four [I,H]/[H,H] matrices, bs: four [1,H] rows.
    """
    x = np.asarray(x, dtype=dtype)
    h_prev = np.asarray(h_prev, dtype=dtype)
    c_prev = np.asarray(c_prev, dtype=dtype)
    pre = [x @ np.asarray(ws[k], dtype=dtype) + h_prev @ np.asarray(us[k], dtype=dtype)
           + np.asarray(bs[k], dtype=dtype) for k in range(4)]
    gate = [sigmoid(p) for p in pre[:3]]
    c = gate[1] * c_prev + gate[0] * np.tanh(pre[3])
    h = gate[2] * np.tanh(c)
    return h, c


def fuse_gate_weights(ws, us):
    """[W;U] with column blocks i|f|o|c~ from per-gate matrices."""
    W = np.concatenate([np.asarray(w) for w in ws], axis=1)
    U = np.concatenate([np.asarray(u) for u in us], axis=1)
    return np.concatenate([W, U], axis=0)


def lstm_layer(xs, WU, bias=None, h0=None, c0=None, dilation=1, dtype=np.float64):
    """Scan of lstm_cell over time; state taken from step t-dilation.

    examples/stacked_rnn/stacked_rnn.py:54-65 (scan over time with zero
    initial state) and, for dilation>1, the recurrence that
    kaleido/frontend/operations/fractaltensor/functional/apply_to_each.py:83-177
    (DilatedMap) induces: h_t = cell(x_t, state_{t-d}), zero state for t<d.

    xs [T, B, I]; returns hs, cs [T, B, H].
    """
    xs = np.asarray(xs, dtype=dtype)
    T, B, _ = xs.shape
    H = np.asarray(WU).shape[1] // 4
    hs = np.zeros((T, B, H), dtype=dtype)
    cs = np.zeros((T, B, H), dtype=dtype)
    zero = np.zeros((B, H), dtype=dtype)
    for t in range(T):
        if t >= dilation:
            hp, cp = hs[t - dilation], cs[t - dilation]
        else:
            hp = zero if h0 is None else np.asarray(h0, dtype=dtype)
            cp = zero if c0 is None else np.asarray(c0, dtype=dtype)
        hs[t], cs[t] = lstm_cell(xs[t], hp, cp, WU, bias, dtype=dtype)
    return hs, cs


def stacked_lstm(xs, WUs, biases=None, dilations=None, dtype=np.float64):
    """L stacked layers, layer-major order; layer l input = layer l-1 hs.

    examples/stacked_rnn/stacked_rnn.py:69-79 (fold over layers).  With
    ``dilations`` it is the dilated RNN of
    examples/dilated_rnn/dilated_rnn.py:16-41 (layer k uses 2**k there).

    xs [T,B,H]; WUs [L,2H,4H]; biases [L,4H] or None.
    Returns hsss, csss [L,T,B,H].
    """
    xs = np.asarray(xs, dtype=dtype)
    L = len(WUs)
    T, B, _ = xs.shape
    H = np.asarray(WUs[0]).shape[1] // 4
    hsss = np.zeros((L, T, B, H), dtype=dtype)
    csss = np.zeros((L, T, B, H), dtype=dtype)
    inp = xs
    for l in range(L):
        d = 1 if dilations is None else int(dilations[l])
        b = None if biases is None else biases[l]
        hsss[l], csss[l] = lstm_layer(inp, WUs[l], b, dilation=d, dtype=dtype)
        inp = hsss[l]
    return hsss, csss


def stacked_lstm_f16(xs, WUs, biases=None, dilations=None):
    """The same stack with fp16 storage: xs, WUs given in fp16, gate sums and the state update in wider
    arithmetic (float64 here; fp16 products are exact in fp32), and every h and c rounded to fp16 when it
    is written -- the rounded values are what the next step and the next layer read.

    This is the numeric form of the reference's CuTe LSTM, whose tensors are all `half` with fp32 MFMA
    accumulators (kaleido/core/device/kernels/lstm.h:253-348, lstm_kernels.h:25-126; element type
    `cutlass::half_t` in benchmarks/rnn/fractaltensor/cute_stacked_lstm/stacked_lstm.cu:16-19), applied to the
    cell of examples/stacked_rnn/stacked_rnn.py:13-36.  Returns hsss, csss [L,T,B,H] as float16.
    """
    xs = np.asarray(xs, dtype=np.float16)
    L = len(WUs)
    T, B, _ = xs.shape
    H = np.asarray(WUs[0]).shape[1] // 4
    hsss = np.zeros((L, T, B, H), dtype=np.float16)
    csss = np.zeros((L, T, B, H), dtype=np.float16)
    zero = np.zeros((B, H), dtype=np.float64)
    inp = xs
    for l in range(L):
        d = 1 if dilations is None else int(dilations[l])
        WU = np.asarray(WUs[l], dtype=np.float16).astype(np.float64)
        b = None if biases is None else np.asarray(biases[l], dtype=np.float64)
        for t in range(T):
            hp = hsss[l, t - d].astype(np.float64) if t >= d else zero
            cp = csss[l, t - d].astype(np.float64) if t >= d else zero
            h, c = lstm_cell(inp[t].astype(np.float64), hp, cp, WU, b, dtype=np.float64)
            hsss[l, t] = h.astype(np.float16)
            csss[l, t] = c.astype(np.float16)
        inp = hsss[l]
    return hsss, csss


def wavefront_diagonals(L, T):
    """The reference's three-region wavefront schedule as a list of stages.

    Region 1 = layer 0 for every t (kernels/lstm/stacked_lstm/region1.h:11-43),
    region 2 = layers >= 1 at t = 0 (region2.h:15-70), region 3 = diagonals
    m = l + t in [2, T+L-1) with l in [max(1, m-T+1), min(L, m))
    (region3.h:44-56).  Each stage is a list of (l, t) cells that may run
    concurrently once all earlier stages are done... with the caveat that
    region 1 and region 2 are themselves sequential chains, so they are
    emitted one cell per stage.
    """
    stages = []
    for t in range(T):  # region 1
        stages.append([(0, t)])
    for l in range(1, L):  # region 2
        stages.append([(l, 0)])
    for m in range(2, T + L - 1):  # region 3
        lb = max(1, m - T + 1)
        ub = min(L, m)
        cells = [(l, m - l) for l in range(lb, ub)]
        if cells:
            stages.append(cells)
    return stages


def stacked_lstm_wavefront(xs, WUs, biases=None, dtype=np.float64):
    """stacked_lstm evaluated in wavefront_diagonals order (same arithmetic)."""
    xs = np.asarray(xs, dtype=dtype)
    L = len(WUs)
    T, B, _ = xs.shape
    H = np.asarray(WUs[0]).shape[1] // 4
    hsss = np.zeros((L, T, B, H), dtype=dtype)
    csss = np.zeros((L, T, B, H), dtype=dtype)
    done = np.zeros((L, T), dtype=bool)
    zero = np.zeros((B, H), dtype=dtype)
    for stage in wavefront_diagonals(L, T):
        for (l, t) in stage:
            if l > 0:
                assert done[l - 1, t], "input dependency not satisfied"
            if t > 0:
                assert done[l, t - 1], "state dependency not satisfied"
            x = xs[t] if l == 0 else hsss[l - 1, t]
            hp = zero if t == 0 else hsss[l, t - 1]
            cp = zero if t == 0 else csss[l, t - 1]
            b = None if biases is None else biases[l]
            hsss[l, t], csss[l, t] = lstm_cell(x, hp, cp, WUs[l], b, dtype=dtype)
        for (l, t) in stage:
            assert not done[l, t], "cell scheduled twice"
            done[l, t] = True
    assert done.all(), "cell never scheduled"
    return hsss, csss


def dilate_indices(n, dilation):
    """Index lists produced by DilatedMap._dilate.

    kaleido/frontend/operations/fractaltensor/functional/apply_to_each.py:123-137:
    if n <= dilation or dilation == 1 the sequence is returned whole, else
    x[i::dilation] for i in range(dilation).
    """
    if dilation <= 0:
        raise ValueError('dilation should be greater than 0.')
    if n <= dilation or dilation == 1:
        return [list(range(n))]
    return [list(range(i, n, dilation)) for i in range(dilation)]


def revert_dilate_indices(groups):
    """Order in which DilatedMap._revert_dilate re-interleaves group items.

    apply_to_each.py:139-158: for i in range(len(group 0)): for j in groups:
    skip when group j has exactly i items.  Returns [(group, pos), ...].
    """
    if len(groups) == 1:
        return [(0, i) for i in range(len(groups[0]))]
    order = []
    max_len = len(groups[0])
    for i in range(max_len):
        for j in range(len(groups)):
            if i == len(groups[j]):
                continue
            order.append((j, i))
    return order


def dilated_lstm_interleaved(xs, WUs, biases=None, dilations=(1,), dtype=np.float64):
    """Dilated stack computed the reference's way: dilate -> scan -> revert.

    examples/dilated_rnn/dilated_rnn.py:16-27 with apply_to_each.py:83-177.
    """
    xs = np.asarray(xs, dtype=dtype)
    L = len(WUs)
    T, B, _ = xs.shape
    H = np.asarray(WUs[0]).shape[1] // 4
    hsss = np.zeros((L, T, B, H), dtype=dtype)
    csss = np.zeros((L, T, B, H), dtype=dtype)
    inp = xs
    for l in range(L):
        groups = dilate_indices(T, int(dilations[l]))
        b = None if biases is None else biases[l]
        outs = [lstm_layer(inp[idx], WUs[l], b, dtype=dtype) for idx in groups]
        flat_t = []
        for (j, i) in revert_dilate_indices(groups):
            flat_t.append((groups[j][i], outs[j][0][i], outs[j][1][i]))
        for pos, (t, h, c) in enumerate(flat_t):
            # _revert_dilate emits items in time order; pos is the output slot
            hsss[l, pos], csss[l, pos] = h, c
            assert pos == t
        inp = hsss[l]
    return hsss, csss


# --------------------------------------------------------------------------
# back-to-back GEMM
# --------------------------------------------------------------------------


def b2b_gemm(A, B_nk, C_pn, round_intermediate=False, dtype=np.float64):
    """D = (A @ B) @ C for one problem, storage layouts of the reference.

    kaleido/core/operators/tests/b2b_gemm_test_utils.h:3-9: A [M,K] and D
    [M,P] row-major; B [K,N] and C [N,P] column-major, i.e. stored as
    B_nk [N,K] and C_pn [P,N] row-major.  With ``round_intermediate`` the
    product P = A@B is rounded to fp16 between the GEMMs as
    kaleido/core/device/kernels/cutlass_wmma.h:512-517 does.
    """
    A = np.asarray(A).astype(dtype)
    Bm = np.asarray(B_nk).astype(dtype).T
    Cm = np.asarray(C_pn).astype(dtype).T
    P = A @ Bm
    if round_intermediate:
        P = P.astype(np.float16).astype(dtype)
    return P @ Cm


# --------------------------------------------------------------------------
# attention / online softmax
# --------------------------------------------------------------------------


def softmax_rows(x, dtype=np.float64):
    """Three-pass row softmax (kaleido/core/device/kernels/softmax.h:165-172)."""
    x = np.asarray(x).astype(dtype)
    m = x.max(axis=-1, keepdims=True)
    e = np.exp(x - m)
    return e / e.sum(axis=-1, keepdims=True)


def md_merge(m1, d1, m2, d2):
    """Merge two (max, denominator) pairs.

    kaleido/core/device/kernels/online_softmax.h:27-30:
    d = d1 + d2*exp(m2-m1) when m1 > m2, else d2 + d1*exp(m1-m2).
    """
    m = np.maximum(m1, m2)
    d = d1 * np.exp(m1 - m) + d2 * np.exp(m2 - m)
    return m, d


def online_softmax_rows(x, chunk=1, dtype=np.float64):
    """Row softmax through a running (m, d) pair, then exp(x-m)/d.

    The accumulation rule is the corrected one, m' = max(m, x);
    d' = d*exp(m-m') + exp(x-m'); the reference's per-thread loop at
    kaleido/core/device/kernels/online_softmax.h:121-128 updates m before
    testing it and so never rescales d, which is why its own test needs a
    1e-1 tolerance (kaleido/core/operators/tests/test_softmax.cc:72-74).
    The final map is online_softmax.h:149-155 without the -64 clamp (the
    clamp only changes terms below exp(-64)).
    """
    x = np.asarray(x).astype(dtype)
    rows, cols = x.shape
    m = np.full((rows, 1), -np.inf, dtype=dtype)
    d = np.zeros((rows, 1), dtype=dtype)
    for s in range(0, cols, chunk):
        blk = x[:, s:s + chunk]
        bm = blk.max(axis=1, keepdims=True)
        bd = np.exp(blk - bm).sum(axis=1, keepdims=True)
        m, d = md_merge(m, d, bm, bd)
    return np.exp(x - m) / d


def attention(Q, K, V, scale, dtype=np.float64):
    """softmax(Q K^T * scale) V per (batch, head); Q,K,V [..., S, D].

    Closed form behind examples/flash_attention/README.md:29-42 and the
    un-blocked per-query form of examples/transformer/multi-head-attention.py:14-31.
    """
    Q = np.asarray(Q).astype(dtype)
    K = np.asarray(K).astype(dtype)
    V = np.asarray(V).astype(dtype)
    S = np.einsum('...qd,...kd->...qk', Q, K) * dtype(scale)
    P = softmax_rows(S, dtype=dtype)
    return np.einsum('...qk,...kd->...qd', P, V)


def flash_attention_blockwise(Q, K, V, scale, block_q=64, block_kv=64, dtype=np.float64):
    """Blockwise attention with the (m, l, o) online-softmax state.

    Restates attn_func / per_block_func of
    examples/flash_attention/flash_attention.py:14-60 step for step (o kept
    normalised every step) with two documented departures: the state is
    initialised as the README's math requires (m=-inf, l=0, o=0; the example
    passes (sum, max, o) into a (max, sum, o) signature, :57-59) and the
    score carries the 1/sqrt(d) ``scale`` that config 3 demands.
    Q [Sq, D], K/V [Skv, D] for a single head.
    """
    Q = np.asarray(Q).astype(dtype)
    K = np.asarray(K).astype(dtype)
    V = np.asarray(V).astype(dtype)
    Sq, D = Q.shape
    Skv = K.shape[0]
    out = np.zeros((Sq, V.shape[1]), dtype=dtype)
    for q0 in range(0, Sq, block_q):
        q = Q[q0:q0 + block_q]
        n = q.shape[0]
        prev_m = np.full((n, 1), -np.inf, dtype=dtype)
        prev_l = np.zeros((n, 1), dtype=dtype)
        prev_o = np.zeros((n, V.shape[1]), dtype=dtype)
        for k0 in range(0, Skv, block_kv):
            k = K[k0:k0 + block_kv]
            v = V[k0:k0 + block_kv]
            w = (q @ k.T) * dtype(scale)
            cur_m = w.max(axis=-1, keepdims=True)
            e = np.exp(w - cur_m)
            ev = e @ v
            cur_l = e.sum(axis=-1, keepdims=True)
            new_m = np.maximum(cur_m, prev_m)
            r_prev = np.exp(prev_m - new_m)
            r_cur = np.exp(cur_m - new_m)
            new_l = r_prev * prev_l + r_cur * cur_l
            prev_o = (prev_o * prev_l * r_prev + r_cur * ev) / new_l
            prev_m, prev_l = new_m, new_l
        out[q0:q0 + block_q] = prev_o
    return out


# ------------------------------------------------------------------ grid RNN

def grid_rnn(src, trg, params, dtype=np.float64):
    """Stacked grid RNN of examples/grid_rnn/grid_rnn.py:40-137 over one (source, target) pair.

    src [S, H], trg [Tg, H]; params: per block ((i2h_x [2H,H], h2h_x [H,H], b_x [H]), (i2h_y, h2h_y, b_y)).
    The outer scan runs over the target positions i, the inner one over the source positions j
    (product(src, trg) puts src along the inner level, access.py:206-244; direction_x scans the outer level,
    grid_rnn.py:99-113, direction_y the inner one, :78-95).  grid_cell (:53-74) forms s = [state_x | state_y]
    with state_x = h_x of position (i-1, j) and state_y = h_y of position (i, j-1), zeros outside the grid,
    and h_x = tanh(s @ i2h_x + x_t @ h2h_x + b_x), h_y = tanh(s @ i2h_y + y_t @ h2h_y + b_y)
    (vanilla_cell is called with the input as its `state` argument and s as `cur`, :47-50, 71-73).
    Returns h_x, h_y [Tg, S, H] of the last block.
    """
    src = np.asarray(src, dtype=dtype)
    trg = np.asarray(trg, dtype=dtype)
    S, H = src.shape
    Tg = trg.shape[0]
    x_in = np.broadcast_to(src[None, :, :], (Tg, S, H)).copy()
    y_in = np.broadcast_to(trg[:, None, :], (Tg, S, H)).copy()
    for (px, py) in params:
        i2h_x, h2h_x, b_x = (np.asarray(p, dtype=dtype) for p in px)
        i2h_y, h2h_y, b_y = (np.asarray(p, dtype=dtype) for p in py)
        hx = np.zeros((Tg, S, H), dtype=dtype)
        hy = np.zeros((Tg, S, H), dtype=dtype)
        for i in range(Tg):
            for j in range(S):
                state_x = hx[i - 1, j] if i > 0 else np.zeros(H, dtype=dtype)
                state_y = hy[i, j - 1] if j > 0 else np.zeros(H, dtype=dtype)
                s = np.concatenate([state_x, state_y])
                hx[i, j] = np.tanh(s @ i2h_x + x_in[i, j] @ h2h_x + b_x.reshape(-1))
                hy[i, j] = np.tanh(s @ i2h_y + y_in[i, j] @ h2h_y + b_y.reshape(-1))
        x_in, y_in = hx, hy
    return x_in, y_in


def grid_rnn_batched(xs, ys, Wx, Ux, bx, Wy, Uy, by, crossed=False, dtype=np.float64):
    """The same recurrence over a batch, in the array layout of the reference's grid benchmark
    (benchmarks/rnn/fractaltensor/grid_lstm/stacked_grid_rnn.cu:31-41): W* [D,H,H], U* [D,2H,H], biases
    [D, 1 or B, H] or None, output hsss [D, L1, L2, 2, B, H] with h_x at index 0 and h_y at 1.
    Position (d, i, j) reads x_in, y_in = hsss[d-1, i, j, 0/1], state_x = hsss[d, i-1, j, 0] and
    state_y = hsss[d, i, j-1, 1] (the gather indices of regions/region8.h:112-140), forms
    h = tanh(in @ W + [state_x | state_y] @ U + b) per direction (utils.h:671-700, 652-663); in the first block
    x_in = xs[i], y_in = ys[j] (regions/region2.h:74-76, crossed=False) or xs[j], ys[i] (the frontend program,
    where product(src, trg) puts src along the inner axis; crossed=True).
    """
    xs = np.asarray(xs, dtype=dtype)
    ys = np.asarray(ys, dtype=dtype)
    Wx, Ux, Wy, Uy = (np.asarray(t, dtype=dtype) for t in (Wx, Ux, Wy, Uy))
    D, H = Wx.shape[0], Wx.shape[-1]
    B = xs.shape[1]
    L1, L2 = (ys.shape[0], xs.shape[0]) if crossed else (xs.shape[0], ys.shape[0])
    hsss = np.zeros((D, L1, L2, 2, B, H), dtype=dtype)
    zeros = np.zeros((B, H), dtype=dtype)
    for d in range(D):
        b_x = np.asarray(bx[d], dtype=dtype) if bx is not None else 0.0
        b_y = np.asarray(by[d], dtype=dtype) if by is not None else 0.0
        for i in range(L1):
            for j in range(L2):
                if d > 0:
                    x_in, y_in = hsss[d - 1, i, j, 0], hsss[d - 1, i, j, 1]
                else:
                    x_in, y_in = (xs[j], ys[i]) if crossed else (xs[i], ys[j])
                state_x = hsss[d, i - 1, j, 0] if i > 0 else zeros
                state_y = hsss[d, i, j - 1, 1] if j > 0 else zeros
                s = np.concatenate([state_x, state_y], axis=1)
                hsss[d, i, j, 0] = np.tanh(x_in @ Wx[d] + s @ Ux[d] + b_x)
                hsss[d, i, j, 1] = np.tanh(y_in @ Wy[d] + s @ Uy[d] + b_y)
    return hsss


# ------------------------------------------------------------------ windowed attention

def window_positions(t, S, window, dilation):
    """Positions of the window centred on t as shifted_slide produces them
    (kaleido/frontend/operations/access.py:376-431): t - half + k*dilation with half = ((window-1)*dilation+1)//2,
    and the wrap of :384-390, x >= S -> x - S, x < 0 -> x + S - 1."""
    half = ((window - 1) * dilation + 1) // 2
    out = []
    for x in range(t - half, t + half + 1, dilation):
        out.append(x + S - 1 if x < 0 else (x - S if x >= S else x))
    return out


def windowed_attention(Q, K, V, window, dilation=1, extra_idx=None, scale=1.0, dtype=np.float64):
    """softmax(scale * q_t . K[P]^T) . V[P] per token with P = window_positions(t) ++ extra_idx[g, t]: the map of
    sparse_attn over the tokens (examples/sparse_attention/sparse_attention.py:25-38, 69-71; keys and values are the
    windowed ones joined with the randomly picked ones, :33-34).  Q, K, V [G, S, D]."""
    Q, K, V = (np.asarray(a, dtype=dtype) for a in (Q, K, V))
    G, S, D = Q.shape
    out = np.zeros_like(Q)
    for g in range(G):
        for t in range(S):
            P = window_positions(t, S, window, dilation)
            if extra_idx is not None:
                P = P + [int(i) for i in extra_idx[g, t]]
            s = scale * (K[g, P] @ Q[g, t])
            e = np.exp(s - s.max())
            out[g, t] = (e / e.sum()) @ V[g, P]
    return out
