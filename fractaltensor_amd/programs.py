"""The hot-path model programs, and the grid RNN next to them, written against the kaleido operator API.

These are the eager counterparts of the reference's example programs: every
cell is a handful of torch calls on one sample and map / scan / fold are
Python loops.  They serve as (1) the operator-level statement of what the
fused kernels compute, used by the parity tests, and (2) the "CPU eager path"
baseline that bench.py times on configuration 1.

  stacked LSTM     examples/stacked_rnn/stacked_rnn.py:13-79 (time-major batch)
  dilated LSTM     examples/dilated_rnn/dilated_rnn.py:16-41 (here over a time-major batch)
  flash attention  examples/flash_attention/flash_attention.py:14-91, with the state
                   initialised as the README's maths requires (max -inf, sum 0, o 0;
                   the example seeds (sum, max, o) into a (max, sum, o) signature) and
                   an explicit score scale
  grid RNN         examples/grid_rnn/grid_rnn.py:40-137 (one sample: source x target grid,
                   two tanh cells per position sharing the state of both directions)
  windowed attn    examples/sparse_attention/sparse_attention.py:25-38, 51-53, 69-71 (one head: every token
                   attends to its shifted_slide window joined with randomly picked positions)
"""
from __future__ import annotations

import torch

from . import kaleido
from .kaleido import FractalTensor, Tensor
from .kaleido import operations as ops


# ---- parameters and inputs ----------------------------------------------------

def make_lstm_params(layers: int, hidden: int, scale: float, seed: int, device: str = 'cpu', bias: bool = True):
    """Wss, Uss: depth-2 [layers][4] of [hidden, hidden] ~ U(-scale, scale); bss: [layers][4] of [1, hidden]."""
    gen = torch.Generator().manual_seed(seed)
    W = (torch.rand((layers, 4, hidden, hidden), generator=gen) * 2 - 1) * scale
    U = (torch.rand((layers, 4, hidden, hidden), generator=gen) * 2 - 1) * scale
    b = (torch.rand((layers, 4, 1, hidden), generator=gen) * 2 - 1) * scale if bias else torch.zeros((layers, 4, 1, hidden))
    to = lambda t: FractalTensor.from_dense(t.to(device), 2)
    return to(W), to(U), to(b)


def make_sequence_batch(seq_len: int, batch: int, hidden: int, seed: int, device: str = 'cpu') -> FractalTensor:
    """Time-major batch: depth-2 [seq_len][batch] of [1, hidden] ~ N(0, 1)."""
    gen = torch.Generator().manual_seed(seed)
    return FractalTensor.from_dense(torch.randn((seq_len, batch, 1, hidden), generator=gen).to(device), 2)


def make_attention_input(batch: int, heads: int, seq_len: int, block: int, head_dim: int, seed: int,
                         device: str = 'cpu', dtype=torch.float32) -> FractalTensor:
    """depth-3 [batch][heads][seq_len/block] of [block, head_dim]."""
    gen = torch.Generator().manual_seed(seed)
    t = torch.randn((batch, heads, seq_len // block, block, head_dim), generator=gen)
    return FractalTensor.from_dense(t.to(device=device, dtype=dtype), 3)


# ---- LSTM ------------------------------------------------------------------------

def lstm_cell(h_prev: Tensor, c_prev: Tensor, x: Tensor, ws: FractalTensor, us: FractalTensor, bs: FractalTensor):
    """One sample, one step: four separate gate projections, gate order i, f, o, candidate."""
    pre = ops.map(lambda p: x @ p[0] + h_prev @ p[1] + p[2], ops.zip(ws, us, bs))
    i, f, o = (ops.sigmoid(pre[k]) for k in range(3))
    c = f * c_prev + i * ops.tanh(pre[3])
    h = o * ops.tanh(c)
    return h, c


def batched_cell(hs_prev, cs_prev, xs, ws, us, bs):
    n = xs.length
    return ops.map(lambda s: lstm_cell(s[0], s[1], s[2], ws, us, bs), ops.zip(hs_prev[0:n], cs_prev[0:n], xs))


def lstm_layer(xss: FractalTensor, ws, us, bs, dilation: int = 1) -> FractalTensor:
    hidden = xss.element_shape[-1]
    zero = ops.repeat(ops.zeros(shape=(1, hidden), device=xss.device), xss[0].length)

    def scan_time(seq):
        hss, css = ops.scan(lambda state, xs: batched_cell(state[0], state[1], xs, ws, us, bs), seq,
                            initializer=(zero, zero))
        return hss, css

    if dilation == 1:
        return scan_time(xss)[0]
    hss, _ = ops.dilated_map(scan_time, xss, dilation=dilation)
    return hss


def stacked_lstm(xss: FractalTensor, Wss, Uss, bss) -> FractalTensor:
    """Layer l reads layer l-1's hidden sequence; returns the last layer's."""
    return ops.fold(lambda seq, p: lstm_layer(seq, p[0], p[1], p[2]), ops.zip(Wss, Uss, bss), initializer=xss)


def dilated_lstm(xss: FractalTensor, Wss, Uss, bss) -> FractalTensor:
    """Layer k uses dilation 2**k."""
    layers = ops.enumerate(Wss, Uss, bss)
    return ops.fold(lambda seq, p: lstm_layer(seq, p[1], p[2], p[3], dilation=2 ** int(p[0].data.item())), layers,
                    initializer=xss)


# ---- attention -----------------------------------------------------------------------

def _attend_block(state, q: Tensor, k: Tensor, v: Tensor, scale: float):
    m_prev, l_prev, o_prev = state
    w = ops.scale(q @ k.T, Tensor.from_tensor(torch.tensor([scale], dtype=q.data.dtype, device=q.data.device)))
    m_cur = ops.max(w, dim=-1, keepdim=True)
    e = ops.exp(w - m_cur)
    ev = e @ v
    l_cur = ops.sum(e, dim=-1, keepdim=True)
    m_new = ops.maximum(m_cur, m_prev)
    r_prev = ops.exp(m_prev - m_new)
    r_cur = ops.exp(m_cur - m_new)
    l_new = r_prev * l_prev + r_cur * l_cur
    o = (o_prev * l_prev * r_prev + r_cur * ev) / l_new
    return m_new, l_new, o


def _attend_query_block(q: Tensor, ks: FractalTensor, vs: FractalTensor, scale: float) -> Tensor:
    rows, dim = q.shape
    dev = q.device
    init = (ops.full(shape=(rows, 1), fill_value=float('-inf'), device=dev), ops.zeros(shape=(rows, 1), device=dev),
            ops.zeros(shape=(rows, dim), device=dev))
    _, _, o = ops.reduce(lambda st, kv: _attend_block(st, q, kv[0], kv[1], scale), ops.zip(ks, vs), initializer=init)
    return o


def flash_attention(qsss: FractalTensor, ksss: FractalTensor, vsss: FractalTensor, scale: float) -> FractalTensor:
    per_head = lambda qkv: ops.map(lambda q: _attend_query_block(q, qkv[1], qkv[2], scale), qkv[0])
    return ops.map(lambda sample: ops.map(per_head, ops.zip(*sample)), ops.zip(qsss, ksss, vsss))


# ---- grid RNN -----------------------------------------------------------------

def make_grid_params(depth: int, hidden: int, seed: int, scale: float = None):
    """Per block the parameters of the two directions: (i2h [2H, H], h2h [H, H], bias [1, H]) each."""
    gen = torch.Generator().manual_seed(seed)
    scale = scale if scale is not None else 1.0 / (3 * hidden) ** 0.5
    mk = lambda *shape: Tensor.from_tensor((torch.rand(shape, generator=gen) * 2 - 1) * scale)
    cell = lambda: (mk(2 * hidden, hidden), mk(hidden, hidden), mk(1, hidden))
    return [(cell(), cell()) for _ in range(depth)]


def _vanilla_cell(state: Tensor, cur: Tensor, i2h: Tensor, h2h: Tensor, bias: Tensor) -> Tensor:
    return ops.tanh(cur @ i2h + state @ h2h + bias)


def _grid_cell(state, cur_input, block):
    """state: the outputs (h_x, h_y) of the position before along the inner direction, of which h_y is used;
    cur_input: (h_x of the same inner position one outer step before, (x_t, y_t) from the block below)."""
    _, state_y = state
    state_x, (x_t, y_t) = cur_input
    px, py = block
    s = ops.cat([state_x, state_y], dim=1)
    return _vanilla_cell(x_t, s, *px), _vanilla_cell(y_t, s, *py)


def _grid_row(state, cur_input, block, hidden: int):
    """One outer step: a scan along the inner direction; state = the row of outputs one outer step before."""
    state_xs, _ = state
    zero = ops.zeros(shape=(1, hidden), device='cpu')
    return ops.scan(lambda s, x: _grid_cell(s, x, block), ops.zip(state_xs, ops.zip(*cur_input)), initializer=(zero, zero))


def _grid_block(inputs, block, hidden: int):
    """One block of the stack: a scan along the outer direction over rows of (x, y) inputs."""
    zeros = ops.repeat(ops.zeros(shape=(1, hidden), device='cpu'), len(inputs[0][0]))
    ys1, ys2 = ops.scan(lambda s, x: _grid_row(s, x, block, hidden), inputs, initializer=(zeros, zeros))
    return ops.zip(ys1, ys2)


def grid_rnn(src: FractalTensor, trg: FractalTensor, params, hidden: int):
    """Stacked grid RNN over one (source, target) pair: src [S] and trg [Tg] of [1, H] Tensors.
    Returns (h_x, h_y), each depth-2 [Tg][S] of [1, H]: the last block's outputs at every grid position.
    Position (i, j) of a block computes, with s = [h_x(i-1, j) | h_y(i, j-1)] (zeros outside the grid),
      h_x(i, j) = tanh(s @ i2h_x + x_in(i, j) @ h2h_x + b_x),  h_y(i, j) = tanh(s @ i2h_y + y_in(i, j) @ h2h_y + b_y),
    where the first block's inputs are x_in(i, j) = src[j], y_in(i, j) = trg[i] and every other block's are
    the outputs of the block below."""
    blocks = kaleido.Iterative.make_iterative(*params)
    yss1, yss2 = ops.fold(lambda inputs, block: _grid_block(inputs, block, hidden), blocks,
                          initializer=ops.zip(*ops.product(src, trg)))
    return yss1, yss2


# ---- windowed (+ random) attention -----------------------------------------------------

def windowed_attention(query: FractalTensor, key: FractalTensor, value: FractalTensor, window_size: int,
                       dilation: int = 1, random_attn_pos: FractalTensor = None) -> FractalTensor:
    """One head of the windowed part of the reference's sparse attention, for every token (the reference runs it
    on the tokens between its global ones): query, key, value depth-1 [S] of [1, D]; random_attn_pos depth-1 [S]
    of [1, R] integer Tensors or None.  Token t attends to the window shifted_slide gives it, joined with
    key[ids], value[ids] of its random positions: softmax(q @ ks^T) @ vs with no score scale."""
    windowed_key, windowed_value = ops.shifted_slide(ops.zip(key, value), window_size=window_size, dilation=dilation)

    def sparse_attn(x):
        if random_attn_pos is None:
            query_token, w_keys, w_values = x
            ks, vs = ops.flatten(w_keys).T, ops.flatten(w_values)
        else:
            query_token, w_keys, w_values, ids = x
            ks = ops.flatten(w_keys.join(key[ids])).T
            vs = ops.flatten(w_values.join(value[ids]))
        return ops.softmax(query_token @ ks, dim=1) @ vs

    if random_attn_pos is None:
        return ops.map(sparse_attn, ops.zip(query, windowed_key, windowed_value))
    return ops.map(sparse_attn, ops.zip(query, windowed_key, windowed_value, random_attn_pos))
