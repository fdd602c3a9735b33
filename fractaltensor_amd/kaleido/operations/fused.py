"""GPU fast paths: the three hot-path programs of the reference as single
kernel calls on FractalTensors that live on the GPU.

  stacked_lstm   the fold-over-layers / scan-over-time / map-over-batch program of
                 examples/stacked_rnn/stacked_rnn.py:23-79
  dilated_lstm   the dilated_map program of examples/dilated_rnn/dilated_rnn.py:16-41
  flash_attention  the map / reduce program of examples/flash_attention/flash_attention.py:14-91
  b2b_gemm       (a @ b) @ c, the computation of benchmarks/fused_two_hgemms
  grid_rnn       the nested-scan program of examples/grid_rnn/grid_rnn.py:40-137 over a batch of samples
  windowed_attention  shifted_slide + the map of sparse_attn of examples/sparse_attention/sparse_attention.py:25-71

A regular (non-ragged) FractalTensor already is a dense row-major tensor in
its flat buffer, so inputs are handed to the kernels as views and outputs are
wrapped back without copies.  Everything here runs through the C ABI in
fractaltensor_amd._core; there is no CPU or PyTorch fallback: CPU inputs are
rejected, and a missing library is an ImportError.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..fractal_tensor import FractalTensor
from ..tensor import Tensor
from ..types import FractalTensorStorage, TensorStorage, torch_type_to_internal_type

__all__ = ['pack_lstm_weights', 'pad_time_major', 'unpad_time_major', 'stacked_lstm', 'dilated_lstm', 'lstm_cell', 'flash_attention', 'b2b_gemm', 'mm',
           'online_softmax', 'embedding_lookup', 'grid_rnn', 'windowed_attention']


def _core():
    from ... import _core
    return _core


def _dense_gpu(ft: FractalTensor, name: str, depth: int) -> torch.Tensor:
    if not isinstance(ft, FractalTensor):
        raise TypeError(f'{name} should be a FractalTensor.')
    if ft.depth != depth:
        raise ValueError(f'{name} should have depth {depth}, got {ft.depth}.')
    if not ft.is_regular():
        raise ValueError(f'{name} is ragged; the fused kernels take regular batches.')
    t = ft.as_dense()
    if not t.is_cuda:
        raise RuntimeError(f'{name} lives on {t.device}; the fused kernels run on the GPU only.')
    return t


def pack_lstm_weights(Wss: FractalTensor, Uss: FractalTensor, bss: Optional[FractalTensor] = None):
    """Per-gate parameters -> the fused layout of the kernels.

    Wss, Uss: depth-2 [L][4] of [H, H] (gate order i, f, o, candidate, as in
    examples/stacked_rnn/rnn_utils.py:28-36); bss: depth-2 [L][4] of [1, H].
    Returns WU [L, 2H, 4H] with column blocks i|f|o|c~ (x rows, then h rows)
    and bias [L, 4H] or None."""
    W = _dense_gpu(Wss, 'Wss', 2)   # [L, 4, H, H]
    U = _dense_gpu(Uss, 'Uss', 2)
    L, G, H, H2 = W.shape
    if G != 4 or H != H2 or U.shape != W.shape:
        raise ValueError('Wss and Uss should be [L][4] of [H, H].')
    WU = torch.cat([W.permute(0, 2, 1, 3).reshape(L, H, 4 * H), U.permute(0, 2, 1, 3).reshape(L, H, 4 * H)], dim=1)
    bias = None
    if bss is not None:
        b = _dense_gpu(bss, 'bss', 2)   # [L, 4, 1, H]
        bias = b.reshape(L, 4 * H).contiguous()
    return WU.contiguous(), bias


def pad_time_major(xss: FractalTensor):
    """Time-major batch [T][B_t] of [1, H] -> (dense [T, B_0, H], batch sizes or None).

    A regular batch is returned as a view.  A ragged one must be what
    examples/utils/data_utils.py:42-66 builds for sequences sorted by length:
    step t holds the first B_t sequences, B_t non-increasing.  It is padded with
    zero rows; rows of a batch are independent in every LSTM layer, so the
    padding rows compute values nobody reads and the rows that matter are exact."""
    if not isinstance(xss, FractalTensor):
        raise TypeError('xss should be a FractalTensor.')
    if xss.depth != 2:
        raise ValueError(f'xss should have depth 2, got {xss.depth}.')
    if xss.is_regular():
        xs = _dense_gpu(xss, 'xss', 2)
        return xs.reshape(xs.shape[0], xs.shape[1], xs.shape[-1]), None
    sizes = [len(step) for step in xss.indices]
    if any(b <= 0 for b in sizes) or any(a < b for a, b in zip(sizes, sizes[1:])):
        raise ValueError('a ragged batch must be time-major with non-increasing, positive batch sizes per step.')
    H = xss.element_shape[-1]
    flat = xss.data.view(-1, H)
    if not flat.is_cuda:
        raise RuntimeError(f'xss lives on {flat.device}; the fused kernels run on the GPU only.')
    xs = torch.zeros((len(sizes), sizes[0], H), dtype=flat.dtype, device=flat.device)
    off = 0
    for t, b in enumerate(sizes):
        xs[t, :b] = flat[off:off + b]
        off += b
    return xs, sizes


def unpad_time_major(dense: torch.Tensor, sizes) -> FractalTensor:
    """dense [T, B_0, H] -> depth-2 [T][B_t] of [1, H] keeping the first B_t rows of step t."""
    T, B0, H = dense.shape
    if sizes is None:
        return FractalTensor.from_dense(dense.reshape(T, B0, 1, H), 2)
    return FractalTensor.from_fractaltensors(
        *[FractalTensor.from_dense(dense[t, :b].reshape(b, 1, H), 1) for t, b in enumerate(sizes)])


def _run_stack(xss, Wss, Uss, bss, dilations, return_all_layers):
    core = _core()
    xs, sizes = pad_time_major(xss)
    WU, bias = pack_lstm_weights(Wss, Uss, bss)
    # a ragged batch goes down with its per-step row counts: 32-row blocks that have ended are skipped
    T_, B_, H_ = xs.shape
    if xs.dtype == torch.float16 and WU.dtype == torch.float16 and H_ % 32 == 0:
        # fp16 program, fp16 kernel: h and c are kept in fp16 like every other tensor of the program
        hsss, csss = core.stacked_lstm_f16(xs, WU, None if bias is None else bias.float(), dilations=dilations,
                                           active_rows=sizes)
    else:
        hsss, csss = core.stacked_lstm(xs.float(), WU.float(), None if bias is None else bias.float(), dilations=dilations,
                                       active_rows=sizes, exact_small_states=True)
    L = WU.shape[0]
    if return_all_layers:
        if sizes is None:
            T, B, H = xs.shape
            return (FractalTensor.from_dense(hsss.view(L, T, B, 1, H), 3),
                    FractalTensor.from_dense(csss.view(L, T, B, 1, H), 3))
        return (FractalTensor.from_fractaltensors(*[unpad_time_major(hsss[l], sizes) for l in range(L)]),
                FractalTensor.from_fractaltensors(*[unpad_time_major(csss[l], sizes) for l in range(L)]))
    return unpad_time_major(hsss[L - 1], sizes)


def stacked_lstm(xss: FractalTensor, Wss: FractalTensor, Uss: FractalTensor, bss: Optional[FractalTensor] = None,
                 return_all_layers: bool = False):
    """Stacked LSTM over a time-major batch.

    xss: depth-2 [T][B_t] of [1, H]: what stacked_rnn.py's `embs` is, either for
    equal-length sequences or the ragged time-major batch of length-sorted
    sequences (shrinking batch per step, stacked_rnn.py:49).  Returns the last layer's hidden sequence as depth-2 [T][B] of
    [1, H], which is what the reference's stacked_lstm returns; with
    return_all_layers the (h, c) of every layer as depth-3 [L][T][B]."""
    return _run_stack(xss, Wss, Uss, bss, None, return_all_layers)


def dilated_lstm(xss: FractalTensor, Wss: FractalTensor, Uss: FractalTensor, bss: Optional[FractalTensor] = None,
                 dilations: Optional[Sequence[int]] = None, return_all_layers: bool = False):
    """Dilated stack: layer k takes its state from step t - dilations[k]
    (default 2**k, the reference's choice, dilated_rnn.py:26).  xss as in stacked_lstm."""
    L = len(Wss)
    if dilations is None:
        dilations = [2 ** k for k in range(L)]
    return _run_stack(xss, Wss, Uss, bss, list(dilations), return_all_layers)


def lstm_cell(hs_prev: FractalTensor, cs_prev: FractalTensor, xs: FractalTensor, ws: FractalTensor,
              us: FractalTensor, bs: Optional[FractalTensor] = None):
    """One batched cell: the `batched_cell` of stacked_rnn.py:40-50 as one launch.
    hs_prev, cs_prev, xs: depth-1 [B] of [1, H]; ws, us: depth-1 [4] of [H, H]; bs: [4] of [1, H]."""
    core = _core()
    x = _dense_gpu(xs, 'xs', 1)
    B, H = x.shape[0], x.shape[-1]
    hp = _dense_gpu(hs_prev, 'hs_prev', 1).reshape(-1, H)[:B].contiguous()
    cp = _dense_gpu(cs_prev, 'cs_prev', 1).reshape(-1, H)[:B].contiguous()
    W = _dense_gpu(ws, 'ws', 1)
    U = _dense_gpu(us, 'us', 1)
    WU = torch.cat([W.permute(1, 0, 2).reshape(W.shape[1], 4 * H), U.permute(1, 0, 2).reshape(H, 4 * H)], dim=0).contiguous()
    bias = None if bs is None else _dense_gpu(bs, 'bs', 1).reshape(4 * H).contiguous()
    h, c = core.lstm_cell(x.reshape(B, -1).contiguous(), hp, cp, WU, bias)
    return FractalTensor.from_dense(h.view(B, 1, H), 1), FractalTensor.from_dense(c.view(B, 1, H), 1)


def flash_attention(qsss: FractalTensor, ksss: FractalTensor, vsss: FractalTensor, scale: Optional[float] = None):
    """Blockwise attention.  qsss, ksss, vsss: depth-3 [batch][head][block] of
    [block_rows, head_dim], the layout flash_attention_utils.create_input builds.
    The result has the structure of qsss.  fp32 inputs are converted to fp16 for
    the kernel (which accumulates in fp32) and the result converted back; `scale`
    multiplies the scores and defaults to 1.0, the reference program's maths
    (attn_func forms query @ key.T unscaled); pass head_dim ** -0.5 for the usual one."""
    core = _core()
    q = _dense_gpu(qsss, 'qsss', 3)   # [B, Hd, nb, rows, D]
    k = _dense_gpu(ksss, 'ksss', 3)
    v = _dense_gpu(vsss, 'vsss', 3)
    B, Hd, nbq, rq, D = q.shape
    to4 = lambda t: t.reshape(t.shape[0], t.shape[1], t.shape[2] * t.shape[3], t.shape[4])
    in_dtype = q.dtype
    O = core.flash_attention(to4(q).half().contiguous(), to4(k).half().contiguous(), to4(v).half().contiguous(),
                             1.0 if scale is None else float(scale))
    return FractalTensor.from_dense(O.to(in_dtype).view(B, Hd, nbq, rq, D), 3)


def b2b_gemm(a, b, c):
    """(a @ b) @ c in one kernel.  a [M,K], b [K,N], c [N,P] Tensors, or
    depth-1 FractalTensors of them (independent problems).  fp16 on the GPU."""
    core = _core()

    def dense(x, name):
        if isinstance(x, FractalTensor):
            return _dense_gpu(x, name, 1)
        if isinstance(x, Tensor):
            if not x.data.is_cuda:
                raise RuntimeError(f'{name} lives on {x.data.device}; the fused kernels run on the GPU only.')
            return x.data.unsqueeze(0)
        raise TypeError(f'{name} should be a Tensor or a FractalTensor.')

    A, Bm, Cm = dense(a, 'a'), dense(b, 'b'), dense(c, 'c')
    in_dtype = A.dtype
    K_, N_, P_ = A.shape[2], Bm.shape[2], Cm.shape[2]
    if core.b2b_gemm_rowmajor_supported(N_, K_, P_):
        # b and c as they are: the kernel transposes them between LDS and the matrix unit
        D = core.b2b_gemm_rowmajor(A.half().contiguous(), Bm.half().contiguous(), Cm.half().contiguous()).to(in_dtype)
    else:
        # the general kernel takes B and C with the contraction index contiguous
        D = core.b2b_gemm(A.half().contiguous(), Bm.half().transpose(1, 2).contiguous(),
                          Cm.half().transpose(1, 2).contiguous()).to(in_dtype)
    if isinstance(a, Tensor):
        return Tensor.from_tensor(D[0])
    return FractalTensor.from_dense(D, 1)


def mm(a: Tensor, b: Tensor) -> Tensor:
    """a @ b for fp16 Tensors on the GPU through the library's own MFMA product (ftk_gemm_f16): a [M,K], b [K,N],
    N a multiple of 128, K of 32, whatever the size.  `ops.mm` routes a product here by itself when it is large enough
    for this kernel to be the faster one (N a multiple of 256 and a 256 x 256 tile per compute unit) and leaves the
    rest with torch; this calls it on any shape the kernel takes."""
    for x, name in ((a, 'a'), (b, 'b')):
        if not isinstance(x, Tensor):
            raise TypeError(f'{name} should be a Tensor.')
        if not x.data.is_cuda:
            raise RuntimeError(f'{name} lives on {x.data.device}; the fused kernels run on the GPU only.')
    in_dtype = a.data.dtype
    return Tensor.from_tensor(_core().gemm(a.data.half().contiguous(), b.data.half().contiguous()).to(in_dtype))


def online_softmax(x: Tensor) -> Tensor:
    """Row softmax of a [rows, cols] fp32 Tensor through the online (max, sum) kernel."""
    return Tensor.from_tensor(_core().online_softmax(x.data.contiguous()))


def embedding_lookup(embedding: Tensor, words: FractalTensor) -> FractalTensor:
    """Rows of `embedding` [V, E] for every word id of `words`: what
    ops.map(lambda ws: ops.map(lambda word: ops.index(ops.slices(embedding, dim=0), word), ws), words)
    builds (examples/stacked_rnn/rnn_utils.py:81-90), as one gather.  `words` is a FractalTensor of any depth
    (regular or ragged) of single integers; the result has its structure with [1, E] elements.  An id outside
    [0, V) raises IndexError, as indexing the sliced matrix does."""
    if not isinstance(words, FractalTensor):
        raise TypeError('words should be a FractalTensor.')
    if not isinstance(embedding, Tensor):
        raise TypeError('embedding should be a Tensor.')
    table = embedding.data
    if table.dim() != 2:
        raise ValueError('embedding should be a [V, E] matrix.')
    if words.element_size != 1:
        raise ValueError('words should hold single integers.')
    ids = words._T
    if ids is None or words.indices is None:
        raise RuntimeError('FractalTensor is not initialized.')
    if not table.is_cuda or not ids.is_cuda:
        raise RuntimeError('embedding_lookup runs on the GPU only; move the embedding and the words there.')
    V, E = table.shape
    out = _core().embedding_gather(table.contiguous().float(), ids.reshape(-1).contiguous())
    typ = TensorStorage((1, E), torch_type_to_internal_type(out.dtype), device=out.device.type)
    for _ in range(words.depth - 1):
        typ = FractalTensorStorage(typ)
    ft = FractalTensor(typ)
    ft.indices = words.indices
    ft._T = out.reshape(-1)
    return ft


def grid_rnn(srcs: FractalTensor, trgs: FractalTensor, params):
    """The stacked grid RNN of examples/grid_rnn/grid_rnn.py:40-137 for a batch of samples in one call per plane
    of the (block, target, source) grid.

    srcs: depth-2 [N][S] of [1, H], trgs: depth-2 [N][Tg] of [1, H] (the two sides of the reference's outer map
    over samples, :127-137; equal lengths within the batch); params: per block ((i2h [2H, H], h2h [H, H],
    bias [1, H]) for the x direction, the same for y), Tensors on the GPU.  Returns (h_x, h_y), each depth-3
    [N][Tg][S] of [1, H]: the last block's outputs at every grid position, as the eager program returns them."""
    core = _core()
    xs = _dense_gpu(srcs, 'srcs', 2)   # [N, S, 1, H]
    ys = _dense_gpu(trgs, 'trgs', 2)   # [N, Tg, 1, H]
    N, S, one, H = xs.shape
    if one != 1 or ys.shape[0] != N or tuple(ys.shape[2:]) != (1, H):
        raise ValueError('srcs and trgs should be [N][S] and [N][Tg] of [1, H].')
    Tg = ys.shape[1]

    def stack(direction: int, which: int, shape):
        ts = []
        for block in params:
            t = block[direction][which]
            t = t.data if isinstance(t, Tensor) else t
            if tuple(t.shape) != shape:
                raise ValueError(f'grid parameter of shape {tuple(t.shape)}, expected {shape}.')
            if not t.is_cuda:
                raise RuntimeError('grid_rnn runs on the GPU only; move the parameters there.')
            ts.append(t.float())
        return torch.stack(ts).contiguous()

    Ux, Wx, bx = stack(0, 0, (2 * H, H)), stack(0, 1, (H, H)), stack(0, 2, (1, H))
    Uy, Wy, by = stack(1, 0, (2 * H, H)), stack(1, 1, (H, H)), stack(1, 2, (1, H))
    xs_t = xs.reshape(N, S, H).transpose(0, 1).contiguous().float()    # [S, N, H]: the source runs along the inner axis
    ys_t = ys.reshape(N, Tg, H).transpose(0, 1).contiguous().float()   # [Tg, N, H]
    hsss = core.grid_rnn(xs_t, ys_t, Wx, Ux, bx, Wy, Uy, by, crossed=True)   # [D, Tg, S, 2, N, H]
    last = hsss[-1].permute(2, 3, 0, 1, 4).contiguous()                      # [2, N, Tg, S, H]
    return (FractalTensor.from_dense(last[0].reshape(N, Tg, S, 1, H), 3),
            FractalTensor.from_dense(last[1].reshape(N, Tg, S, 1, H), 3))


def windowed_attention(query: FractalTensor, key: FractalTensor, value: FractalTensor, window_size: int,
                       dilation: int = 1, random_attn_pos: Optional[FractalTensor] = None) -> FractalTensor:
    """ops.shifted_slide(ops.zip(key, value), window_size, dilation) followed by the map of sparse_attn over the
    tokens (examples/sparse_attention/sparse_attention.py:25-38, 51-53, 69-71), as one kernel.

    query, key, value: regular FractalTensors of one structure, depth >= 1, of [1, D] tokens; the innermost level is
    the sequence, the outer ones (heads, batch) are independent.  random_attn_pos: the same structure of [1, R]
    integer tokens, or None.  The result has the structure of `query`."""
    if not all(isinstance(t, FractalTensor) for t in (query, key, value)):
        raise TypeError('query, key and value should be FractalTensors.')
    depth = query.depth
    q = _dense_gpu(query, 'query', depth)
    k = _dense_gpu(key, 'key', depth)
    v = _dense_gpu(value, 'value', depth)
    if q.shape != k.shape or q.shape != v.shape or q.shape[-2] != 1:
        raise ValueError('query, key and value should have one structure of [1, D] tokens.')
    S, D = q.shape[-3], q.shape[-1]
    extra = None
    if random_attn_pos is not None:
        r = _dense_gpu(random_attn_pos, 'random_attn_pos', depth)
        if r.shape[:-1] != q.shape[:-1] or r.is_floating_point():
            raise ValueError('random_attn_pos should have the structure of query and hold [1, R] integers.')
        extra = r.reshape(-1, S, r.shape[-1]).to(torch.int32).contiguous()
    out = _core().windowed_attention(q.reshape(-1, S, D).float().contiguous(), k.reshape(-1, S, D).float().contiguous(),
                                     v.reshape(-1, S, D).float().contiguous(), window_size, dilation, extra, 1.0)
    return FractalTensor.from_dense(out.reshape(q.shape), depth)
