"""Routing of unchanged operator programs to the fused kernels.

The reference's hot-path programs are compositions of fold / scan / map /
dilated_map / reduce over user functions (examples/stacked_rnn/stacked_rnn.py:54-79,
examples/dilated_rnn/dilated_rnn.py:16-41,
examples/flash_attention/flash_attention.py:47-91).  When such a composition is
called on FractalTensors that live on the GPU, `fold` and `map` ask this module
first.  A call is routed to one fused kernel launch when

  1. its operands have the structure of one of the programs (cheap checks on
     depths, element shapes, devices, types), and
  2. the user function has been SEEN to compute that program: it is run once,
     eagerly, on a small probe input (a few time steps and rows, or two key
     blocks) and its result must equal the fused kernel's on the same probe to
     the tolerance of the path (1e-4 for fp32 LSTMs, 1e-2 for fp16 ones and for
     attention).  What the operands cannot tell is read off the probe: the
     dilation of every layer (the dilated_map calls the function makes are
     noted) and the score scale of the attention (solved from a probe with one
     non-zero key).

The verdict is kept per function (code object and the scalars in its closure)
and operand structure, so the probe runs once per program, not per call.
Anything that does not match, or whose probe fails or raises, runs as the
eager loop it always was: that is the reference's execution model on torch's
GPU operators, not a substitute for a missing kernel.  A routed call needs
libftkernels.so; if it is missing the import error surfaces.

`(a @ b) @ c` is routed differently, since operators are eager and nothing can
be looked at when `a @ b` runs: on fp16 GPU tensors of shapes the back-to-back
GEMM kernels take, `a @ b` is left pending (kaleido.Tensor.pending_product) and
a following `@ c` runs the fused kernel on (a, b, c); any other use of the
product forms it with torch, as before.  The arithmetic is that of the two fp16
GEMMs (the intermediate rounded to fp16, fp32 accumulation).

  enabled                   False (or FTK_DISPATCH=0 in the environment) switches routing off
  allow_half_attention      route fp32 attention programs to the fp16 kernel too (off: a
                            routed program never computes in less than its own precision)
  stats                     counts of routed calls, probes and declined probes
"""
from __future__ import annotations

import math
import os
import threading
from typing import Callable, Optional

import torch

from ..fractal_tensor import FractalTensor, Iterative
from ..tensor import Tensor

enabled = os.environ.get('FTK_DISPATCH', '1') != '0'
allow_half_attention = False
stats = {'stacked_lstm': 0, 'dilated_lstm': 0, 'flash_attention': 0, 'b2b_gemm': 0, 'probes': 0, 'declined': 0}

_verdicts: dict = {}
_MAX_VERDICTS = 256
_local = threading.local()


def reset() -> None:
    """Forget every verdict and zero the counters."""
    _verdicts.clear()
    for k in stats:
        stats[k] = 0


def _core():
    from ... import _core
    return _core


def _probing() -> bool:
    return getattr(_local, 'depth', 0) > 0


class _Probe:
    """While a probe runs, nested operator calls stay eager and dilated_map calls are noted."""

    def __enter__(self):
        _local.depth = getattr(_local, 'depth', 0) + 1
        self.saved = getattr(_local, 'dilations', None)
        _local.dilations = []
        return self

    def __exit__(self, *exc):
        self.dilations = _local.dilations
        _local.dilations = self.saved
        _local.depth -= 1
        return False


def note_dilation(dilation: int) -> None:
    """Called by dilated_map: which dilation the function under probe asked for."""
    if _probing() and getattr(_local, 'dilations', None) is not None:
        _local.dilations.append(int(dilation))


def _fingerprint(f, level: int = 0):
    """What identifies a user function between calls: its code and the scalars and functions it closes over
    (a lambda is a new object at every call of the program, its code object is not)."""
    code = getattr(f, '__code__', None)
    if code is None:
        return ('object', id(f))
    parts = [code]
    for cell in (getattr(f, '__closure__', None) or ()):
        try:
            v = cell.cell_contents
        except ValueError:
            continue
        if isinstance(v, (int, float, str, bool, type(None))):
            parts.append(v)
        elif isinstance(v, (Tensor, FractalTensor, Iterative, torch.Tensor)):
            parts.append(type(v).__name__)     # data: its structure is checked per call
        elif callable(v) and hasattr(v, '__code__') and level < 4:
            parts.append(_fingerprint(v, level + 1))
        else:
            parts.append(('id', id(v)))
    return tuple(parts)


def _remember(key, verdict):
    if len(_verdicts) >= _MAX_VERDICTS:
        _verdicts.clear()
    _verdicts[key] = verdict


def _rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    got, ref = got.float(), ref.float()
    if not bool(torch.isfinite(got).all()):
        return math.inf
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# ------------------------------------------------------------------ stacked / dilated LSTM behind fold

def _lstm_fields(item):
    """(index or None, ws, us, bs) of one layer's fold item, or None if it is not [ws, us, bs] / [i, ws, us, bs]."""
    if not isinstance(item, (list, tuple)) or len(item) not in (3, 4):
        return None
    idx = None
    if len(item) == 4:
        idx, item = item[0], item[1:]
        if not isinstance(idx, Tensor) or idx.data.numel() != 1 or idx.data.is_floating_point():
            return None
    ws, us, bs = item
    for p in (ws, us, bs):
        if not isinstance(p, FractalTensor) or p.depth != 1 or len(p) != 4 or p.data is None or not p.data.is_cuda:
            return None
    H = ws.element_shape[-1]
    if tuple(ws.element_shape) != (H, H) or tuple(us.element_shape) != (H, H) or tuple(bs.element_shape) != (1, H):
        return None
    return idx, ws, us, bs


def _pack_layer(ws, us, bs):
    """[4] of [H, H], [4] of [H, H], [4] of [1, H] -> WU [2H, 4H] with column blocks i|f|o|candidate, bias [4H]."""
    W, U = ws.as_dense(), us.as_dense()
    H = W.shape[-1]
    WU = torch.cat([W.permute(1, 0, 2).reshape(H, 4 * H), U.permute(1, 0, 2).reshape(H, 4 * H)], dim=0)
    return WU, bs.as_dense().reshape(4 * H)


def _run_lstm(xs: torch.Tensor, WU: torch.Tensor, bias: torch.Tensor, dilations, active=None):
    """xs [T, B, H] -> the last layer's h [T, B, H], through the kernel of the operands' type."""
    core = _core()
    T = xs.shape[0]
    eff = [d if T > d else 1 for d in dilations]      # a sequence no longer than the dilation is one group, scanned in order
    dil = None if all(d == 1 for d in eff) else eff
    if xs.dtype == torch.float16:
        hsss, _ = core.stacked_lstm_f16(xs.contiguous(), WU.contiguous(), bias.float().contiguous(), dilations=dil, active_rows=active)
    else:
        hsss, _ = core.stacked_lstm(xs.contiguous(), WU.contiguous(), bias.contiguous(), dilations=dil, active_rows=active)
    return hsss[-1]


def _probe_lstm_layer(func: Callable, item, fields, H: int, dtype, seq_depth: int, gen) -> Optional[int]:
    """Runs func on a probe sequence with this layer's own parameters.  Returns the dilation it asked for (1 if
    none) when the result equals the fused layer's, else None."""
    _, ws, us, bs = fields
    WU, bias = _pack_layer(ws, us, bs)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    B = 2 if seq_depth == 2 else 1
    T = 3
    for _ in range(2):                                     # second pass: a probe longer than the dilation just seen
        x = torch.randn((T, B, 1, H), generator=gen).to(device='cuda', dtype=dtype)
        probe = FractalTensor.from_dense(x, 2) if seq_depth == 2 else FractalTensor.from_dense(x[:, 0], 1)
        with _Probe() as p:
            out = func(probe, item)
        asked = p.dilations
        if len(asked) > 1 or not isinstance(out, FractalTensor) or out.depth != seq_depth or not out.is_regular():
            return None
        d = asked[0] if asked else 1
        if d < 1:
            return None
        if d >= T:                                          # the recurrence did not show yet
            T = d + 2
            continue
        got = out.as_dense().reshape(-1, B, H)
        if got.shape[0] != T:
            return None
        ref = _run_lstm(x.reshape(T, B, H), WU[None], bias[None], [d])
        return d if _rel_err(got, ref) <= tol else None
    return None


def try_fold(func: Callable, xs, initializer, kwargs):
    """fold(lambda s, p: layer(s, *p), zip(Wss, Uss, bss) | enumerate(Wss, Uss, bss), initializer=sequence(s))."""
    if not enabled or _probing() or kwargs or not isinstance(xs, Iterative) or len(xs) == 0:
        return NotImplemented
    seq = initializer
    if not isinstance(seq, FractalTensor) or seq.depth not in (1, 2) or seq.data is None or not seq.data.is_cuda:
        return NotImplemented
    if len(seq.element_shape) != 2 or seq.element_shape[0] != 1:
        return NotImplemented
    H = seq.element_shape[1]
    dtype = seq.data.dtype
    if H % 32 or dtype not in (torch.float32, torch.float16):
        return NotImplemented
    layers = [_lstm_fields(item) for item in xs]
    if any(f is None for f in layers):
        return NotImplemented
    indexed = layers[0][0] is not None
    for f in layers:
        if (f[0] is not None) != indexed or f[1].element_shape[-1] != H or any(p.data.dtype != dtype for p in f[1:]):
            return NotImplemented
    L = len(layers)
    regular = seq.is_regular()
    if seq.depth == 1 and not regular:
        return NotImplemented

    key = ('fold', _fingerprint(func), indexed, L if indexed else 0, H, dtype, seq.depth)
    if key not in _verdicts:
        stats['probes'] += 1
        verdict = None
        try:
            gen = torch.Generator().manual_seed(20240229)
            # without an index the function cannot tell the layers apart except through their parameters
            which = range(L) if indexed else range(1)
            ds = [_probe_lstm_layer(func, xs[l], layers[l], H, dtype, seq.depth, gen) for l in which]
            if all(d is not None for d in ds):
                verdict = {'dilations': ds if indexed else None, 'dilation': ds[0]}
        except Exception:
            verdict = None
        if verdict is None:
            stats['declined'] += 1
        _remember(key, verdict)
    verdict = _verdicts[key]
    if verdict is None:
        return NotImplemented
    dilations = verdict['dilations'] if verdict['dilations'] is not None else [verdict['dilation']] * L
    dilated = any(d != 1 for d in dilations)

    from . import fused
    packed = [_pack_layer(f[1], f[2], f[3]) for f in layers]
    WU = torch.stack([p[0] for p in packed])
    bias = torch.stack([p[1] for p in packed])
    if seq.depth == 1:
        T = len(seq)
        h = _run_lstm(seq.as_dense().reshape(T, 1, H), WU, bias, dilations)
        stats['dilated_lstm' if dilated else 'stacked_lstm'] += 1
        return FractalTensor.from_dense(h.reshape(T, 1, H), 1)
    if not regular and dilated:
        return NotImplemented                   # steps of different widths inside interleaved groups: left to the eager loop
    try:
        dense, sizes = fused.pad_time_major(seq)
    except ValueError:
        return NotImplemented                   # ragged, but not a time-major batch of length-sorted sequences
    h = _run_lstm(dense, WU, bias, dilations, sizes)
    stats['dilated_lstm' if dilated else 'stacked_lstm'] += 1
    return fused.unpad_time_major(h, sizes)


# ------------------------------------------------------------------ blockwise attention behind map

def _attention_operands(xs):
    """zip(qsss, ksss, vsss) -> dense q [B, Hd, nq, rq, D], k, v [B, Hd, nk, rk, D] as views, or None."""
    src = getattr(xs, 'sources', None)
    if not isinstance(xs, Iterative) or src is None or len(src) != 3:
        return None
    for t in src:
        if not isinstance(t, FractalTensor) or t.depth != 3 or t.data is None or not t.data.is_cuda or not t.is_regular():
            return None
        if len(t.element_shape) != 2:
            return None
    q, k, v = (t.as_dense() for t in src)
    if k.shape != v.shape or q.shape[:2] != k.shape[:2] or q.shape[-1] != k.shape[-1] or q.dtype != k.dtype or q.dtype != v.dtype:
        return None
    if q.shape[-1] not in (32, 64, 96, 128):
        return None
    return q, k, v


def _probe_attention(func: Callable, rq: int, rk: int, D: int, gen) -> Optional[float]:
    """The score scale of the program, if func is blockwise softmax(scale * q k^T) v; None otherwise."""
    core = _core()
    nk = 2
    n = nk * rk
    mk = lambda t: FractalTensor.from_dense(t.cuda(), 2)

    def run(q, k, v):      # one sample's item: [heads = 1][blocks] of [rows, D] each
        with _Probe():
            out = func([mk(q.reshape(1, 1, rq, D)), mk(k.reshape(1, nk, rk, D)), mk(v.reshape(1, nk, rk, D))])
        if not isinstance(out, FractalTensor) or out.depth != 2 or out.dense_shape() != (1, 1) or tuple(out.element_shape) != (rq, D):
            return None
        return out.as_dense().reshape(rq, D).float()

    # 1. one non-zero key a, whose value is the first unit vector: out[i, 0] = p_i with logit(p_i) = s q_i.a - log(n - 1)
    q = torch.randn((rq, D), generator=gen)
    a = torch.randn((D,), generator=gen) / D ** 0.5
    k = torch.zeros((n, D)); k[0] = a
    v = torch.zeros((n, D)); v[0, 0] = 1.0
    out = run(q, k, v)
    if out is None:
        return None
    p = out[:, 0].double().cpu()
    if not bool(((p > 0) & (p < 1)).all()) or float(out[:, 1:].abs().max()) > 1e-6:
        return None
    z = torch.log(p * (n - 1) / (1 - p))
    qa = (q.double() @ a.double())
    s = float((z * qa).sum() / (qa * qa).sum())
    if not math.isfinite(s) or s <= 0:
        return None
    for known in (1.0, D ** -0.5):
        if abs(s - known) <= 1e-4 * known:
            s = known
    # 2. a random probe (values that fp16 holds exactly) against the kernel with that scale
    q, k, v = (torch.randn(shape, generator=gen).half().float() for shape in ((rq, D), (n, D), (n, D)))
    out = run(q, k, v)
    if out is None:
        return None
    ref = core.flash_attention(q.half().cuda().reshape(1, 1, rq, D), k.half().cuda().reshape(1, 1, n, D),
                               v.half().cuda().reshape(1, 1, n, D), s).reshape(rq, D)
    return s if _rel_err(out, ref) <= 1e-2 else None


def try_map(func: Callable, xs, kwargs):
    """map(lambda sample: map(per_head, zip(*sample)), zip(qsss, ksss, vsss)): blockwise attention per (sample, head)."""
    if not enabled or _probing() or kwargs:
        return NotImplemented
    ops = _attention_operands(xs)
    if ops is None:
        return NotImplemented
    q, k, v = ops
    if q.dtype != torch.float16 and not (q.dtype == torch.float32 and allow_half_attention):
        return NotImplemented
    B, Hd, nq, rq, D = q.shape
    nk, rk = k.shape[2], k.shape[3]
    key = ('map', _fingerprint(func), rq, rk, D)
    if key not in _verdicts:
        stats['probes'] += 1
        try:
            scale = _probe_attention(func, rq, rk, D, torch.Generator().manual_seed(20240301))
        except Exception:
            scale = None
        if scale is None:
            stats['declined'] += 1
        _remember(key, None if scale is None else {'scale': scale})
    verdict = _verdicts[key]
    if verdict is None:
        return NotImplemented
    core = _core()
    to4 = lambda t: t.reshape(B, Hd, t.shape[2] * t.shape[3], D)
    O = core.flash_attention(to4(q).half().contiguous(), to4(k).half().contiguous(), to4(v).half().contiguous(), verdict['scale'])
    stats['flash_attention'] += 1
    return FractalTensor.from_dense(O.to(q.dtype).view(B, Hd, nq, rq, D), 3)


# ------------------------------------------------------------------ (a @ b) @ c behind Tensor.__matmul__

def _b2b_candidate(t: torch.Tensor) -> bool:
    return t is not None and t.is_cuda and t.dtype == torch.float16 and t.dim() == 2 and t.is_contiguous()


def try_mm(x, y):
    """x @ y: the fused back-to-back GEMM when x is a pending a @ b, a pending product when x @ y could be the
    first half of one, NotImplemented otherwise."""
    if not enabled or _probing() or not isinstance(x, Tensor) or not isinstance(y, Tensor):
        return NotImplemented
    c = y._payload if y._pending is None else None
    if x._pending is not None:
        a, b = x._pending
        if c is None or not _b2b_candidate(c) or c.shape[0] != b.shape[1] or c.shape[1] % 32:
            return NotImplemented                       # mm goes on with torch and forms the pending product on the way
        core = _core()
        K, N, P = a.shape[1], b.shape[1], c.shape[1]
        if core.b2b_gemm_rowmajor_supported(N, K, P):   # b and c as they are
            D = core.b2b_gemm_rowmajor(a[None], b[None], c[None])[0]
        else:                                           # the general kernels take b and c with the contraction index contiguous
            D = core.b2b_gemm(a[None], b.t().contiguous()[None], c.t().contiguous()[None])[0]
        stats['b2b_gemm'] += 1
        return Tensor.from_tensor(D)
    a = x._payload
    b = c
    if not (_b2b_candidate(a) and _b2b_candidate(b)) or a.shape[1] != b.shape[0]:
        return NotImplemented
    if a.shape[1] not in (32, 64, 96, 128) or b.shape[1] % 32 or a.shape[0] < 32:
        return NotImplemented                           # not a first product the fused kernels take
    return Tensor.pending_product(a, b)
