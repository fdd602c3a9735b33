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
  allow_half_attention      route fp32 attention programs to the fp16 kernel instead of the fp32
                            one (off: a routed program never computes in less than its own precision)
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
stats = {'stacked_lstm': 0, 'dilated_lstm': 0, 'lstm_scan': 0, 'flash_attention': 0, 'b2b_gemm': 0, 'gemm': 0, 'probes': 0, 'declined': 0,
         'weight_cache_hits': 0, 'repeated_on_f32_products': 0}

_verdicts: dict = {}
_MAX_VERDICTS = 256
_DEVICE = 'cuda'                       # where routed operands live and probes are built


def _on_device(t: torch.Tensor) -> bool:
    return t.is_cuda
_local = threading.local()


def reset() -> None:
    """Forget every verdict and zero the counters."""
    _verdicts.clear()
    clear_weight_cache()
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


_SCALARS = (int, float, str, bool, bytes, type(None))


def _code_names(code, seen=None):
    """Global names a code object reads, those of the lambdas and functions defined inside it included."""
    names = list(code.co_names)
    for c in code.co_consts:
        if hasattr(c, 'co_names'):
            names.extend(_code_names(c))
    return names


def _fingerprint(f, level: int = 0, seen=None):
    """What identifies a user function between calls (a lambda is a new object at every call of the program, its
    code object is not): its code, its default arguments, the scalars and functions it closes over, and the scalars
    and functions its code reaches through module globals -- so that a layer function, a cell or a scale that is
    redefined at module level under an unchanged caller is a different key.  Other callables (functools.partial,
    callable objects) are keyed on the object itself, which the key then keeps alive; data (tensors) only by kind:
    operand structure is checked on every call."""
    seen = set() if seen is None else seen
    code = getattr(f, '__code__', None)
    if code is None:
        try:
            hash(f)
        except TypeError:
            return ('unhashable', type(f).__name__, id(f))
        return ('object', f)
    if id(f) in seen or level > 6:
        return ('seen', code)
    seen.add(id(f))

    def of_value(v):
        if isinstance(v, _SCALARS):
            return v
        if isinstance(v, (Tensor, FractalTensor, Iterative, torch.Tensor)):
            return type(v).__name__
        if isinstance(v, (tuple, list)) and len(v) <= 16 and all(isinstance(e, _SCALARS) for e in v):
            return tuple(v)
        if callable(v) and hasattr(v, '__code__'):
            return _fingerprint(v, level + 1, seen)
        if isinstance(v, type(os)):                       # a module: its name (ops, torch, math ...)
            return ('module', v.__name__)
        if isinstance(v, type):
            return ('class', v.__module__, v.__qualname__)
        return ('id', type(v).__name__, id(v))

    parts = [code]
    for d in (getattr(f, '__defaults__', None) or ()):
        parts.append(of_value(d))
    for k, d in sorted((getattr(f, '__kwdefaults__', None) or {}).items()):
        parts.append((k, of_value(d)))
    for cell in (getattr(f, '__closure__', None) or ()):
        try:
            parts.append(of_value(cell.cell_contents))
        except ValueError:
            continue
    g = getattr(f, '__globals__', None) or {}
    for name in _code_names(code):
        if name in g:
            v = g[name]
            if isinstance(v, _SCALARS) or (callable(v) and hasattr(v, '__code__')):
                parts.append((name, of_value(v)))
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


# ------------------------------------------------------------------ stacked / dilated LSTM behind fold, map and scan

def _is_gate_params(p, shape) -> bool:
    return (isinstance(p, FractalTensor) and p.depth == 1 and p.data is not None and _on_device(p.data) and p.indices is not None
            and len(p) == 4 and tuple(p.element_shape) == tuple(shape))


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
    if not isinstance(ws, FractalTensor) or len(ws.element_shape) != 2:
        return None
    H = ws.element_shape[-1]
    if not (_is_gate_params(ws, (H, H)) and _is_gate_params(us, (H, H)) and _is_gate_params(bs, (1, H))):
        return None
    return idx, ws, us, bs


def _pack_layer(ws, us, bs):
    """[4] of [H, H], [4] of [H, H], [4] of [1, H] -> WU [2H, 4H] with column blocks i|f|o|candidate, bias [4H]."""
    W, U = ws.as_dense(), us.as_dense()
    H = W.shape[-1]
    WU = torch.cat([W.permute(1, 0, 2).reshape(H, 4 * H), U.permute(1, 0, 2).reshape(H, 4 * H)], dim=0)
    return WU, bs.as_dense().reshape(4 * H)


# Packed weights of the last few routed programs, so that a routed call does not re-pack and re-stack every layer
# (config 4: 67 MB) in front of a 3 ms launch.  A key holds, per parameter tensor, the address and torch's version
# counter (which every in-place torch operation on the buffer or a view of it advances); an entry keeps the source
# buffers alive, so an address cannot come back as another tensor while its entry exists.  Writes that bypass
# torch (a kernel given the raw pointer) are not seen: clear_weight_cache() after such a write.
_weights: dict = {}
_MAX_WEIGHTS = 4
_fading_stacks: set = set()        # packed weights whose last launch on split products met states too small for them


def clear_weight_cache() -> None:
    _weights.clear()
    _fading_stacks.clear()


def _packed_stack(layers):
    """layers: [(idx, ws, us, bs)] -> WU [L, 2H, 4H], bias [L, 4H], cached per parameter identity and version."""
    srcs = [p.data for f in layers for p in f[1:]]
    key = tuple((t.data_ptr(), t._version, t.numel(), t.dtype) for t in srcs)
    hit = _weights.get(key)
    if hit is not None:
        stats['weight_cache_hits'] += 1
        return hit[0], hit[1]
    packed = [_pack_layer(f[1], f[2], f[3]) for f in layers]
    WU = torch.stack([p[0] for p in packed]).contiguous()
    bias = torch.stack([p[1] for p in packed]).contiguous()
    if len(_weights) >= _MAX_WEIGHTS:
        _weights.pop(next(iter(_weights)))
    _weights[key] = (WU, bias, srcs)
    return WU, bias


def _effective(dilations, T: int):
    """A sequence no longer than a layer's dilation is one group, scanned in order (apply_to_each.py:128-129)."""
    return [d if T > d else 1 for d in dilations]


def _run_lstm(xs: torch.Tensor, WU: torch.Tensor, bias: torch.Tensor, dilations, active=None, both: bool = False):
    """xs [T, B, H] -> the last layer's h [T, B, H] (with `both`: its h and c), through the kernel of the operands' type."""
    core = _core()
    eff = _effective(dilations, xs.shape[0])
    dil = None if all(d == 1 for d in eff) else eff
    if xs.dtype == torch.float16:
        hsss, csss = core.stacked_lstm_f16(xs.contiguous(), WU.contiguous(), bias.float().contiguous(), dilations=dil, active_rows=active)
    else:
        # A program's every layer is accurate relative to its own size: a stack whose hidden states fall below what
        # the split products' planes resolve is computed again on fp32 products, and goes there directly next time.
        key = (WU.data_ptr(), WU._version)
        counter = 'stacked_lstm_repeated_on_f32_products'
        before = core.launch_counts.get(counter, 0)
        hsss, csss = core.stacked_lstm(xs.contiguous(), WU.contiguous(), bias.contiguous(), dilations=dil, active_rows=active,
                                       products='f32' if key in _fading_stacks else None, exact_small_states=True)
        if core.launch_counts.get(counter, 0) != before:
            if len(_fading_stacks) >= 64:
                _fading_stacks.clear()
            _fading_stacks.add(key)
            stats['repeated_on_f32_products'] += 1
    return (hsss[-1], csss[-1]) if both else hsss[-1]


def _run_batch_major(flat: torch.Tensor, lengths, WU, bias, dilations, both: bool = False):
    """Sequences stored one after the other (flat [sum(lengths), H], sample b owning lengths[b] consecutive rows),
    each scanned on its own from a zero state: the time-major batch the kernels take is built on the device -- a
    transpose when all lengths agree, otherwise the samples sorted by length (longest first, the ragged form of
    examples/utils/data_utils.py:42-66) and padded with zero rows -- and the result is put back in the order it
    came in.  Samples whose lengths make a dilation act differently (a sequence no longer than the dilation is
    scanned in order) go down as launches of their own.  Returns h [sum(lengths), H] (with `both`: h and c), and
    the number of launches."""
    B, H = len(lengths), flat.shape[-1]
    outs = [torch.empty_like(flat) for _ in range(2 if both else 1)]
    groups: dict = {}
    for b, n in enumerate(lengths):
        groups.setdefault(tuple(_effective(dilations, n)), []).append(b)
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    launches = 0
    for eff, members in groups.items():
        lens = [lengths[b] for b in members]
        T, Bg = max(lens), len(members)
        if len(groups) == 1 and min(lens) == T:                      # regular: [B, T, H] -> [T, B, H]
            res = _run_lstm(flat.view(B, T, H).transpose(0, 1).contiguous(), WU, bias, list(eff), None, both)
            for o, r in zip(outs, res if both else (res,)):
                o.view(B, T, H).copy_(r.transpose(0, 1))
            launches += 1
            continue
        order = sorted(range(Bg), key=lambda j: -lens[j])            # stable: longest first
        import numpy as np
        N = flat.shape[0]
        gather = np.full((T, Bg), N, dtype=np.int64)                # N: the zero row appended below
        for col, j in enumerate(order):
            n = lens[j]
            gather[:n, col] = offs[members[j]] + np.arange(n)
        live = gather < N
        active = live.sum(axis=1).tolist()
        gidx = torch.from_numpy(gather.reshape(-1)).to(flat.device)
        padded = torch.cat([flat, flat.new_zeros((1, H))]).index_select(0, gidx).view(T, Bg, H)
        res = _run_lstm(padded, WU, bias, list(eff), None if min(lens) == T else active, both)
        src = torch.from_numpy(np.nonzero(live.reshape(-1))[0]).to(flat.device)        # places of the padded batch that hold a row
        dst = gidx.index_select(0, src)                                                  # the row of `flat` each of them is
        for o, r in zip(outs, res if both else (res,)):
            o.index_copy_(0, dst, r.reshape(T * Bg, H).index_select(0, src))
        launches += 1
    return (outs if both else outs[0]), launches


def _rows_to_batch_major(rows: torch.Tensor, lengths) -> FractalTensor:
    """rows [sum(lengths), H] -> depth-2 [B][T_b] of [1, H]."""
    H = rows.shape[-1]
    if len(set(lengths)) == 1:
        return FractalTensor.from_dense(rows.view(len(lengths), lengths[0], 1, H), 2)
    proto = FractalTensor.from_dense(rows[:1].view(1, 1, 1, H), 2)
    ft = FractalTensor(proto._type.dtype)
    ft.indices = [list(range(n)) for n in lengths]
    ft.data = rows
    return ft


def _probe_lstm_layer(func: Callable, item, fields, H: int, dtype, seq_depth: int, gen):
    """Runs func on a probe sequence with this layer's own parameters.  Returns (dilation it asked for (1 if none),
    layout) when the result equals the fused layer's, else None.  layout: 'time' (a depth-2 operand is [T][B]),
    'batch' (it is [B][T]: every sample scanned on its own), 'single' (depth 1)."""
    _, ws, us, bs = fields
    WU, bias = _pack_layer(ws, us, bs)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    n0, n1 = (3, 4) if seq_depth == 2 else (3, 1)
    for _ in range(2):                                     # second pass: a probe longer than the dilation just seen
        x = torch.randn((n0, n1, 1, H), generator=gen)
        if n1 > 1:
            x[:, n1 - 1] *= 4.0                            # one row of larger magnitude: saturated gates are probed too
        else:
            x[n0 - 1] *= 4.0
        x = x.to(device=_DEVICE, dtype=dtype)
        probe = FractalTensor.from_dense(x, 2) if seq_depth == 2 else FractalTensor.from_dense(x[:, 0], 1)
        with _Probe() as p:
            out = func(probe, item)
        asked = set(p.dilations)
        if len(asked) > 1 or not isinstance(out, FractalTensor) or out.depth != seq_depth or not out.is_regular():
            return None
        d = asked.pop() if asked else 1
        if d < 1:
            return None
        if d >= min(n0, n1) and (seq_depth == 2 or d >= n0):    # the recurrence did not show yet
            n0, n1 = (d + 2, d + 3) if seq_depth == 2 else (d + 2, 1)
            continue
        got = out.as_dense().reshape(-1, H)
        if got.shape[0] != n0 * n1:
            return None
        got = got.view(n0, n1, H)
        xs = x.reshape(n0, n1, H)
        if _rel_err(got, _run_lstm(xs, WU[None], bias[None], [d])) <= tol:
            return d, ('time' if seq_depth == 2 else 'single')
        if seq_depth == 2:
            ref = _run_lstm(xs.transpose(0, 1).contiguous(), WU[None], bias[None], [d]).transpose(0, 1)
            if _rel_err(got, ref) <= tol:
                return d, 'batch'
        return None
    return None


def _match_fold(xs, H: int, dtype):
    """The fold items as LSTM layers [(idx, ws, us, bs)] of hidden size H and type dtype, or None."""
    if not isinstance(xs, Iterative) or len(xs) == 0:
        return None
    layers = [_lstm_fields(item) for item in xs]
    if any(f is None for f in layers):
        return None
    indexed = layers[0][0] is not None
    for f in layers:
        if (f[0] is not None) != indexed or f[1].element_shape[-1] != H or any(p.data.dtype != dtype for p in f[1:]):
            return None
    return layers


def _fold_verdict(func: Callable, xs, layers, H: int, dtype, seq_depth: int):
    """{'dilations': per layer, 'layout': ...} if func has been seen to compute an LSTM layer on every probed item, else None."""
    indexed = layers[0][0] is not None
    L = len(layers)
    key = ('fold', _fingerprint(func), indexed, L if indexed else 0, H, dtype, seq_depth)
    if key not in _verdicts:
        stats['probes'] += 1
        verdict = None
        try:
            gen = torch.Generator().manual_seed(20240229)
            # without an index the function cannot tell the layers apart except through their parameters
            which = range(L) if indexed else range(1)
            seen = [_probe_lstm_layer(func, xs[l], layers[l], H, dtype, seq_depth, gen) for l in which]
            if all(v is not None for v in seen) and len({v[1] for v in seen}) == 1:
                verdict = {'dilations': [v[0] for v in seen] if indexed else None, 'dilation': seen[0][0], 'layout': seen[0][1]}
        except Exception:
            verdict = None
        if verdict is None:
            stats['declined'] += 1
        _remember(key, verdict)
    verdict = _verdicts[key]
    if verdict is None:
        return None
    dilations = verdict['dilations'] if verdict['dilations'] is not None else [verdict['dilation']] * L
    return {'dilations': dilations, 'layout': verdict['layout']}


def _sequence_operand(seq, depths=(1, 2)):
    """(H, dtype) of a GPU FractalTensor of [1, H] rows that the LSTM kernels take, else None."""
    if not isinstance(seq, FractalTensor) or seq.depth not in depths or seq.data is None or not _on_device(seq.data) or seq.indices is None:
        return None
    if len(seq.element_shape) != 2 or seq.element_shape[0] != 1:
        return None
    H, dtype = seq.element_shape[1], seq.data.dtype
    if H % 32 or dtype not in (torch.float32, torch.float16):
        return None
    return H, dtype


class _Deferred:
    """Stands for the result of a fold or scan that was recorded instead of run (see _Capture)."""

    def __init__(self, kind, func, xs, initializer, fields: int):
        self.kind, self.func, self.xs, self.initializer = kind, func, xs, initializer
        self.fields = [_DeferredField(self, i) for i in range(fields)]

    def __iter__(self):
        return iter(self.fields)

    def __len__(self):
        return len(self.fields)

    def __getitem__(self, i):
        return self.fields[i]


class _DeferredField:
    def __init__(self, parent, i):
        self.parent, self.i = parent, i


class _Capture:
    """While a map looks at what its function does with one item, a fold or scan over LSTM-shaped operands inside it
    is recorded and answered with a placeholder instead of being run.  If the function hands that placeholder back
    untouched, the map is a batch of such folds / scans and runs as one launch."""

    def __enter__(self):
        self.saved = getattr(_local, 'capture', None)
        _local.capture = []
        return self

    def __exit__(self, *exc):
        self.calls = _local.capture
        _local.capture = self.saved
        return False


def _capturing():
    return getattr(_local, 'capture', None)


def try_fold(func: Callable, xs, initializer, kwargs):
    """fold(lambda s, p: layer(s, *p), zip(Wss, Uss, bss) | enumerate(Wss, Uss, bss), initializer=sequence(s))."""
    if not enabled or _probing() or kwargs:
        return NotImplemented
    seq = initializer
    op = _sequence_operand(seq)
    if op is None:
        return NotImplemented
    H, dtype = op
    layers = _match_fold(xs, H, dtype)
    if layers is None:
        return NotImplemented
    cap = _capturing()
    if cap is not None:
        if seq.depth != 1:
            return NotImplemented
        cap.append(_Deferred('fold', func, xs, seq, 0))
        return cap[-1]
    regular = seq.is_regular()
    if seq.depth == 1 and not regular:
        return NotImplemented
    verdict = _fold_verdict(func, xs, layers, H, dtype, seq.depth)
    if verdict is None:
        return NotImplemented
    dilations = verdict['dilations']
    dilated = any(d != 1 for d in dilations)
    name = 'dilated_lstm' if dilated else 'stacked_lstm'

    from . import fused
    if seq.depth == 1:
        WU, bias = _packed_stack(layers)
        T = len(seq)
        h = _run_lstm(seq.as_dense().reshape(T, 1, H), WU, bias, dilations)
        stats[name] += 1
        return FractalTensor.from_dense(h.reshape(T, 1, H), 1)
    if verdict['layout'] == 'batch':                 # [B][T_b]: every sample scanned on its own (stacked_lstm1.py:40-76)
        lengths = [len(sample) for sample in seq.indices]
        if min(lengths) <= 0:
            return NotImplemented
        WU, bias = _packed_stack(layers)
        h, launches = _run_batch_major(seq.data.view(-1, H), lengths, WU, bias, dilations)
        stats[name] += launches
        return _rows_to_batch_major(h, lengths)
    if not regular and dilated:
        return NotImplemented                   # steps of different widths inside interleaved groups: left to the eager loop
    try:
        dense, sizes = fused.pad_time_major(seq)
    except ValueError:
        return NotImplemented                   # ragged, but not a time-major batch of length-sorted sequences
    WU, bias = _packed_stack(layers)
    h = _run_lstm(dense, WU, bias, dilations, sizes)
    stats[name] += 1
    return fused.unpad_time_major(h, sizes)


# ---- one layer written as a scan over time (stacked_rnn.py:54-65; per sample: stacked_lstm1.py:40-51)

def _closure_values(f, level: int = 0, seen=None):
    """Values a function closes over, holds as defaults or (FractalTensors only) reads from its module's globals,
    those of the functions it closes over included."""
    seen = set() if seen is None else seen
    if id(f) in seen or level > 3:
        return
    seen.add(id(f))
    vals = list(getattr(f, '__defaults__', None) or ())
    for cell in (getattr(f, '__closure__', None) or ()):
        try:
            vals.append(cell.cell_contents)
        except ValueError:
            pass
    code, g = getattr(f, '__code__', None), getattr(f, '__globals__', None) or {}
    if code is not None:                                   # parameters held at module level count as well
        vals.extend(g[n] for n in _code_names(code) if isinstance(g.get(n), FractalTensor))
    for v in vals:
        if callable(v) and hasattr(v, '__code__'):
            yield from _closure_values(v, level + 1, seen)
        else:
            yield v


def _scan_parameters(func: Callable, H: int, dtype):
    """The gate parameters a step function closes over: ([H,H] x 4, [H,H] x 4, [1,H] x 4) FractalTensors, the two
    square ones in the order found (which of them multiplies x is settled by the probe).  None unless there is
    exactly one such set."""
    square, rows = [], []
    for v in _closure_values(func):
        if _is_gate_params(v, (H, H)) and v.data.dtype == dtype and not any(v is s for s in square):
            square.append(v)
        elif _is_gate_params(v, (1, H)) and v.data.dtype == dtype and not any(v is r for r in rows):
            rows.append(v)
    if len(square) != 2 or len(rows) != 1:
        return None
    return square[0], square[1], rows[0]


def _scan_state(initializer, depth: int, H: int, dtype):
    """(h0, c0) as [B, H] tensors if the initializer is the LSTM state of a scan over a depth-`depth` operand."""
    if not isinstance(initializer, (tuple, list)) or len(initializer) != 2:
        return None
    out = []
    for s in initializer:
        if depth == 1:
            if not isinstance(s, Tensor) or tuple(s.shape) != (1, H) or not _on_device(s.data) or s.data.dtype != dtype:
                return None
            out.append(s.data.reshape(1, H))
        else:
            if _sequence_operand(s, (1,)) != (H, dtype) or not s.is_regular():
                return None
            out.append(s.as_dense().reshape(-1, H))
    return out if out[0].shape == out[1].shape else None


def _probe_scan(func: Callable, params, H: int, dtype, depth: int, gen):
    """Which of the two square parameter sets multiplies x (0 or 1) if the step function is an LSTM cell over them."""
    from .functional import scan as eager_scan
    T, B = 4, (3 if depth == 2 else 1)
    x = torch.randn((T, B, 1, H), generator=gen)
    x[:, B - 1] *= 4.0
    x = x.to(device=_DEVICE, dtype=dtype)
    zero = lambda: torch.zeros((B, 1, H), device=_DEVICE, dtype=dtype)
    if depth == 2:
        probe, init = FractalTensor.from_dense(x, 2), (FractalTensor.from_dense(zero(), 1), FractalTensor.from_dense(zero(), 1))
    else:
        probe, init = FractalTensor.from_dense(x[:, 0], 1), (Tensor.from_tensor(zero()[0]), Tensor.from_tensor(zero()[0]))
    with _Probe():
        out = eager_scan(func, probe, initializer=init)
    if not isinstance(out, list) or len(out) != 2 or any(not isinstance(o, FractalTensor) or not o.is_regular() for o in out):
        return None
    got = [o.as_dense().reshape(-1, H) for o in out]
    if any(g.shape[0] != T * B for g in got):
        return None
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for first in (0, 1):
        WU, bias = _pack_layer(params[first], params[1 - first], params[2])
        h, c = _run_lstm(x.reshape(T, B, H), WU[None], bias[None], [1], both=True)
        if _rel_err(got[0], h.reshape(-1, H)) <= tol and _rel_err(got[1], c.reshape(-1, H)) <= tol:
            return first
    return None


def try_scan(func: Callable, xs, initializer, kwargs):
    """scan(lambda state, x: cell(*state, x, ws, us, bs), sequence(s), initializer=(h0, c0)) -> [hs, cs]."""
    if not enabled or _probing() or kwargs or initializer is None:
        return NotImplemented
    op = _sequence_operand(xs)
    if op is None:
        return NotImplemented
    H, dtype = op
    state = _scan_state(initializer, xs.depth, H, dtype)
    if state is None:
        return NotImplemented
    params = _scan_parameters(func, H, dtype)
    if params is None:
        return NotImplemented
    cap = _capturing()
    if cap is not None:
        if xs.depth != 1:
            return NotImplemented
        cap.append(_Deferred('scan', func, xs, initializer, 2))
        return cap[-1]
    key = ('scan', _fingerprint(func), H, dtype, xs.depth)
    if key not in _verdicts:
        stats['probes'] += 1
        try:
            first = _probe_scan(func, params, H, dtype, xs.depth, torch.Generator().manual_seed(20240302))
        except Exception:
            first = None
        if first is None:
            stats['declined'] += 1
        _remember(key, None if first is None else {'x_first': first})
    verdict = _verdicts[key]
    if verdict is None:
        return NotImplemented
    first = verdict['x_first']
    layers = [(None, params[first], params[1 - first], params[2])]
    from . import fused
    if xs.depth == 1:
        if not xs.is_regular():
            return NotImplemented
        T, sizes = len(xs), None
        dense = xs.as_dense().reshape(T, 1, H)
    else:
        try:
            dense, sizes = fused.pad_time_major(xs)
        except ValueError:
            return NotImplemented
    if state[0].shape[0] != dense.shape[1]:
        return NotImplemented
    WU, bias = _packed_stack(layers)
    zero_state = not bool(torch.count_nonzero(state[0])) and not bool(torch.count_nonzero(state[1]))
    if zero_state:
        h, c = _run_lstm(dense, WU, bias, [1], sizes, both=True)
    elif sizes is None:                                    # a layer that goes on from a given state: one fused cell per step
        h, c = _core().lstm_layer(dense.contiguous(), WU[0], bias[0].float(), state[0].contiguous(), state[1].contiguous())
    else:
        return NotImplemented
    stats['lstm_scan'] += 1
    if xs.depth == 1:
        return [FractalTensor.from_dense(t.reshape(T, 1, H), 1) for t in (h, c)]
    return [fused.unpad_time_major(t, sizes) for t in (h, c)]


# ---- a map over samples whose function is one fold / scan of the sample (dilated_rnn.py:39-41, stacked_lstm1.py:60-62)

def _captured_program(func: Callable, sample):
    """What func does with one sample, if that is exactly one recorded fold or scan of the sample whose result it
    returns as it is: (deferred, which fields it returns, whether as a tuple), else None."""
    with _Capture() as cap:
        try:
            ret = func(sample)
        except Exception:
            return None
    if len(cap.calls) != 1:
        return None
    d = cap.calls[0]
    seq = d.initializer if d.kind == 'fold' else d.xs
    if seq is not sample:
        return None
    if ret is d:
        return d, None, False
    if isinstance(ret, _DeferredField) and ret.parent is d:
        return d, [ret.i], False
    if isinstance(ret, (tuple, list)) and ret and all(isinstance(r, _DeferredField) and r.parent is d for r in ret):
        return d, [r.i for r in ret], True
    return None


def _try_map_of_sequences(func: Callable, xs):
    """map(lambda sample: fold(layer, params, initializer=sample) | scan(cell, sample, initializer=state), samples)
    over a GPU batch [B][T_b] of [1, H]: all samples in one launch."""
    op = _sequence_operand(xs, (2,))
    if op is None or len(xs) == 0 or min(len(s) for s in xs.indices) <= 0:
        return NotImplemented
    H, dtype = op
    key = ('map-of', _fingerprint(func), H, dtype)
    if _verdicts.get(key, True) is None:
        return NotImplemented                              # seen before: not a fold / scan of the sample
    B = len(xs)
    first, last = xs[0], xs[B - 1]
    prog = _captured_program(func, first)
    other = _captured_program(func, last) if prog is not None else None
    same = (prog is not None and other is not None and prog[1:] == other[1:] and prog[0].kind == other[0].kind
            and _fingerprint(prog[0].func) == _fingerprint(other[0].func))
    if same and prog[0].kind == 'fold':
        same = prog[0].xs is other[0].xs                   # the same parameters for every sample
    if not same:
        _remember(key, None)
        return NotImplemented
    d, fields, as_tuple = prog
    lengths = [len(s) for s in xs.indices]
    flat = xs.data.view(-1, H)
    if d.kind == 'fold':
        layers = _match_fold(d.xs, H, dtype)
        verdict = None if layers is None else _fold_verdict(d.func, d.xs, layers, H, dtype, 1)
        if verdict is None or verdict['layout'] != 'single':
            return NotImplemented
        WU, bias = _packed_stack(layers)
        h, launches = _run_batch_major(flat, lengths, WU, bias, verdict['dilations'])
        stats['dilated_lstm' if any(v != 1 for v in verdict['dilations']) else 'stacked_lstm'] += launches
        return _rows_to_batch_major(h, lengths)
    # scan: the state every sample starts from must be zero (one launch cannot start rows from different states here)
    states = [_scan_state(p[0].initializer, 1, H, dtype) for p in (prog, other)]
    if any(s is None or bool(torch.count_nonzero(s[0])) or bool(torch.count_nonzero(s[1])) for s in states):
        return NotImplemented
    params = _scan_parameters(d.func, H, dtype)
    if params is None:
        return NotImplemented
    skey = ('scan', _fingerprint(d.func), H, dtype, 1)
    if skey not in _verdicts:
        stats['probes'] += 1
        try:
            x_first = _probe_scan(d.func, params, H, dtype, 1, torch.Generator().manual_seed(20240302))
        except Exception:
            x_first = None
        if x_first is None:
            stats['declined'] += 1
        _remember(skey, None if x_first is None else {'x_first': x_first})
    if _verdicts[skey] is None:
        return NotImplemented
    x_first = _verdicts[skey]['x_first']
    WU, bias = _packed_stack([(None, params[x_first], params[1 - x_first], params[2])])
    (h, c), launches = _run_batch_major(flat, lengths, WU, bias, [1], both=True)
    stats['lstm_scan'] += launches
    outs = [_rows_to_batch_major(t, lengths) for t in (h, c)]
    if fields is None:
        return outs
    picked = [outs[i] for i in fields]
    return picked if as_tuple else picked[0]


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


def _probe_attention(func: Callable, rq: int, rk: int, D: int, gen, dtype=torch.float16) -> Optional[float]:
    """The score scale of the program, if func is blockwise softmax(scale * q k^T) v; None otherwise.  The probe runs
    in the program's own element type against the kernel of that type (1e-2 for fp16, 1e-4 for fp32)."""
    core = _core()
    nk = 2
    n = nk * rk
    mk = lambda t: FractalTensor.from_dense(t.to(device='cuda', dtype=dtype), 2)

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
    if dtype == torch.float32:
        ref = core.flash_attention_f32(q.cuda().reshape(1, 1, rq, D), k.cuda().reshape(1, 1, n, D), v.cuda().reshape(1, 1, n, D), s)
        return s if _rel_err(out, ref.reshape(rq, D)) <= 1e-4 else None
    ref = core.flash_attention(q.half().cuda().reshape(1, 1, rq, D), k.half().cuda().reshape(1, 1, n, D),
                               v.half().cuda().reshape(1, 1, n, D), s).reshape(rq, D)
    return s if _rel_err(out, ref) <= 1e-2 else None


def try_map(func: Callable, xs, kwargs):
    """map(lambda sample: map(per_head, zip(*sample)), zip(qsss, ksss, vsss)): blockwise attention per (sample, head)."""
    if not enabled or _probing() or kwargs:
        return NotImplemented
    if _capturing() is not None:
        return NotImplemented
    if isinstance(xs, FractalTensor):
        return _try_map_of_sequences(func, xs)
    ops = _attention_operands(xs)
    if ops is None:
        return NotImplemented
    q, k, v = ops
    if q.dtype not in (torch.float16, torch.float32):
        return NotImplemented
    B, Hd, nq, rq, D = q.shape
    nk, rk = k.shape[2], k.shape[3]
    key = ('map', _fingerprint(func), rq, rk, D, q.dtype)
    if key not in _verdicts:
        stats['probes'] += 1
        try:
            scale = _probe_attention(func, rq, rk, D, torch.Generator().manual_seed(20240301), q.dtype)
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
    if q.dtype == torch.float32 and not allow_half_attention:       # a program computes in its own precision
        O = core.flash_attention_f32(to4(q).contiguous(), to4(k).contiguous(), to4(v).contiguous(), verdict['scale'])
    else:
        O = core.flash_attention(to4(q).half().contiguous(), to4(k).half().contiguous(), to4(v).half().contiguous(), verdict['scale'])
    stats['flash_attention'] += 1
    return FractalTensor.from_dense(O.to(q.dtype).view(B, Hd, nq, rq, D), 3)


# ------------------------------------------------------------------ (a @ b) @ c behind Tensor.__matmul__

def _b2b_candidate(t: torch.Tensor) -> bool:
    return t is not None and t.is_cuda and t.dtype == torch.float16 and t.dim() == 2 and t.is_contiguous()


_cu_count: dict = {}


def _try_own_gemm(a: torch.Tensor, b: torch.Tensor):
    """a @ b through the library's product kernel (ftk_gemm_f16) where it is the faster of the two: N a multiple of 256,
    K of 32, and at least one 256 x 256 output tile per compute unit; NotImplemented (torch's product) otherwise."""
    M, K = a.shape
    N = b.shape[1]
    if N % 256 or K % 32 or M < 1:
        return NotImplemented
    dev = a.device.index if a.device.index is not None else torch.cuda.current_device()
    if dev not in _cu_count:
        _cu_count[dev] = torch.cuda.get_device_properties(dev).multi_processor_count
    if -(-M // 256) * (N // 256) < _cu_count[dev]:
        return NotImplemented
    stats['gemm'] += 1
    return Tensor.from_tensor(_core().gemm(a, b))


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
        elif core.b2b_gemm_supported(N, K, P):          # the general kernels take b and c with the contraction index contiguous
            D = core.b2b_gemm(a[None], b.t().contiguous()[None], c.t().contiguous()[None])[0]
        else:
            return NotImplemented                       # a shape no fused kernel takes: two torch products, as before
        stats['b2b_gemm'] += 1
        return Tensor.from_tensor(D)
    a = x._payload
    b = c
    if not (_b2b_candidate(a) and _b2b_candidate(b)) or a.shape[1] != b.shape[0]:
        return NotImplemented
    if a.shape[1] not in (32, 64, 96, 128) or b.shape[1] % 32 or a.shape[0] < 32:
        return _try_own_gemm(a, b)                      # not a first product the fused kernels take
    if not _core().b2b_gemm_supported(b.shape[1], a.shape[1], 32):
        return NotImplemented                           # N beyond what any of the kernels holds (whatever P turns out to be)
    return Tensor.pending_product(a, b)
