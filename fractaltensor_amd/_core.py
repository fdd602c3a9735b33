"""ctypes binding of libftkernels.so, the C ABI declared in include/ftk.h.

This is the only place the package touches native code.  The library is
required: importing this module without a built libftkernels.so raises, and
no function here has a CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libftkernels.so')

# every symbol include/ftk.h declares; checked at load time
EXPORTS = (
    'ftk_version', 'ftk_last_error', 'ftk_device_info_query',
    'ftk_lstm_cell_f32', 'ftk_lstm_cell_f16', 'ftk_lstm_layer_f32', 'ftk_lstm_layer_f16', 'ftk_lstm_elementwise_f32',
    'ftk_stacked_lstm_workspace_bytes', 'ftk_stacked_lstm_f32', 'ftk_dilated_lstm_f32',
    'ftk_stacked_lstm_wavefront_f32', 'ftk_stacked_lstm_ragged_f32', 'ftk_lstm_set_products', 'ftk_lstm_get_products',
    'ftk_stacked_lstm_opts_f32', 'ftk_stacked_lstm_status', 'ftk_stacked_lstm_small_states', 'ftk_stacked_lstm_noalloc_f32',
    'ftk_stacked_lstm_f16_workspace_bytes', 'ftk_stacked_lstm_f16',
    'ftk_b2b_gemm_f16', 'ftk_b2b_gemm_f16_supported', 'ftk_b2b_gemm_rowmajor_f16', 'ftk_gemm_f16', 'ftk_batched_gemm_f16', 'ftk_flash_attn_f16', 'ftk_flash_attn_f16_workspace_bytes', 'ftk_flash_attn_ws_f16', 'ftk_flash_attn_f32_workspace_bytes', 'ftk_flash_attn_f32', 'ftk_online_softmax_f32', 'ftk_embedding_gather_f32',
    'ftk_grid_rnn_workspace_bytes', 'ftk_grid_rnn_f32', 'ftk_windowed_attn_f32',
)


class FtkError(RuntimeError):
    """A non-zero return from the C ABI; carries the code and ftk_last_error()."""

    def __init__(self, code: int, message: str):
        super().__init__(f'libftkernels error {code}: {message}')
        self.code = code


class LstmOptions(ctypes.Structure):
    """ftk_lstm_options of include/ftk.h."""
    _fields_ = [('products', ctypes.c_int), ('spin_limit', ctypes.c_int)]


class DeviceInfo(ctypes.Structure):
    _fields_ = [('compute_units', ctypes.c_int), ('lds_bytes_per_block', ctypes.c_int),
                ('clock_khz', ctypes.c_int), ('wavefront_size', ctypes.c_int),
                ('persistent_slots', ctypes.c_int), ('arch', ctypes.c_char * 32)]


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f'{LIB_PATH} is missing: build it with `make -C fractaltensor_amd/csrc` '
            '(or __graft_entry__.build()); there is no fallback path')
    lib = ctypes.CDLL(LIB_PATH)
    for name in EXPORTS:
        if not hasattr(lib, name):
            raise ImportError(f'{LIB_PATH} does not export {name}')
    lib.ftk_version.restype = ctypes.c_int
    lib.ftk_last_error.restype = ctypes.c_char_p
    lib.ftk_stacked_lstm_workspace_bytes.restype = ctypes.c_size_t
    lib.ftk_stacked_lstm_workspace_bytes.argtypes = [ctypes.c_int] * 4
    lib.ftk_stacked_lstm_f16_workspace_bytes.restype = ctypes.c_size_t
    lib.ftk_stacked_lstm_f16_workspace_bytes.argtypes = [ctypes.c_int] * 4
    lib.ftk_grid_rnn_workspace_bytes.restype = ctypes.c_size_t
    lib.ftk_grid_rnn_workspace_bytes.argtypes = [ctypes.c_int] * 2
    lib.ftk_flash_attn_f32_workspace_bytes.restype = ctypes.c_size_t
    lib.ftk_flash_attn_f32_workspace_bytes.argtypes = [ctypes.c_int] * 5
    lib.ftk_flash_attn_f16_workspace_bytes.restype = ctypes.c_size_t
    lib.ftk_flash_attn_f16_workspace_bytes.argtypes = [ctypes.c_int] * 5
    for name in EXPORTS:
        if name not in ('ftk_last_error', 'ftk_stacked_lstm_workspace_bytes', 'ftk_stacked_lstm_f16_workspace_bytes', 'ftk_grid_rnn_workspace_bytes',
                        'ftk_flash_attn_f32_workspace_bytes', 'ftk_flash_attn_f16_workspace_bytes'):
            getattr(lib, name).restype = ctypes.c_int
    return lib


lib = _load()


def _check(rc: int) -> None:
    if rc != 0:
        raise FtkError(rc, lib.ftk_last_error().decode('utf-8', 'replace'))


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _req(t: torch.Tensor, dtype, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f'{name} must be a torch.Tensor')
    if not t.is_cuda:
        raise RuntimeError(f'{name} must live on the GPU (got {t.device}); there is no CPU path')
    if t.dtype != dtype:
        raise TypeError(f'{name} must be {dtype}, got {t.dtype}')
    if not t.is_contiguous():
        raise ValueError(f'{name} must be contiguous')
    return t


def _req_out(t: torch.Tensor, dtype, shape, name: str) -> torch.Tensor:
    """A caller-supplied output: the kernels write the full shape, so anything smaller would be overrun."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f'{name} must be a torch.Tensor')
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f'{name} must be {tuple(shape)}, got {tuple(t.shape)}')
    return _req(t, dtype, name)


def _req_workspace(t: torch.Tensor) -> torch.Tensor:
    if not isinstance(t, torch.Tensor) or not t.is_cuda or not t.is_contiguous():
        raise ValueError('workspace must be a contiguous CUDA tensor')
    return t


# calls of the fused entry points made through this binding, by name (what routed an operator program here)
launch_counts: dict = {}


def _count(name: str) -> None:
    launch_counts[name] = launch_counts.get(name, 0) + 1


def version() -> int:
    return lib.ftk_version()


def device_info() -> DeviceInfo:
    info = DeviceInfo()
    _check(lib.ftk_device_info_query(ctypes.byref(info)))
    return info


def lstm_cell(x, h_prev, c_prev, WU, bias=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Fused cell: x [B,I], h_prev/c_prev [B,H] or None, WU [(I+H),4H], bias [4H] or None."""
    f32 = torch.float32
    _req(x, f32, 'x'); _req(WU, f32, 'WU')
    B, I = x.shape
    H = WU.shape[1] // 4
    if WU.shape != (I + H, 4 * H):
        raise ValueError(f'WU must be [(I+H), 4H] = [{I + H}, {4 * H}], got {tuple(WU.shape)}')
    for t, n in ((h_prev, 'h_prev'), (c_prev, 'c_prev')):
        if t is not None and _req(t, f32, n).shape != (B, H):
            raise ValueError(f'{n} must be [{B}, {H}]')
    if bias is not None and _req(bias, f32, 'bias').numel() != 4 * H:
        raise ValueError('bias must have 4H elements')
    h = torch.empty((B, H), dtype=f32, device=x.device)
    c = torch.empty((B, H), dtype=f32, device=x.device)
    _check(lib.ftk_lstm_cell_f32(_ptr(x), _ptr(h_prev), _ptr(c_prev), _ptr(WU), _ptr(bias), _ptr(h), _ptr(c),
                                 ctypes.c_int(B), ctypes.c_int(I), ctypes.c_int(H), _stream()))
    return h, c


def lstm_layer(xs, WU, bias=None, h0=None, c0=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """One layer over T steps from an initial state: xs [T,B,I], WU [(I+H),4H], bias [4H] or None, h0/c0 [B,H] or
    None (zero state) -> hs, cs [T,B,H].  fp32 throughout, or fp16 storage (bias fp32) when xs is fp16."""
    dt = xs.dtype
    if dt not in (torch.float32, torch.float16):
        raise TypeError('xs must be float32 or float16')
    _req(xs, dt, 'xs'); _req(WU, dt, 'WU')
    T, B, I = xs.shape
    H = WU.shape[1] // 4
    if WU.shape != (I + H, 4 * H):
        raise ValueError(f'WU must be [(I+H), 4H] = [{I + H}, {4 * H}], got {tuple(WU.shape)}')
    for t, n in ((h0, 'h0'), (c0, 'c0')):
        if t is not None and _req(t, dt, n).shape != (B, H):
            raise ValueError(f'{n} must be [{B}, {H}]')
    if bias is not None and _req(bias, torch.float32, 'bias').numel() != 4 * H:
        raise ValueError('bias must have 4H elements')
    hs = torch.empty((T, B, H), dtype=dt, device=xs.device)
    cs = torch.empty((T, B, H), dtype=dt, device=xs.device)
    fn = lib.ftk_lstm_layer_f32 if dt == torch.float32 else lib.ftk_lstm_layer_f16
    ci = ctypes.c_int
    _check(fn(_ptr(xs), _ptr(WU), _ptr(bias), _ptr(h0), _ptr(c0), _ptr(hs), _ptr(cs), ci(T), ci(B), ci(I), ci(H), _stream()))
    return hs, cs


def lstm_cell_f16(x, h_prev, c_prev, WU, bias=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """The fused cell with fp16 storage: x [B,I], h_prev/c_prev [B,H] or None, WU [(I+H),4H] fp16, bias [4H]
    fp32 or None; I and H multiples of 32.  Gate sums in fp32, h and c rounded to fp16 when written."""
    f16 = torch.float16
    _req(x, f16, 'x'); _req(WU, f16, 'WU')
    B, I = x.shape
    H = WU.shape[1] // 4
    if WU.shape != (I + H, 4 * H):
        raise ValueError(f'WU must be [(I+H), 4H] = [{I + H}, {4 * H}], got {tuple(WU.shape)}')
    for t, n in ((h_prev, 'h_prev'), (c_prev, 'c_prev')):
        if t is not None and _req(t, f16, n).shape != (B, H):
            raise ValueError(f'{n} must be [{B}, {H}]')
    if bias is not None and _req(bias, torch.float32, 'bias').numel() != 4 * H:
        raise ValueError('bias must have 4H elements')
    h = torch.empty((B, H), dtype=f16, device=x.device)
    c = torch.empty((B, H), dtype=f16, device=x.device)
    _check(lib.ftk_lstm_cell_f16(_ptr(x), _ptr(h_prev), _ptr(c_prev), _ptr(WU), _ptr(bias), _ptr(h), _ptr(c),
                                 ctypes.c_int(B), ctypes.c_int(I), ctypes.c_int(H), _stream()))
    return h, c


def lstm_elementwise(gates, bias, c_prev, out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
                     ) -> Tuple[torch.Tensor, torch.Tensor]:
    """State update on pre-activation gates [B,4H] (the unfused baseline's second kernel)."""
    f32 = torch.float32
    _req(gates, f32, 'gates')
    B, H4 = gates.shape
    H = H4 // 4
    if gates.dim() != 2 or H4 % 4:
        raise ValueError(f'gates must be [B, 4H], got {tuple(gates.shape)}')
    if bias is not None and _req(bias, f32, 'bias').numel() != 4 * H:
        raise ValueError('bias must have 4H elements')
    if c_prev is not None and tuple(_req(c_prev, f32, 'c_prev').shape) != (B, H):
        raise ValueError(f'c_prev must be [{B}, {H}], got {tuple(c_prev.shape)}')
    if out is None:
        h = torch.empty((B, H), dtype=f32, device=gates.device)
        c = torch.empty((B, H), dtype=f32, device=gates.device)
    else:
        h, c = out
        _req_out(h, f32, (B, H), 'h'); _req_out(c, f32, (B, H), 'c')
    _check(lib.ftk_lstm_elementwise_f32(_ptr(gates), _ptr(bias), _ptr(c_prev), _ptr(h), _ptr(c),
                                        ctypes.c_int(B), ctypes.c_int(H), _stream()))
    return h, c


def stacked_lstm_workspace_bytes(L: int, T: int, B: int, H: int) -> int:
    return int(lib.ftk_stacked_lstm_workspace_bytes(L, T, B, H))


def stacked_lstm(xs, WU, bias=None, dilations: Optional[Sequence[int]] = None, schedule: str = 'auto',
                 out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                 workspace: Optional[torch.Tensor] = None,
                 active_rows: Optional[Sequence[int]] = None, products: Optional[str] = None,
                 spin_limit: int = 0, check: Optional[bool] = None, exact_small_states: bool = False
                 ) -> Tuple[torch.Tensor, torch.Tensor]:
    """xs [T,B,H], WU [L,2H,4H], bias [L,4H] or None -> hsss, csss [L,T,B,H].

    schedule: 'auto' (persistent kernel when the shape allows, else per-stage
    launches) or 'wavefront' (always per-stage launches).
    active_rows: for a ragged time-major batch (rows sorted by decreasing length), the number of rows still
    running at each step; only the live (t, row) places of the outputs are defined then.
    products: 'f32' / 'f16x3' for this call, None for the process-wide mode (set_lstm_products).
    spin_limit: polls a bounded wait of the persistent kernel makes before giving up (0 = the default).
    check: wait for the stream and raise FtkError (code -6) if the persistent launch gave up a wait and left
    the outputs incomplete.  Default: True when the workspace is allocated here (nobody else could look at its
    status word afterwards), False when the caller passes one (check it with stacked_lstm_check(workspace)).
    exact_small_states: after a call on split products, wait for the stream and, if hidden states too small for
    the fixed scale of their fp16 planes were written (stacked_lstm_small_states), compute the stack again on fp32
    products, so that layers that fade towards zero are accurate relative to their own size as well.
    """
    f32 = torch.float32
    _req(xs, f32, 'xs'); _req(WU, f32, 'WU')
    T, B, H = xs.shape
    L = WU.shape[0]
    if WU.shape != (L, 2 * H, 4 * H):
        raise ValueError(f'WU must be [L, 2H, 4H] = [{L}, {2 * H}, {4 * H}], got {tuple(WU.shape)}')
    if bias is not None and _req(bias, f32, 'bias').shape != (L, 4 * H):
        raise ValueError('bias must be [L, 4H]')
    if out is None:
        hsss = torch.empty((L, T, B, H), dtype=f32, device=xs.device)
        csss = torch.empty((L, T, B, H), dtype=f32, device=xs.device)
    else:
        hsss, csss = out
        _req_out(hsss, f32, (L, T, B, H), 'hsss'); _req_out(csss, f32, (L, T, B, H), 'csss')
    if products is not None and products not in LSTM_PRODUCTS:
        raise ValueError(f"products must be one of {sorted(LSTM_PRODUCTS)} or None, got {products!r}")
    _count('stacked_lstm')
    dil = None
    if dilations is not None:
        if len(dilations) != L:
            raise ValueError('dilations must have one entry per layer')
        dil = (ctypes.c_int * L)(*[int(d) for d in dilations])
    ci = ctypes.c_int
    if schedule == 'wavefront':
        _check(lib.ftk_stacked_lstm_wavefront_f32(_ptr(xs), _ptr(WU), _ptr(bias), dil, _ptr(hsss), _ptr(csss),
                                                  ci(L), ci(T), ci(B), ci(H), _stream()))
        return hsss, csss
    if schedule != 'auto':
        raise ValueError("schedule must be 'auto' or 'wavefront'")
    need = stacked_lstm_workspace_bytes(L, T, B, H)
    if check is None:
        check = workspace is None
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=xs.device)
    _req_workspace(workspace)
    ws_bytes = ctypes.c_size_t(workspace.numel() * workspace.element_size())
    act = None
    if active_rows is not None:
        if len(active_rows) != T:
            raise ValueError('active_rows must have one entry per step')
        act = (ctypes.c_int * T)(*[int(v) for v in active_rows])
    if products is not None or spin_limit:
        opts = LstmOptions(LSTM_PRODUCTS[products] if products is not None else -1, int(spin_limit))
        _check(lib.ftk_stacked_lstm_opts_f32(_ptr(xs), _ptr(WU), _ptr(bias), dil, act, _ptr(hsss), _ptr(csss), ci(L), ci(T),
                                             ci(B), ci(H), ctypes.byref(opts), _ptr(workspace), ws_bytes, _stream()))
    elif act is not None:
        _check(lib.ftk_stacked_lstm_ragged_f32(_ptr(xs), _ptr(WU), _ptr(bias), dil, act, _ptr(hsss), _ptr(csss),
                                               ci(L), ci(T), ci(B), ci(H), _ptr(workspace), ws_bytes, _stream()))
    elif dil is None:
        _check(lib.ftk_stacked_lstm_f32(_ptr(xs), _ptr(WU), _ptr(bias), _ptr(hsss), _ptr(csss),
                                        ci(L), ci(T), ci(B), ci(H), _ptr(workspace), ws_bytes, _stream()))
    else:
        _check(lib.ftk_dilated_lstm_f32(_ptr(xs), _ptr(WU), _ptr(bias), dil, _ptr(hsss), _ptr(csss),
                                        ci(L), ci(T), ci(B), ci(H), _ptr(workspace), ws_bytes, _stream()))
    if check:
        stacked_lstm_check(workspace)
    if exact_small_states and products != 'f32' and stacked_lstm_small_states(workspace):
        _count('stacked_lstm_repeated_on_f32_products')
        return stacked_lstm(xs, WU, bias, dilations=dilations, out=(hsss, csss), workspace=workspace, active_rows=active_rows,
                            products='f32', spin_limit=spin_limit, check=check)
    return hsss, csss


def stacked_lstm_noalloc(xs, WU, bias, out: Tuple[torch.Tensor, torch.Tensor], dilations: Optional[Sequence[int]] = None) -> None:
    """ftk_stacked_lstm_noalloc_f32: the fp32-product persistent stack (H = 256) into caller-supplied hsss, csss
    [L,T,B,H], with the launch's flags in the library's built-in per-device scratch.  Nothing is allocated, here or in
    the library; the status word is read with stacked_lstm_check(None)."""
    f32 = torch.float32
    _req(xs, f32, 'xs'); _req(WU, f32, 'WU')
    T, B, H = xs.shape
    L = WU.shape[0]
    if WU.shape != (L, 2 * H, 4 * H):
        raise ValueError(f'WU must be [L, 2H, 4H] with H={H}, got {tuple(WU.shape)}')
    if bias is not None and _req(bias, f32, 'bias').numel() != L * 4 * H:
        raise ValueError('bias must be [L, 4H]')
    hsss, csss = out
    _req_out(hsss, f32, (L, T, B, H), 'hsss'); _req_out(csss, f32, (L, T, B, H), 'csss')
    dil = None
    if dilations is not None:
        if len(dilations) != L:
            raise ValueError('one dilation per layer')
        dil = (ctypes.c_int * L)(*[int(d) for d in dilations])
    ci = ctypes.c_int
    _check(lib.ftk_stacked_lstm_noalloc_f32(_ptr(xs), _ptr(WU), _ptr(bias), dil, _ptr(hsss), _ptr(csss), ci(L), ci(T), ci(B),
                                            ci(H), _stream()))


def stacked_lstm_check(workspace: Optional[torch.Tensor]) -> None:
    """Waits for the current stream and raises FtkError (code -6) if the last stacked-LSTM call given this
    workspace drained early because a bounded wait of the persistent kernel ran out.  None: the built-in scratch
    that stacked_lstm_noalloc uses on the current device."""
    if workspace is not None:
        _req_workspace(workspace)
    _check(lib.ftk_stacked_lstm_status(_ptr(workspace), _stream()))


def stacked_lstm_small_states(workspace: torch.Tensor) -> bool:
    """Waits for the current stream; True if the last fp32 stacked-LSTM call given this workspace ran on split
    products and wrote hidden states too small for the fixed scale of their fp16 planes (four neighbouring units of a
    row all below 2^-26 and not all zero): such values reach the cells that read them with fewer than 13 bits.
    The whole output is still accurate relative to its largest value; layers that faded that far are not accurate
    relative to themselves.  stacked_lstm(..., exact_small_states=True) repeats such a call on fp32 products."""
    _req_workspace(workspace)
    rc = lib.ftk_stacked_lstm_small_states(_ptr(workspace), _stream())
    if rc < 0:
        _check(rc)
    return rc == 1


def stacked_lstm_f16(xs, WU, bias=None, dilations: Optional[Sequence[int]] = None,
                     out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, workspace: Optional[torch.Tensor] = None,
                     active_rows: Optional[Sequence[int]] = None, check: Optional[bool] = None
                     ) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp16 storage: xs [T,B,H], WU [L,2H,4H] fp16, bias [L,4H] fp32 or None -> hsss, csss [L,T,B,H] fp16.
    H a multiple of 32: H = 512, and H = 256 with an even batch, run in the persistent kernel, every other
    shape as one launch of the streaming cell kernel per stage of independent cells."""
    f16 = torch.float16
    _req(xs, f16, 'xs'); _req(WU, f16, 'WU')
    T, B, H = xs.shape
    L = WU.shape[0]
    if WU.shape != (L, 2 * H, 4 * H):
        raise ValueError(f'WU must be [L, 2H, 4H] = [{L}, {2 * H}, {4 * H}], got {tuple(WU.shape)}')
    if bias is not None and _req(bias, torch.float32, 'bias').shape != (L, 4 * H):
        raise ValueError('bias must be [L, 4H]')
    if out is None:
        hsss = torch.empty((L, T, B, H), dtype=f16, device=xs.device)
        csss = torch.empty((L, T, B, H), dtype=f16, device=xs.device)
    else:
        hsss, csss = out
        _req_out(hsss, f16, (L, T, B, H), 'hsss'); _req_out(csss, f16, (L, T, B, H), 'csss')
    _count('stacked_lstm_f16')
    dil = None
    if dilations is not None:
        if len(dilations) != L:
            raise ValueError('dilations must have one entry per layer')
        dil = (ctypes.c_int * L)(*[int(d) for d in dilations])
    act = None
    if active_rows is not None:
        if len(active_rows) != T:
            raise ValueError('active_rows must have one entry per step')
        act = (ctypes.c_int * T)(*[int(v) for v in active_rows])
    if check is None:
        check = workspace is None
    if workspace is None:
        workspace = torch.empty(int(lib.ftk_stacked_lstm_f16_workspace_bytes(L, T, B, H)), dtype=torch.uint8, device=xs.device)
    _req_workspace(workspace)
    ci = ctypes.c_int
    _check(lib.ftk_stacked_lstm_f16(_ptr(xs), _ptr(WU), _ptr(bias), dil, act, _ptr(hsss), _ptr(csss), ci(L), ci(T), ci(B),
                                    ci(H), _ptr(workspace), ctypes.c_size_t(workspace.numel() * workspace.element_size()),
                                    _stream()))
    if check:
        stacked_lstm_check(workspace)
    return hsss, csss


LSTM_PRODUCTS = {'f32': 0, 'f16x3': 1}


def set_lstm_products(mode: str) -> None:
    """How the persistent stacked-LSTM kernel forms the gate GEMM's products.

    'f32': one fp32 MFMA per product.  'f16x3' (default): each fp32 operand as an fp16 value plus an fp16
    remainder under a shared power-of-two scale, three fp16 MFMAs per fp32 one, fp32 accumulation; only the
    remainder-times-remainder term (2^-22 of a product) is dropped.
    """
    if mode not in LSTM_PRODUCTS:
        raise ValueError(f"mode must be one of {sorted(LSTM_PRODUCTS)}, got {mode!r}")
    _check(lib.ftk_lstm_set_products(ctypes.c_int(LSTM_PRODUCTS[mode])))


def get_lstm_products() -> str:
    code = int(lib.ftk_lstm_get_products())
    return next(k for k, v in LSTM_PRODUCTS.items() if v == code)


def persistent_status(workspace: torch.Tensor) -> int:
    """Error word a persistent stacked-LSTM launch left in its workspace (synchronises).

    0 = every bounded wait completed; 1 = a wait ran out of polls and the launch drained early.
    """
    torch.cuda.synchronize()
    return int(workspace[:4].view(torch.int32).item())


def b2b_gemm(A, B_nk, C_pn, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """D = (A @ B) @ C.  A [G,M,K]; B_nk [G,N,K] (B stored column-major); C_pn [G,P,N]; D [G,M,P]; fp16."""
    f16 = torch.float16
    _req(A, f16, 'A'); _req(B_nk, f16, 'B_nk'); _req(C_pn, f16, 'C_pn')
    squeeze = A.dim() == 2
    if squeeze:
        A, B_nk, C_pn = A[None], B_nk[None], C_pn[None]
    G, M, K = A.shape
    N = B_nk.shape[1]
    P = C_pn.shape[1]
    if B_nk.shape != (G, N, K) or C_pn.shape != (G, P, N):
        raise ValueError(f'shape mismatch: A {tuple(A.shape)}, B_nk {tuple(B_nk.shape)}, C_pn {tuple(C_pn.shape)}')
    D = out if out is not None else torch.empty((G, M, P), dtype=f16, device=A.device)
    _req_out(D, f16, (G, M, P), 'D')
    _count('b2b_gemm')
    ci = ctypes.c_int
    _check(lib.ftk_b2b_gemm_f16(_ptr(A), _ptr(B_nk), _ptr(C_pn), _ptr(D), ci(G), ci(M), ci(N), ci(K), ci(P), _stream()))
    return D[0] if squeeze and out is None else D


def b2b_gemm_supported(N: int, K: int, P: int) -> bool:
    """Shapes ftk_b2b_gemm_f16 takes on the current device (the fused kernels' LDS fit, or N <= 2048 for the general one)."""
    return bool(lib.ftk_b2b_gemm_f16_supported(ctypes.c_int(N), ctypes.c_int(K), ctypes.c_int(P)))


def b2b_gemm_rowmajor_supported(N: int, K: int, P: int) -> bool:
    """Shapes ftk_b2b_gemm_rowmajor_f16 is built for."""
    return K in (64, 128) and N in (64, 128) and P % 128 == 0


def b2b_gemm_rowmajor(A, B, C, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """D = (A @ B) @ C with every operand row-major: A [G,M,K], B [G,K,N], C [G,N,P], D [G,M,P]; fp16.
    K and N in {64, 128}, P a multiple of 128."""
    f16 = torch.float16
    _req(A, f16, 'A'); _req(B, f16, 'B'); _req(C, f16, 'C')
    squeeze = A.dim() == 2
    if squeeze:
        A, B, C = A[None], B[None], C[None]
    G, M, K = A.shape
    N = B.shape[2]
    P = C.shape[2]
    if B.shape != (G, K, N) or C.shape != (G, N, P):
        raise ValueError(f'shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, C {tuple(C.shape)}')
    D = out if out is not None else torch.empty((G, M, P), dtype=f16, device=A.device)
    _req_out(D, f16, (G, M, P), 'D')
    _count('b2b_gemm_rowmajor')
    ci = ctypes.c_int
    _check(lib.ftk_b2b_gemm_rowmajor_f16(_ptr(A), _ptr(B), _ptr(C), _ptr(D), ci(G), ci(M), ci(N), ci(K), ci(P), _stream()))
    return D[0] if squeeze and out is None else D


def gemm(A, B, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """C = A @ B, fp16 storage, fp32 accumulation, row-major: A [M,K] or [G,M,K], B [K,N] or [G,K,N].
    N a multiple of 128, K of 32."""
    f16 = torch.float16
    _req(A, f16, 'A'); _req(B, f16, 'B')
    if A.dim() != B.dim() or A.dim() not in (2, 3):
        raise ValueError('A and B must both be matrices or both be batches of matrices')
    batched = A.dim() == 3
    G = A.shape[0] if batched else 1
    M, K = A.shape[-2:]
    N = B.shape[-1]
    if B.shape[-2] != K or (batched and B.shape[0] != G):
        raise ValueError(f'shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}')
    C = out if out is not None else torch.empty((*A.shape[:-1], N), dtype=f16, device=A.device)
    _req_out(C, f16, (*A.shape[:-1], N), 'C')
    ci = ctypes.c_int
    _count('gemm')
    if batched:
        _check(lib.ftk_batched_gemm_f16(_ptr(A), _ptr(B), _ptr(C), ci(G), ci(M), ci(N), ci(K), _stream()))
    else:
        _check(lib.ftk_gemm_f16(_ptr(A), _ptr(B), _ptr(C), ci(M), ci(N), ci(K), _stream()))
    return C


def flash_attention(Q, K, V, scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                    workspace: Optional[torch.Tensor] = None, split_keys: bool = True) -> torch.Tensor:
    """O = softmax(Q K^T scale) V.  Q [B,Hd,Sq,D], K/V [B,Hd,Skv,D], fp16, non-causal.
    A grid that does not fill the chip (few queries, heads and samples) with many keys is split over the keys and
    merged (ftk_flash_attn_ws_f16); the workspace for that is allocated here unless one is given, split_keys=False
    keeps the single launch."""
    f16 = torch.float16
    _req(Q, f16, 'Q'); _req(K, f16, 'K'); _req(V, f16, 'V')
    B, Hd, Sq, D = Q.shape
    Skv = K.shape[2]
    if K.shape != (B, Hd, Skv, D) or V.shape != (B, Hd, Skv, D):
        raise ValueError(f'shape mismatch: Q {tuple(Q.shape)}, K {tuple(K.shape)}, V {tuple(V.shape)}')
    if scale is None:
        scale = D ** -0.5
    O = out if out is not None else torch.empty_like(Q)
    _req_out(O, f16, Q.shape, 'O')
    _count('flash_attention')
    ci = ctypes.c_int
    need = int(lib.ftk_flash_attn_f16_workspace_bytes(B, Hd, Sq, Skv, D)) if split_keys else 0
    if need:
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=Q.device)
        _req_workspace(workspace)
        _count('flash_attention_split_keys')
        _check(lib.ftk_flash_attn_ws_f16(_ptr(Q), _ptr(K), _ptr(V), _ptr(O), ci(B), ci(Hd), ci(Sq), ci(Skv), ci(D), ctypes.c_float(scale),
                                         _ptr(workspace), ctypes.c_size_t(workspace.numel() * workspace.element_size()), _stream()))
        return O
    _check(lib.ftk_flash_attn_f16(_ptr(Q), _ptr(K), _ptr(V), _ptr(O), ci(B), ci(Hd), ci(Sq), ci(Skv), ci(D),
                                  ctypes.c_float(scale), _stream()))
    return O


def flash_attention_f32(Q, K, V, scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                        workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Non-causal attention with fp32 Q [B,Hd,Sq,D], K, V [B,Hd,Skv,D] -> O [B,Hd,Sq,D] fp32; D of 32, 64, 96 or 128.
    Every product as three fp16 MFMAs of split operands, fp32 accumulation and softmax state."""
    f32 = torch.float32
    _req(Q, f32, 'Q'); _req(K, f32, 'K'); _req(V, f32, 'V')
    if Q.dim() != 4 or K.dim() != 4 or K.shape != V.shape or Q.shape[:2] != K.shape[:2] or Q.shape[3] != K.shape[3]:
        raise ValueError(f'Q [B,Hd,Sq,D] and K, V [B,Hd,Skv,D] expected, got {tuple(Q.shape)}, {tuple(K.shape)}, {tuple(V.shape)}')
    B, Hd, Sq, D = Q.shape
    Skv = K.shape[2]
    if scale is None:
        scale = D ** -0.5
    O = out if out is not None else torch.empty_like(Q)
    _req_out(O, f32, (B, Hd, Sq, D), 'O')
    need = int(lib.ftk_flash_attn_f32_workspace_bytes(B, Hd, Sq, Skv, D))
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=Q.device)
    _req_workspace(workspace)
    _count('flash_attention_f32')
    ci = ctypes.c_int
    _check(lib.ftk_flash_attn_f32(_ptr(Q), _ptr(K), _ptr(V), _ptr(O), ci(B), ci(Hd), ci(Sq), ci(Skv), ci(D), ctypes.c_float(scale),
                                  _ptr(workspace), ctypes.c_size_t(workspace.numel() * workspace.element_size()), _stream()))
    return O


def read_fa_trace(tiles: int):
    """Timeline of one wave of workgroup 0 of the last flash-attention launch: [tiles, 6] in us.  Only a tuning
    build of the library (make TRACE=1, run with FTK_FA_TRACE=1+wave) records it."""
    import numpy as np
    fn = getattr(lib, 'ftk_debug_read_fa_trace', None)
    if fn is None:
        raise RuntimeError('this build of libftkernels.so has no attention timeline: build it with make TRACE=1')
    fn.restype = ctypes.c_int
    buf = (ctypes.c_longlong * (tiles * 6))()
    _check(fn(buf, ctypes.c_int(tiles * 6)))
    return np.frombuffer(buf, dtype=np.int64).reshape(tiles, 6).astype(np.float64) / 100.0


def embedding_gather(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None,
                     check: bool = True) -> torch.Tensor:
    """table [V,E] fp32, ids int32/int64 of any shape -> [*ids.shape, E]: rows of the table.

    check=True reads back the count of ids outside [0,V) (one synchronising copy of 4 bytes) and raises
    IndexError like indexing a FractalTensor does; check=False leaves such rows zero-filled."""
    _req(table, torch.float32, 'table')
    if ids.dtype not in (torch.int32, torch.int64):
        raise TypeError(f'ids must be int32 or int64, got {ids.dtype}')
    if not ids.is_cuda or not ids.is_contiguous():
        raise RuntimeError('ids must be a contiguous CUDA tensor')
    if table.dim() != 2:
        raise ValueError('table must be [V, E]')
    V, E = table.shape
    n = ids.numel()
    if out is None:
        out = torch.empty((*ids.shape, E), dtype=torch.float32, device=table.device)
    else:
        _req(out, torch.float32, 'out')
        if out.numel() != n * E:
            raise ValueError('out must hold ids.numel() * E elements')
    if n == 0:
        return out
    bad = torch.zeros(1, dtype=torch.int32, device=table.device) if check else None
    _check(lib.ftk_embedding_gather_f32(_ptr(table), _ptr(ids), ctypes.c_int(1 if ids.dtype == torch.int64 else 0),
                                        _ptr(out), ctypes.c_longlong(n), ctypes.c_int(V), ctypes.c_int(E),
                                        _ptr(bad), _stream()))
    if check and int(bad.item()) != 0:
        raise IndexError(f'{int(bad.item())} ids are outside [0, {V})')
    return out


def online_softmax(x) -> torch.Tensor:
    """Row softmax of x [rows, cols], fp32."""
    _req(x, torch.float32, 'x')
    rows, cols = x.shape
    y = torch.empty_like(x)
    _check(lib.ftk_online_softmax_f32(_ptr(x), _ptr(y), ctypes.c_int(rows), ctypes.c_int(cols), _stream()))
    return y


def grid_rnn(xs, ys, Wx, Ux, bx, Wy, Uy, by, crossed: bool = False, out: Optional[torch.Tensor] = None,
             workspace: Optional[torch.Tensor] = None, relay_weights: bool = True) -> torch.Tensor:
    """Stacked grid RNN, fp32.  W* [D, H, H], U* [D, 2H, H], biases [D, 1 or B, H] or both None.
    crossed=False: xs [L1, B, H] feeds the first grid axis, ys [L2, B, H] the second (the layout of the
    reference's grid benchmark); crossed=True: xs [L2, B, H] is indexed by the second axis and ys [L1, B, H] by the
    first (the layout of its frontend program).  Returns hsss [D, L1, L2, 2, B, H]: h_x at index 0, h_y at 1.
    workspace: uint8 device tensor for the re-laid parameters (allocated here if None); relay_weights=False runs
    the kernel that reads the parameters where they lie."""
    for name, t in (('xs', xs), ('ys', ys), ('Wx', Wx), ('Ux', Ux), ('Wy', Wy), ('Uy', Uy)):
        _req(t, torch.float32, name)
    if xs.dim() != 3 or ys.dim() != 3 or xs.shape[1:] != ys.shape[1:]:
        raise ValueError(f'xs and ys must be [L, B, H] with equal B and H, got {tuple(xs.shape)} and {tuple(ys.shape)}')
    _, B, H = xs.shape
    L1, L2 = (ys.shape[0], xs.shape[0]) if crossed else (xs.shape[0], ys.shape[0])
    D = Wx.shape[0]
    for name, t, shape in (('Wx', Wx, (D, H, H)), ('Wy', Wy, (D, H, H)), ('Ux', Ux, (D, 2 * H, H)), ('Uy', Uy, (D, 2 * H, H))):
        if tuple(t.shape) != shape:
            raise ValueError(f'{name} must be {shape}, got {tuple(t.shape)}')
    if (bx is None) != (by is None):
        raise ValueError('give both biases or neither')
    bias_rows = 1
    if bx is not None:
        _req(bx, torch.float32, 'bx')
        _req(by, torch.float32, 'by')
        bias_rows = bx.shape[1]
        if tuple(bx.shape) != (D, bias_rows, H) or bx.shape != by.shape or bias_rows not in (1, B):
            raise ValueError(f'biases must both be [D, 1 or B, H], got {tuple(bx.shape)} and {tuple(by.shape)}')
    if out is None:
        out = torch.empty((D, L1, L2, 2, B, H), dtype=torch.float32, device=xs.device)
    else:
        _req(out, torch.float32, 'out')
        if tuple(out.shape) != (D, L1, L2, 2, B, H):
            raise ValueError(f'out must be {(D, L1, L2, 2, B, H)}, got {tuple(out.shape)}')
    if relay_weights and workspace is None:
        shared = Wx.data_ptr() == Wy.data_ptr() and Ux.data_ptr() == Uy.data_ptr()
        workspace = torch.empty(lib.ftk_grid_rnn_workspace_bytes(D, H) // (2 if shared else 1), dtype=torch.uint8, device=xs.device)
    ws_ptr, ws_bytes = (_ptr(workspace), workspace.numel()) if relay_weights else (None, 0)
    _check(lib.ftk_grid_rnn_f32(_ptr(xs), _ptr(ys), _ptr(Wx), _ptr(Ux), _ptr(bx), _ptr(Wy), _ptr(Uy), _ptr(by), _ptr(out),
                                ctypes.c_int(D), ctypes.c_int(L1), ctypes.c_int(L2), ctypes.c_int(B), ctypes.c_int(H),
                                ctypes.c_int(bias_rows), ctypes.c_int(1 if crossed else 0), ws_ptr, ctypes.c_size_t(ws_bytes), _stream()))
    return out


def windowed_attention(Q, K, V, window: int, dilation: int = 1, extra_idx: Optional[torch.Tensor] = None,
                       scale: float = 1.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Q, K, V [G, S, D] fp32: every token attends to the `window` positions centred on it (`dilation` apart,
    wrapped at the ends as shifted_slide wraps them) and to extra_idx[g, t, :] (int32 [G, S, R]) if given."""
    for name, t in (('Q', Q), ('K', K), ('V', V)):
        _req(t, torch.float32, name)
    if Q.dim() != 3 or K.shape != Q.shape or V.shape != Q.shape:
        raise ValueError(f'Q, K and V must be [G, S, D] of one shape, got {tuple(Q.shape)}, {tuple(K.shape)}, {tuple(V.shape)}')
    G, S, D = Q.shape
    R = 0
    if extra_idx is not None:
        _req(extra_idx, torch.int32, 'extra_idx')
        if extra_idx.dim() != 3 or tuple(extra_idx.shape[:2]) != (G, S):
            raise ValueError(f'extra_idx must be [G, S, R], got {tuple(extra_idx.shape)}')
        R = extra_idx.shape[2]
        if R == 0:
            extra_idx = None
        elif int(extra_idx.min()) < 0 or int(extra_idx.max()) >= S:
            raise IndexError(f'extra_idx holds a position outside [0, {S})')
    if out is None:
        out = torch.empty_like(Q)
    else:
        _req(out, torch.float32, 'out')
        if out.shape != Q.shape:
            raise ValueError(f'out must be {tuple(Q.shape)}, got {tuple(out.shape)}')
    _check(lib.ftk_windowed_attn_f32(_ptr(Q), _ptr(K), _ptr(V), _ptr(extra_idx), _ptr(out), ctypes.c_int(G), ctypes.c_int(S),
                                     ctypes.c_int(D), ctypes.c_int(window), ctypes.c_int(dilation), ctypes.c_int(R),
                                     ctypes.c_float(scale), _stream()))
    return out
