"""CPU-side checks of the C-ABI library: it loads, exports every symbol that
include/ftk.h declares, and rejects bad arguments before touching a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, 'include', 'ftk.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(ftk_[a-z0-9_]+)\s*\(', text)))


def test_header_and_binding_agree():
    import fractaltensor_amd._core as core
    assert sorted(core.EXPORTS) == declared_symbols()


def test_library_exports_every_declared_symbol():
    import fractaltensor_amd._core as core
    lib = ctypes.CDLL(core.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name
    assert core.version() >= 100


def test_argument_errors_come_back_as_codes_not_crashes():
    import fractaltensor_amd._core as core
    lib = core.lib
    nul = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)   # never dereferenced: validation fails first
    ci = ctypes.c_int
    assert lib.ftk_lstm_cell_f32(nul, nul, nul, nul, nul, nul, nul, ci(1), ci(32), ci(32), nul) == -1
    assert b'non-NULL' in lib.ftk_last_error()
    assert lib.ftk_lstm_cell_f32(one, nul, nul, one, nul, one, one, ci(4), ci(30), ci(32), nul) == -2
    assert lib.ftk_lstm_cell_f32(one, one, nul, one, nul, one, one, ci(4), ci(32), ci(32), nul) == -1
    assert lib.ftk_b2b_gemm_f16(one, one, one, one, ci(1), ci(64), ci(48), ci(64), ci(64), nul) == -2
    assert lib.ftk_b2b_gemm_f16(one, one, one, one, ci(0), ci(64), ci(64), ci(64), ci(64), nul) == -1
    assert lib.ftk_b2b_gemm_f16(one, one, one, one, ci(1), ci(64), ci(64), ci(24), ci(64), nul) == -2   # K % 16
    assert lib.ftk_b2b_gemm_rowmajor_f16(one, one, one, one, ci(1), ci(64), ci(64), ci(96), ci(128), nul) == -2
    assert lib.ftk_b2b_gemm_rowmajor_f16(one, nul, one, one, ci(1), ci(64), ci(64), ci(64), ci(128), nul) == -1
    assert lib.ftk_gemm_f16(one, one, one, ci(64), ci(96), ci(64), nul) == -2
    assert lib.ftk_gemm_f16(one, ctypes.c_void_p(18), one, ci(64), ci(256), ci(64), nul) == -1 and b'aligned' in lib.ftk_last_error()
    assert lib.ftk_batched_gemm_f16(one, one, nul, ci(2), ci(64), ci(128), ci(64), nul) == -1
    assert lib.ftk_flash_attn_f16(one, one, one, one, ci(1), ci(1), ci(64), ci(64), ci(48), ctypes.c_float(1), nul) == -2
    cf = ctypes.c_float
    assert lib.ftk_flash_attn_f32(one, nul, one, one, ci(1), ci(1), ci(64), ci(64), ci(64), cf(1), one, ctypes.c_size_t(1 << 30), nul) == -1
    assert lib.ftk_flash_attn_f32(one, one, one, one, ci(1), ci(1), ci(64), ci(64), ci(48), cf(1), one, ctypes.c_size_t(1 << 30), nul) == -2
    assert lib.ftk_flash_attn_f32(ctypes.c_void_p(20), one, one, one, ci(1), ci(1), ci(64), ci(64), ci(64), cf(1), one, ctypes.c_size_t(1 << 30), nul) == -1
    assert lib.ftk_flash_attn_f32(one, one, one, one, ci(1), ci(1), ci(64), ci(64), ci(64), cf(0), one, ctypes.c_size_t(1 << 30), nul) == -1
    assert lib.ftk_flash_attn_f32(one, one, one, one, ci(1), ci(1), ci(64), ci(64), ci(64), cf(1), nul, ctypes.c_size_t(0), nul) == -3
    assert lib.ftk_flash_attn_f32_workspace_bytes(ci(2), ci(3), ci(100), ci(77), ci(64)) >= 4 * 6 * (2 * 77) * 64   # K's and V's planes
    assert lib.ftk_b2b_gemm_f16_supported(ci(48), ci(64), ci(64)) == 0          # N % 32
    assert lib.ftk_stacked_lstm_small_states(nul, nul) == -1
    assert lib.ftk_online_softmax_f32(nul, one, ci(1), ci(1), nul) == -1
    assert lib.ftk_stacked_lstm_wavefront_f32(one, one, nul, nul, one, one, ci(1), ci(1), ci(1), ci(48), nul) == -2
    assert lib.ftk_embedding_gather_f32(one, one, ci(0), one, ctypes.c_longlong(4), ci(8), ci(6), nul, nul) == -2
    assert lib.ftk_embedding_gather_f32(one, nul, ci(0), one, ctypes.c_longlong(4), ci(8), ci(8), nul, nul) == -1
    assert lib.ftk_stacked_lstm_ragged_f32(one, one, nul, nul, nul, one, one, ci(1), ci(1), ci(1), ci(32), nul, ctypes.c_size_t(0), nul) == -1
    assert lib.ftk_lstm_cell_f16(one, nul, nul, one, nul, one, one, ci(4), ci(48), ci(64), nul) == -2
    assert lib.ftk_lstm_layer_f32(one, one, nul, one, nul, one, one, ci(2), ci(4), ci(32), ci(32), nul) == -1
    assert lib.ftk_lstm_layer_f16(one, one, nul, nul, nul, one, one, ci(2), ci(4), ci(32), ci(40), nul) == -2
    assert lib.ftk_lstm_layer_f32(one, one, nul, nul, nul, one, one, ci(0), ci(4), ci(32), ci(32), nul) == -1
    assert lib.ftk_lstm_cell_f16(one, one, nul, one, nul, one, one, ci(4), ci(64), ci(64), nul) == -1
    assert lib.ftk_stacked_lstm_f16(one, one, nul, nul, nul, one, one, ci(1), ci(1), ci(4), ci(80), nul, ctypes.c_size_t(0), nul) == -2
    # a shape whose weights are streamed needs the workspace for their re-laid copy
    assert lib.ftk_stacked_lstm_f16(one, one, nul, nul, nul, one, one, ci(2), ci(3), ci(4), ci(1024), nul, ctypes.c_size_t(0), nul) == -3
    # the status block (256 bytes, its first int the status word) and the re-laid weights
    assert lib.ftk_stacked_lstm_f16_workspace_bytes(2, 3, 4, 1024) == 256 + 2 * 2048 * 4096 * 2
    # per-call options: an unknown products mode, a negative poll limit; the status query without a workspace
    opts = core.LstmOptions(7, 0)
    stack = lambda o: lib.ftk_stacked_lstm_opts_f32(one, one, nul, nul, nul, one, one, ci(1), ci(1), ci(1), ci(32), o, nul,
                                                    ctypes.c_size_t(0), nul)
    assert stack(ctypes.byref(opts)) == -1
    assert stack(ctypes.byref(core.LstmOptions(-1, -5))) == -1
    assert lib.ftk_stacked_lstm_status(nul, nul) == -1
    assert lib.ftk_stacked_lstm_workspace_bytes(32, 64, 256, 256) > 0
    assert lib.ftk_stacked_lstm_workspace_bytes(0, 64, 256, 256) == 0
    # grid RNN: null operands, a hidden size that is no multiple of 32, bias rows that are neither 1 nor B, one bias only
    cz, cf = ctypes.c_size_t, ctypes.c_float
    grid = lambda *p, H=32, rows=1, bx=one, by=one: lib.ftk_grid_rnn_f32(*p, bx, one, one, by, one, ci(1), ci(2), ci(2), ci(4), ci(H),
                                                                         ci(rows), ci(0), nul, cz(0), nul)
    assert grid(nul, one, one, one) == -1
    assert grid(one, one, one, one, H=48) == -2
    assert grid(one, one, one, one, rows=3) == -1
    assert grid(one, one, one, one, by=nul) == -1
    assert lib.ftk_grid_rnn_workspace_bytes(32, 256) == 2 * 32 * 3 * 256 * 256 * 4
    assert lib.ftk_grid_rnn_workspace_bytes(0, 256) == 0
    # windowed attention: even window, head size off the 16-byte pieces, a span longer than the sequence, indices without a count
    wa = lambda S=8, D=16, W=3, dl=1, R=0, idx=nul, q=one: lib.ftk_windowed_attn_f32(q, one, one, idx, one, ci(1), ci(S), ci(D), ci(W),
                                                                                       ci(dl), ci(R), cf(1.0), nul)
    assert wa(q=nul) == -1
    assert wa(W=4) == -2
    assert wa(D=6) == -2
    assert wa(W=5, dl=4) == -2
    assert wa(idx=one) == -1
    assert wa(R=2) == -1
    assert wa(q=ctypes.c_void_p(8)) == -1          # not 16-byte aligned


def test_wrappers_check_supplied_outputs_before_any_launch():
    """A caller-supplied output of the wrong shape must never reach a kernel (it would be overrun), and a workspace
    must be device memory.  The shape is looked at first, so host tensors are enough to show it."""
    import torch
    import fractaltensor_amd._core as core
    f32 = torch.float32
    with pytest.raises(ValueError, match=r'hsss must be \(2, 3, 4, 32\)'):
        core._req_out(torch.empty((2, 3, 4, 16), dtype=f32), f32, (2, 3, 4, 32), 'hsss')
    with pytest.raises(RuntimeError, match='no CPU path'):      # right shape: the next check is the device
        core._req_out(torch.empty((2, 3, 4, 32), dtype=f32), f32, (2, 3, 4, 32), 'hsss')
    with pytest.raises(ValueError, match='workspace'):
        core._req_workspace(torch.empty(16, dtype=torch.uint8))
    with pytest.raises(ValueError, match='workspace'):
        core._req_workspace(None)


def test_wrappers_refuse_cpu_tensors():
    import torch
    import fractaltensor_amd._core as core
    x = torch.zeros((4, 32))
    with pytest.raises(RuntimeError, match='no CPU path'):
        core.lstm_cell(x, None, None, torch.zeros((64, 128)))
    with pytest.raises(RuntimeError, match='no CPU path'):
        core.online_softmax(x)
