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
    assert lib.ftk_b2b_gemm_rowmajor_f16(one, one, one, one, ci(1), ci(64), ci(64), ci(96), ci(128), nul) == -2
    assert lib.ftk_b2b_gemm_rowmajor_f16(one, nul, one, one, ci(1), ci(64), ci(64), ci(64), ci(128), nul) == -1
    assert lib.ftk_gemm_f16(one, one, one, ci(64), ci(96), ci(64), nul) == -2
    assert lib.ftk_batched_gemm_f16(one, one, nul, ci(2), ci(64), ci(128), ci(64), nul) == -1
    assert lib.ftk_flash_attn_f16(one, one, one, one, ci(1), ci(1), ci(64), ci(64), ci(48), ctypes.c_float(1), nul) == -2
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
    assert lib.ftk_stacked_lstm_f16_workspace_bytes(2, 3, 4, 1024) == 2 * 2048 * 4096 * 2
    assert lib.ftk_stacked_lstm_workspace_bytes(32, 64, 256, 256) > 0
    assert lib.ftk_stacked_lstm_workspace_bytes(0, 64, 256, 256) == 0


def test_wrappers_refuse_cpu_tensors():
    import torch
    import fractaltensor_amd._core as core
    x = torch.zeros((4, 32))
    with pytest.raises(RuntimeError, match='no CPU path'):
        core.lstm_cell(x, None, None, torch.zeros((64, 128)))
    with pytest.raises(RuntimeError, match='no CPU path'):
        core.online_softmax(x)
