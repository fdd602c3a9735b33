"""ctypes loader for oracle/liboracle.so (the plain-C oracle).

TEST INFRASTRUCTURE ONLY: see the package docstring.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, 'liboracle.so')
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle.c with gcc (a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(['make', '-C', _HERE, '-B' if force else '-s', 'liboracle.so'])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ('orc_lstm_cell_f32', 'orc_stacked_lstm_f32', 'orc_b2b_gemm_f16',
                     'orc_flash_attn_f16', 'orc_online_softmax_f32'):
            getattr(_lib, name).restype = ctypes.c_int
        _lib.orc_half_to_float.restype = ctypes.c_float
        _lib.orc_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.orc_float_to_half.restype = ctypes.c_uint16
        _lib.orc_float_to_half.argtypes = [ctypes.c_float]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _f16(a):
    return np.ascontiguousarray(a, dtype=np.float16)


def lstm_cell(x, h_prev, c_prev, WU, bias=None):
    x, h_prev, c_prev, WU, bias = map(_f32, (x, h_prev, c_prev, WU, bias))
    B, I = x.shape
    H = WU.shape[1] // 4
    h = np.empty((B, H), np.float32)
    c = np.empty((B, H), np.float32)
    rc = lib().orc_lstm_cell_f32(_p(x), _p(h_prev), _p(c_prev), _p(WU), _p(bias), _p(h), _p(c),
                                 ctypes.c_int(B), ctypes.c_int(I), ctypes.c_int(H))
    assert rc == 0
    return h, c


def stacked_lstm(xs, WUs, biases=None, dilations=None):
    xs, WUs, biases = map(_f32, (xs, WUs, biases))
    T, B, H = xs.shape
    L = WUs.shape[0]
    assert WUs.shape == (L, 2 * H, 4 * H)
    dil = None if dilations is None else np.ascontiguousarray(dilations, dtype=np.int32)
    hsss = np.empty((L, T, B, H), np.float32)
    csss = np.empty((L, T, B, H), np.float32)
    rc = lib().orc_stacked_lstm_f32(_p(xs), _p(WUs), _p(biases), _p(dil), _p(hsss), _p(csss),
                                    ctypes.c_int(L), ctypes.c_int(T), ctypes.c_int(B), ctypes.c_int(H))
    assert rc == 0
    return hsss, csss


def b2b_gemm(A, B_nk, C_pn, round_intermediate=True):
    """A [G,M,K], B_nk [G,N,K], C_pn [G,P,N] fp16 -> D [G,M,P] fp32."""
    A, B_nk, C_pn = map(_f16, (A, B_nk, C_pn))
    G, M, K = A.shape
    N = B_nk.shape[1]
    P = C_pn.shape[1]
    D = np.empty((G, M, P), np.float32)
    rc = lib().orc_b2b_gemm_f16(_p(A), _p(B_nk), _p(C_pn), _p(D), ctypes.c_int(G), ctypes.c_int(M),
                                ctypes.c_int(N), ctypes.c_int(K), ctypes.c_int(P),
                                ctypes.c_int(1 if round_intermediate else 0))
    assert rc == 0
    return D


def flash_attention(Q, K, V, scale, block_kv=64):
    """Q [BH,Sq,D], K/V [BH,Skv,D] fp16 -> O [BH,Sq,D] fp32."""
    Q, K, V = map(_f16, (Q, K, V))
    BH, Sq, D = Q.shape
    Skv = K.shape[1]
    O = np.empty((BH, Sq, D), np.float32)
    rc = lib().orc_flash_attn_f16(_p(Q), _p(K), _p(V), _p(O), ctypes.c_int(BH), ctypes.c_int(Sq),
                                  ctypes.c_int(Skv), ctypes.c_int(D), ctypes.c_float(scale),
                                  ctypes.c_int(block_kv))
    assert rc == 0
    return O


def online_softmax(x):
    x = _f32(x)
    rows, cols = x.shape
    y = np.empty_like(x)
    rc = lib().orc_online_softmax_f32(_p(x), _p(y), ctypes.c_int(rows), ctypes.c_int(cols))
    assert rc == 0
    return y
