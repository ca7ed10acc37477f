"""numpy front end of oracle/lstm_oracle.c (test infrastructure only)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblstm_oracle.so")
_lib = None

FLAG_FP16_OPERANDS = 1   # round x, W_ih, W_hh to fp16 before use
FLAG_FP16_FEEDBACK = 2   # h is fed back through an fp16 cast (reference src/kernels.cu:150-155)
FLAG_FP16_OUTPUT = 4     # y holds fp16-rounded values
FLAG_FP16_DG = 8         # backward: pre-activation gradients are rounded to fp16 before the GEMMs that consume them


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "lstm_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O2", "-fPIC", "-shared", "-std=c99", "-o", _SO, src, "-lm"])
    return _SO


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_SO)
        dp, sz, i32 = ctypes.POINTER(ctypes.c_double), ctypes.c_size_t, ctypes.c_int
        lib.oracle_lstm_forward.argtypes = [sz] * 4 + [dp] * 7 + [i32] + [dp] * 6
        lib.oracle_lstm_forward.restype = i32
        lib.oracle_lstm_backward.argtypes = [sz] * 4 + [dp] * 9 + [i32] + [dp] * 6
        lib.oracle_lstm_backward.restype = i32
        lib.oracle_pack_stride_v1.argtypes = [sz, sz]
        lib.oracle_pack_stride_v1.restype = sz
        lib.oracle_pack_weights_v1.argtypes = [sz, sz, dp, dp, dp]
        lib.oracle_checkpoints.argtypes = [sz] * 4 + [dp, dp]
        lib.oracle_chunk_steps.argtypes = [i32, sz]
        lib.oracle_chunk_steps.restype = sz
        lib.oracle_round_fp16.argtypes = [ctypes.c_double]
        lib.oracle_round_fp16.restype = ctypes.c_double
        _lib = lib
    return _lib


def _d(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float64)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def round_fp16(v: float) -> float:
    return _load().oracle_round_fp16(float(v))


def chunk_steps(chunk: int, T: int) -> int:
    return int(_load().oracle_chunk_steps(int(chunk), int(T)))


def forward(x, w_ih, w_hh, b_ih=None, b_hh=None, h0=None, c0=None, flags: int = 0):
    """x (T,B,I) -> dict(y, hn, cn, gates (T,B,4H), h_all, c_all (T+1,B,H)), all float64."""
    lib = _load()
    x, w_ih, w_hh, b_ih, b_hh, h0, c0 = map(_d, (x, w_ih, w_hh, b_ih, b_hh, h0, c0))
    T, B, I = x.shape
    H = w_hh.shape[1]
    assert w_ih.shape == (4 * H, I) and w_hh.shape == (4 * H, H)
    out = dict(y=np.zeros((T, B, H)), hn=np.zeros((B, H)), cn=np.zeros((B, H)), gates=np.zeros((T, B, 4 * H)),
               h_all=np.zeros((T + 1, B, H)), c_all=np.zeros((T + 1, B, H)))
    rc = lib.oracle_lstm_forward(T, B, I, H, _p(x), _p(w_ih), _p(w_hh), _p(b_ih), _p(b_hh), _p(h0), _p(c0),
                                 int(flags), _p(out["y"]), _p(out["hn"]), _p(out["cn"]), _p(out["gates"]),
                                 _p(out["h_all"]), _p(out["c_all"]))
    if rc != 0:
        raise MemoryError("oracle_lstm_forward failed")
    return out


def backward(x, w_ih, w_hh, fwd, dY, d_hn=None, d_cn=None, flags: int = 0):
    """BPTT from a forward() result -> dict(dx, dw_ih, dw_hh, db, dh0, dc0), all float64."""
    lib = _load()
    x, w_ih, w_hh, dY, d_hn, d_cn = map(_d, (x, w_ih, w_hh, dY, d_hn, d_cn))
    T, B, I = x.shape
    H = w_hh.shape[1]
    out = dict(dx=np.zeros((T, B, I)), dw_ih=np.zeros((4 * H, I)), dw_hh=np.zeros((4 * H, H)), db=np.zeros(4 * H),
               dh0=np.zeros((B, H)), dc0=np.zeros((B, H)))
    rc = lib.oracle_lstm_backward(T, B, I, H, _p(x), _p(w_ih), _p(w_hh), _p(_d(fwd["gates"])), _p(_d(fwd["h_all"])),
                                  _p(_d(fwd["c_all"])), _p(dY), _p(d_hn), _p(d_cn), int(flags), _p(out["dx"]),
                                  _p(out["dw_ih"]), _p(out["dw_hh"]), _p(out["db"]), _p(out["dh0"]), _p(out["dc0"]))
    if rc != 0:
        raise MemoryError("oracle_lstm_backward failed")
    return out


def pack_weights_v1(w_ih, w_hh):
    lib = _load()
    w_ih, w_hh = _d(w_ih), _d(w_hh)
    H, I = w_hh.shape[1], w_ih.shape[1]
    stride = int(lib.oracle_pack_stride_v1(I, H))
    out = np.zeros((4 * H, stride))
    lib.oracle_pack_weights_v1(I, H, _p(w_ih), _p(w_hh), _p(out))
    return out


def checkpoints(all_states, R: int):
    lib = _load()
    a = _d(all_states)
    T = a.shape[0] - 1
    n = (T + R - 1) // R
    out = np.zeros((n,) + a.shape[1:])
    lib.oracle_checkpoints(T, a.shape[1], a.shape[2], int(R), _p(a), _p(out))
    return out
