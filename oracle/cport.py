"""ctypes bindings of ``fp8_oracle.c``.  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libfp8_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (``make -C oracle``)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        i64, vp, f32, c_int = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_int
        L.orc_bf16_to_f32.restype = f32
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_bf16.argtypes = [f32]
        L.orc_e4m3_to_f32.restype = f32
        L.orc_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.orc_f32_to_e4m3.restype = ctypes.c_uint8
        L.orc_f32_to_e4m3.argtypes = [f32]
        L.orc_quant_rowwise.restype = None
        L.orc_quant_rowwise.argtypes = [vp, i64, i64, i64, vp, vp]
        L.orc_quant_static.restype = None
        L.orc_quant_static.argtypes = [vp, i64, i64, i64, f32, vp]
        L.orc_weight_quant.restype = None
        L.orc_weight_quant.argtypes = [vp, i64, i64, vp, vp]
        L.orc_linear.restype = c_int
        L.orc_linear.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, c_int, vp, vp]
        for name in ("orc_gelu_tanh", "orc_gelu_erf", "orc_silu"):
            getattr(L, name).restype = f32
            getattr(L, name).argtypes = [f32]
        L.orc_num_threads.restype = c_int
        for name in ("orc_f32_to_e4m3_array", "orc_e4m3_to_f32_array", "orc_f32_to_bf16_array"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, i64, vp]
        L.orc_act_array.restype = None
        L.orc_act_array.argtypes = [c_int, vp, i64, vp]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def quant_rowwise(x_bits: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """``x_bits``: uint16 [M, K] bf16 bit patterns -> (uint8 codes [M,K], f32 scale [M])."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    M, K = x_bits.shape
    q = np.empty((M, K), np.uint8)
    s = np.empty((M,), np.float32)
    lib().orc_quant_rowwise(_p(x_bits), M, K, K, _p(q), _p(s))
    return q, s


def quant_static(x_bits: np.ndarray, input_scale: float) -> np.ndarray:
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    M, K = x_bits.shape
    q = np.empty((M, K), np.uint8)
    lib().orc_quant_static(_p(x_bits), M, K, K, ctypes.c_float(input_scale), _p(q))
    return q


def weight_quant(w_bits: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    N, K = w_bits.shape
    q = np.empty((N, K), np.uint8)
    s = np.empty((N,), np.float32)
    lib().orc_weight_quant(_p(w_bits), N, K, _p(q), _p(s))
    return q, s


def linear(xq, x_scale, wq, w_scale, bias_bits=None, epi: int = 0, want_f32: bool = False):
    """uint8 codes + f32 scales (+ uint16 bf16 bias bits) -> uint16 bf16 bits [M, N_out]."""
    xq = np.ascontiguousarray(xq, dtype=np.uint8)
    wq = np.ascontiguousarray(wq, dtype=np.uint8)
    x_scale = np.ascontiguousarray(x_scale, dtype=np.float32).reshape(-1)
    w_scale = np.ascontiguousarray(w_scale, dtype=np.float32).reshape(-1)
    M, K = xq.shape
    N = wq.shape[0]
    n_out = N // 2 if epi in (1, 2, 3) else N
    out = np.empty((M, n_out), np.uint16)
    f32 = np.empty((M, N), np.float32) if want_f32 else None
    b = None if bias_bits is None else np.ascontiguousarray(bias_bits, dtype=np.uint16)
    rc = lib().orc_linear(_p(xq), _p(x_scale), _p(wq), _p(w_scale),
                          None if b is None else _p(b), M, N, K, int(epi), _p(out),
                          None if f32 is None else _p(f32))
    if rc != 0:
        raise RuntimeError(f"orc_linear failed rc={rc}")
    return (out, f32) if want_f32 else out


def f32_to_e4m3(v: np.ndarray) -> np.ndarray:
    """float32 array (bit patterns preserved) -> uint8 e4m3fn codes."""
    flat = np.ascontiguousarray(v, dtype=np.float32).reshape(-1)
    out = np.empty(flat.shape, np.uint8)
    lib().orc_f32_to_e4m3_array(_p(flat), flat.size, _p(out))
    return out.reshape(np.shape(v))


def e4m3_to_f32(c: np.ndarray) -> np.ndarray:
    flat = np.ascontiguousarray(c, dtype=np.uint8).reshape(-1)
    out = np.empty(flat.shape, np.float32)
    lib().orc_e4m3_to_f32_array(_p(flat), flat.size, _p(out))
    return out.reshape(np.shape(c))


def f32_to_bf16(v: np.ndarray) -> np.ndarray:
    flat = np.ascontiguousarray(v, dtype=np.float32).reshape(-1)
    out = np.empty(flat.shape, np.uint16)
    lib().orc_f32_to_bf16_array(_p(flat), flat.size, _p(out))
    return out.reshape(np.shape(v))


def act(epi: int, v: np.ndarray) -> np.ndarray:
    flat = np.ascontiguousarray(v, dtype=np.float32).reshape(-1)
    out = np.empty(flat.shape, np.float32)
    lib().orc_act_array(int(epi), _p(flat), flat.size, _p(out))
    return out.reshape(np.shape(v))
