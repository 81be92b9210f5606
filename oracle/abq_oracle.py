"""ctypes front end of the CPU oracle (oracle/abq_oracle.c) plus numpy closed forms.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
CPU-baseline leg.  The shipped library never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libabq_oracle.so")


def build(force=False):
    """Compile the C oracle (and oracle/_ref when the reference tree is mounted)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i32p = ctypes.POINTER(ctypes.c_int32)
        u32p = ctypes.POINTER(ctypes.c_uint32)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        c_int = ctypes.c_int
        L.abq_oracle_pack_i32.argtypes = [i32p, u32p, c_int, c_int, c_int]
        L.abq_oracle_pack_u4.argtypes = [u32p, u32p, c_int, c_int, c_int]
        L.abq_oracle_pack_f16.argtypes = [u16p, ctypes.c_float, u32p, c_int, c_int, c_int]
        L.abq_oracle_unpack.argtypes = [u32p, i32p, c_int, c_int, c_int, c_int]
        L.abq_oracle_gemm_bitserial.argtypes = [u32p, u32p, i32p] + [c_int] * 6
        L.abq_oracle_gemm_popc.argtypes = [u32p, u32p, i32p] + [c_int] * 7
        L.abq_oracle_gemm_popc.restype = c_int
        L.abq_oracle_gemm_int.argtypes = [i32p, i32p, i32p, c_int, c_int, c_int]
        L.abq_oracle_gemm_int.restype = c_int
        L.abq_oracle_epilogue_f16.argtypes = [i32p, ctypes.c_uint16, u16p, c_int]
        L.abq_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.abq_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.abq_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.abq_oracle_f16_to_f32.restype = ctypes.c_float
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def pack_i32(values, bits):
    """values int32 [rows, k] -> planes uint32 [bits, rows, k/32]."""
    v = np.ascontiguousarray(values, dtype=np.int32)
    rows, k = v.shape
    assert k % 32 == 0
    out = np.zeros((bits, rows, k // 32), dtype=np.uint32)
    lib().abq_oracle_pack_i32(_p(v, ctypes.c_int32), _p(out, ctypes.c_uint32), rows, k, bits)
    return out


def pack_u4(words, rows, k, bits=4):
    """words uint32 [rows*k/8] (8 nibbles per word, first element in the top nibble)."""
    w = np.ascontiguousarray(words, dtype=np.uint32)
    assert w.size == rows * k // 8 and k % 32 == 0
    out = np.zeros((bits, rows, k // 32), dtype=np.uint32)
    lib().abq_oracle_pack_u4(_p(w, ctypes.c_uint32), _p(out, ctypes.c_uint32), rows, k, bits)
    return out


def pack_f16(values_f16, scale, bits):
    """values float16 [rows, k], scale python float -> planes."""
    v = np.ascontiguousarray(values_f16, dtype=np.float16)
    rows, k = v.shape
    out = np.zeros((bits, rows, k // 32), dtype=np.uint32)
    lib().abq_oracle_pack_f16(_p(v.view(np.uint16), ctypes.c_uint16), float(scale),
                              _p(out, ctypes.c_uint32), rows, k, bits)
    return out


def unpack(planes, signed):
    p = np.ascontiguousarray(planes, dtype=np.uint32)
    bits, rows, kw = p.shape
    out = np.zeros((rows, kw * 32), dtype=np.int32)
    lib().abq_oracle_unpack(_p(p, ctypes.c_uint32), _p(out, ctypes.c_int32), rows, kw * 32, bits,
                            int(bool(signed)))
    return out


def gemm_bitserial(x_planes, w_planes, signed):
    xp = np.ascontiguousarray(x_planes, dtype=np.uint32)
    wp = np.ascontiguousarray(w_planes, dtype=np.uint32)
    q, M, kw = xp.shape
    p, N, kw2 = wp.shape
    assert kw == kw2
    d = np.zeros((M, N), dtype=np.int32)
    lib().abq_oracle_gemm_bitserial(_p(wp, ctypes.c_uint32), _p(xp, ctypes.c_uint32),
                                    _p(d, ctypes.c_int32), M, N, kw * 32, p, q, int(bool(signed)))
    return d


def gemm_popc(x_planes, w_planes, signed, threads=0):
    xp = np.ascontiguousarray(x_planes, dtype=np.uint32)
    wp = np.ascontiguousarray(w_planes, dtype=np.uint32)
    q, M, kw = xp.shape
    p, N, kw2 = wp.shape
    assert kw == kw2
    d = np.zeros((M, N), dtype=np.int32)
    used = lib().abq_oracle_gemm_popc(_p(wp, ctypes.c_uint32), _p(xp, ctypes.c_uint32),
                                      _p(d, ctypes.c_int32), M, N, kw * 32, p, q,
                                      int(bool(signed)), int(threads))
    return d, used


def gemm_int(x_int, w_int):
    x = np.ascontiguousarray(x_int, dtype=np.int32)
    w = np.ascontiguousarray(w_int, dtype=np.int32)
    M, K = x.shape
    N, K2 = w.shape
    assert K == K2
    d = np.zeros((M, N), dtype=np.int32)
    ovf = lib().abq_oracle_gemm_int(_p(x, ctypes.c_int32), _p(w, ctypes.c_int32),
                                    _p(d, ctypes.c_int32), M, N, K)
    assert ovf == 0, "result does not fit int32"
    return d


def epilogue_f16(acc, scale_f16):
    a = np.ascontiguousarray(acc, dtype=np.int32)
    out = np.zeros(a.shape, dtype=np.uint16)
    s = np.array([scale_f16], dtype=np.float16).view(np.uint16)[0]
    lib().abq_oracle_epilogue_f16(_p(a, ctypes.c_int32), int(s), _p(out, ctypes.c_uint16), a.size)
    return out.view(np.float16)


# --------------------------------------------------------------------------- numpy closed forms

def value_range(bits, signed):
    return (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if signed else (0, (1 << bits) - 1)


def np_pack(values, bits):
    """Independent numpy statement of the plane layout (engine/common/pack.cu:54-62):
    bit (31-e) of planes[b, r, j] is bit b of values[r, 32j+e]."""
    v = np.asarray(values).astype(np.int64)
    rows, k = v.shape
    g = (v.reshape(rows, k // 32, 32) & 0xFFFFFFFF).astype(np.uint64)
    shifts = (31 - np.arange(32)).astype(np.uint64)
    out = np.zeros((bits, rows, k // 32), dtype=np.uint32)
    for b in range(bits):
        out[b] = (((g >> np.uint64(b)) & np.uint64(1)) << shifts).sum(axis=2).astype(np.uint32)
    return out


def np_gemm(x_int, w_int):
    """Closed form D = X . W^T in int64 (then checked to fit int32)."""
    d = np.asarray(x_int, dtype=np.int64) @ np.asarray(w_int, dtype=np.int64).T
    assert np.abs(d).max(initial=0) < 2 ** 31
    return d.astype(np.int32)
