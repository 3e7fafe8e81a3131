"""ctypes front end of the CPU oracle (libw4a32_oracle.so, built from w4a32_oracle.c).

Test infrastructure only: the tests, the smoke check and the benchmark's CPU-baseline
leg import this; the shipped library never does. Every function is a thin call into
the C restatement, which cites the reference lines it follows.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libw4a32_oracle.so")
BLOCK_LEN = 32


def build(force=False):
    """Compile the oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        sz, vp, ci, fl = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.orc_bf16_from_f32_trunc.restype = ctypes.c_uint16
        L.orc_bf16_from_f32_trunc.argtypes = [fl]
        L.orc_bf16_from_f32_rne.restype = ctypes.c_uint16
        L.orc_bf16_from_f32_rne.argtypes = [fl]
        L.orc_f32_from_bf16.restype = fl
        L.orc_f32_from_bf16.argtypes = [ctypes.c_uint16]
        L.orc_fill_uniform_random.restype = None
        L.orc_fill_uniform_random.argtypes = [sz, sz, vp, sz]
        L.orc_quant_rhs_qs4c32.restype = None
        L.orc_quant_rhs_qs4c32.argtypes = [sz, sz, sz, vp, vp, vp, ci]
        L.orc_quant_lhs_qa8dx.restype = None
        L.orc_quant_lhs_qa8dx.argtypes = [sz, sz, vp, sz, vp]
        L.orc_matmul_qa8dx_qs4c32.restype = None
        L.orc_matmul_qa8dx_qs4c32.argtypes = [sz, sz, sz, sz, vp, vp, vp, vp, vp, fl, fl, ci]
        L.orc_dequant_qs4c32.restype = None
        L.orc_dequant_qs4c32.argtypes = [sz, sz, sz, vp, vp, vp]
        L.orc_linear_w4a32.restype = None
        L.orc_linear_w4a32.argtypes = [sz, sz, sz, vp, vp, vp, vp, vp, ci]
        L.orc_has_avx512_vnni.restype = ci
        L.orc_has_avx512_vnni.argtypes = []
        L.orc_linear_w4a32_vnni.restype = ci
        L.orc_linear_w4a32_vnni.argtypes = [sz, sz, sz, vp, vp, vp, vp, vp, ci]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _f32c(a):
    return np.ascontiguousarray(a, dtype=np.float32)


FLT_MAX = float(np.finfo(np.float32).max)


def bf16_trunc(v):
    return int(lib().orc_bf16_from_f32_trunc(float(np.float32(v))))


def bf16_rne(v):
    return int(lib().orc_bf16_from_f32_rne(float(np.float32(v))))


def f32_from_bf16(u):
    return float(lib().orc_f32_from_bf16(int(u)))


def fill_uniform_random(rows, cols, seed):
    out = np.empty((rows, cols), dtype=np.float32)
    lib().orc_fill_uniform_random(rows, cols, _p(out), seed)
    return out


def quant_rhs(w, bf16_rne_mode=False):
    """w f32 [N,K] -> (u4 uint8 [N,ceil(K/2)], scales uint16(bf16 bits) [N,ceil(K/32)])."""
    w = _f32c(w)
    n, k = w.shape
    u4 = np.empty((n, (k + 1) // 2), dtype=np.uint8)
    sc = np.empty((n, (k + BLOCK_LEN - 1) // BLOCK_LEN), dtype=np.uint16)
    lib().orc_quant_rhs_qs4c32(n, k, BLOCK_LEN, _p(w), _p(u4), _p(sc), int(bool(bf16_rne_mode)))
    return u4, sc


def quant_lhs(x):
    """x f32 [M,K] -> (a_q int8 [M,K], recip_scale f32 [M], neg_zero_point int32 [M])."""
    x = _f32c(x)
    m, k = x.shape
    raw = np.empty((m, k + 8), dtype=np.int8)
    lib().orc_quant_lhs_qa8dx(m, k, _p(x), k, _p(raw))
    recip = raw[:, 0:4].copy().view(np.float32).reshape(m)
    neg_zp = raw[:, 4:8].copy().view(np.int32).reshape(m)
    return raw[:, 8:].copy(), recip, neg_zp, raw


def matmul_packed(lhs_raw, u4, sc, bias=None, threads=1, lo=-FLT_MAX, hi=FLT_MAX):
    m = lhs_raw.shape[0]
    k = lhs_raw.shape[1] - 8
    n = u4.shape[0]
    out = np.empty((m, n), dtype=np.float32)
    b = _f32c(bias) if bias is not None else None
    lib().orc_matmul_qa8dx_qs4c32(m, n, k, BLOCK_LEN, _p(lhs_raw), _p(u4), _p(sc), _p(b),
                                  _p(out), lo, hi, threads)
    return out


def dequant(u4, sc, k):
    n = u4.shape[0]
    out = np.empty((n, k), dtype=np.float32)
    lib().orc_dequant_qs4c32(n, k, BLOCK_LEN, _p(u4), _p(sc), _p(out))
    return out


def linear(x, u4, sc, bias=None, threads=1):
    """The whole op: per-row int8 quantization of x, integer block dots, f32 scaling."""
    x = _f32c(x)
    m, k = x.shape
    n = u4.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    b = _f32c(bias) if bias is not None else None
    lib().orc_linear_w4a32(m, n, k, _p(x), _p(u4), _p(sc), _p(b), _p(y), threads)
    return y


def has_vnni():
    """True when this CPU runs the AVX-512 VNNI form of the product."""
    return bool(lib().orc_has_avx512_vnni())


def linear_vnni(x, u4, sc, bias=None, threads=1):
    """linear() with the block dots on vpdpbusd: same results bit for bit; raises without AVX-512 VNNI."""
    x = _f32c(x)
    m, k = x.shape
    n = u4.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    b = _f32c(bias) if bias is not None else None
    rc = lib().orc_linear_w4a32_vnni(m, n, k, _p(x), _p(u4), _p(sc), _p(b), _p(y), threads)
    if rc != 0:
        raise RuntimeError("AVX-512 VNNI form unavailable (CPU lacks it, or K is not a multiple of 32)")
    return y
