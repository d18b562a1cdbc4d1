"""ctypes/numpy front end of the CPU checker (TEST INFRASTRUCTURE ONLY).

Loads ``liborc.so`` (scalar restatement of the reference, the parity oracle) and
``liborc_simd.so`` (restatement of the reference's x86 SIMD dispatch kernels, the
timed CPU baseline).  Nothing in the shipped package imports this module; only
the tests, the smoke check and the benchmark's ``cpu_baseline`` leg do.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_sz = C.c_size_t


def build(force: bool = False) -> None:
    """Compile both checker libraries with the Makefile beside this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE, "all"], check=True, capture_output=True)


def _load(name: str) -> C.CDLL:
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    return C.CDLL(path)


_orc = None
_simd = None


def orc() -> C.CDLL:
    global _orc
    if _orc is None:
        _orc = _load("liborc.so")
        _orc.orc_fp16_bits_to_f32.restype = C.c_float
        _orc.orc_fp16_bits_to_f32.argtypes = [C.c_uint16]
        _orc.orc_bf16_bits_to_f32.restype = C.c_float
        _orc.orc_bf16_bits_to_f32.argtypes = [C.c_uint16]
        _orc.orc_f32_to_fp16_bits.restype = C.c_uint16
        _orc.orc_f32_to_fp16_bits.argtypes = [C.c_float]
        _orc.orc_f32_to_bf16_bits.restype = C.c_uint16
        _orc.orc_f32_to_bf16_bits.argtypes = [C.c_float]
        for fn in ("orc_unpack_low", "orc_unpack_high", "orc_nibble_lo", "orc_nibble_hi"):
            getattr(_orc, fn).restype = C.c_int8
            getattr(_orc, fn).argtypes = [C.c_uint8]
        _orc.orc_argmax_last.restype = C.c_uint32
    return _orc


def simd() -> C.CDLL:
    global _simd
    if _simd is None:
        _simd = _load("liborc_simd.so")
        _simd.simd_pack_i8_b_for_matmul.restype = C.c_void_p
    return _simd


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# ---- conversions -------------------------------------------------------------

def fp16_bits_to_f32(bits) -> np.ndarray:
    b = _c(bits, np.uint16)
    out = np.empty(b.shape, np.float32)
    orc().orc_fp16_to_f32_array(_p(b), _p(out), _sz(b.size))
    return out


def bf16_bits_to_f32(bits) -> np.ndarray:
    b = _c(bits, np.uint16)
    out = np.empty(b.shape, np.float32)
    orc().orc_bf16_to_f32_array(_p(b), _p(out), _sz(b.size))
    return out


def f32_to_bf16_bits(x) -> np.ndarray:
    v = _c(x, np.float32)
    out = np.empty(v.shape, np.uint16)
    orc().orc_f32_to_bf16_array(_p(v), _p(out), _sz(v.size))
    return out


def f32_to_fp16_bits_trunc(x) -> np.ndarray:
    v = _c(x, np.float32)
    out = np.empty(v.shape, np.uint16)
    orc().orc_f32_to_fp16_array(_p(v), _p(out), _sz(v.size))
    return out


# ---- int4 ----------------------------------------------------------------------

def packed_int4_gemv_scalar(weight_packed, scales, activation, m_w, k, group_size) -> np.ndarray:
    w, s, x = _c(weight_packed, np.uint8), _c(scales, np.float32), _c(activation, np.float32)
    assert w.size == m_w * k // 2 and s.size == m_w * (k // group_size) and x.size == k
    out = np.empty(m_w, np.float32)
    orc().orc_packed_int4_gemv_scalar(_p(w), _p(s), _p(x), _p(out), _sz(m_w), _sz(k), _sz(group_size))
    return out


def packed_int4_gemm_scalar(weight_packed, scales, activation, m, n, k, group_size) -> np.ndarray:
    w, s, x = _c(weight_packed, np.uint8), _c(scales, np.float32), _c(activation, np.float32)
    assert w.size == n * k // 2 and s.size == n * (k // group_size) and x.size == m * k
    out = np.empty((m, n), np.float32)
    orc().orc_packed_int4_gemm_scalar(_p(w), _p(s), _p(x), _p(out), _sz(m), _sz(n), _sz(k), _sz(group_size))
    return out


def pack_int4_symmetric_per_group(weights, m_w, k, group_size):
    w = _c(weights, np.float32)
    assert w.size == m_w * k
    packed = np.empty(m_w * k // 2, np.uint8)
    scales = np.empty(m_w * (k // group_size), np.float32)
    orc().orc_pack_int4_symmetric_per_group(_p(w), _sz(m_w), _sz(k), _sz(group_size), _p(packed), _p(scales))
    return packed, scales


def dequantize_int4_to_f32(packed, scale, zero_point) -> np.ndarray:
    b = _c(packed, np.uint8)
    out = np.empty(b.size * 2, np.float32)
    orc().orc_dequantize_int4_to_f32(_p(b), _sz(b.size), C.c_float(scale), C.c_int8(zero_point), _p(out))
    return out


def quantize_f32_to_int4(data, scale, zero_point) -> np.ndarray:
    d = _c(data, np.float32)
    out = np.empty((d.size + 1) // 2, np.uint8)
    orc().orc_quantize_f32_to_int4(_p(d), _sz(d.size), C.c_float(scale), C.c_int8(zero_point), _p(out))
    return out


def matmul_nbits(b, scales, zero_points, activation, m, n, k, group_size) -> np.ndarray:
    """MatMulNBits definition: uint4 nibbles, per-group scale and uint4 zero point (None => 8)."""
    bb, s, x = _c(b, np.uint8), _c(scales, np.float32), _c(activation, np.float32)
    zp = None if zero_points is None else _c(zero_points, np.uint8)
    out = np.empty((m, n), np.float32)
    orc().orc_matmul_nbits_dequant_dot(_p(bb), _p(s), _p(zp) if zp is not None else None, _p(x), _p(out),
                                       _sz(m), _sz(n), _sz(k), _sz(group_size))
    return out


# ---- int8 ----------------------------------------------------------------------

def int8_matmul_scalar(a, b, m, k, n) -> np.ndarray:
    aa, bb = _c(a, np.int8), _c(b, np.int8)
    assert aa.size == m * k and bb.size == k * n
    out = np.empty((m, n), np.int32)
    orc().orc_int8_matmul_scalar(_p(aa), _p(bb), _sz(m), _sz(k), _sz(n), _p(out))
    return out


def transpose_b(b, k, n) -> np.ndarray:
    bb = _c(b, np.int8)
    bt = np.empty(n * k, np.int8)
    orc().orc_transpose_b(_p(bb), _sz(k), _sz(n), _p(bt))
    return bt


def int8_matmul_prepacked_scalar(a, bt, m, k, n) -> np.ndarray:
    aa, bb = _c(a, np.int8), _c(bt, np.int8)
    out = np.empty((m, n), np.int32)
    orc().orc_int8_matmul_prepacked_scalar(_p(aa), _p(bb), _sz(m), _sz(k), _sz(n), _p(out))
    return out


def i8_col_sums(b, k, n) -> np.ndarray:
    bb = _c(b, np.int8)
    out = np.empty(n, np.int32)
    orc().orc_i8_col_sums(_p(bb), _sz(k), _sz(n), _p(out))
    return out


def u8i8_matmul_zp(a, a_zp, b, m, k, n) -> np.ndarray:
    aa, bb = _c(a, np.uint8), _c(b, np.int8)
    out = np.empty((m, n), np.int32)
    orc().orc_u8i8_matmul_zp(_p(aa), C.c_int32(a_zp), _p(bb), _sz(m), _sz(k), _sz(n), _p(out))
    return out


# ---- quantize / requantize -------------------------------------------------------

def quantize_linear_f32_to_i8(data, scale, zero_point) -> np.ndarray:
    d = _c(data, np.float32)
    out = np.empty(d.shape, np.int8)
    orc().orc_quantize_linear_f32_to_i8(_p(d), _sz(d.size), C.c_float(scale), C.c_float(zero_point), _p(out))
    return out


def quantize_linear_f32_to_f32_i8(data, scale, zero_point) -> np.ndarray:
    d = _c(data, np.float32)
    out = np.empty(d.shape, np.float32)
    orc().orc_quantize_linear_f32_to_f32_i8(_p(d), _sz(d.size), C.c_float(scale), C.c_float(zero_point), _p(out))
    return out


def requant_i32_row_to_i8(acc, bias, composite, y_zp, relu, c) -> np.ndarray:
    a = _c(acc, np.int32)
    b = None if bias is None else _c(bias, np.int32)
    out = np.empty(a.shape, np.int8)
    orc().orc_requant_i32_row_to_i8(_p(a), _sz(a.size), _p(b) if b is not None else None,
                                    C.c_float(composite), C.c_float(y_zp), C.c_int(int(relu)), _p(out), _sz(c))
    return out


def requant_i8_per_channel(acc, corr, composite, y_zp, c) -> np.ndarray:
    a, co, cp = _c(acc, np.int32), _c(corr, np.int32), _c(composite, np.float32)
    out = np.empty(a.shape, np.int8)
    orc().orc_requant_i8_per_channel(_p(a), _sz(a.size), _p(co), _p(cp), C.c_float(y_zp), _p(out), _sz(c))
    return out


ROUND_HALF_AWAY = 0
ROUND_TIES_EVEN = 1


def requant_general(acc, c, corr, composite, y_zp, round_mode, lo, hi) -> np.ndarray:
    """composite: float (per tensor) or array of length c (per channel).  Returns int32."""
    a = _c(acc, np.int32)
    co = None if corr is None else _c(corr, np.int32)
    if np.ndim(composite) == 0:
        cv, cs = None, float(composite)
    else:
        cv, cs = _c(composite, np.float32), 0.0
    out = np.empty(a.shape, np.int32)
    orc().orc_requant_general(_p(a), _sz(a.size), _sz(c), _p(co) if co is not None else None,
                              _p(cv) if cv is not None else None, C.c_float(cs), C.c_float(y_zp),
                              C.c_int(round_mode), C.c_float(lo), C.c_float(hi), _p(out))
    return out


def dynamic_quantize_linear(x):
    d = _c(x, np.float32)
    y = np.empty(d.shape, np.float32)
    s, z = C.c_float(), C.c_float()
    orc().orc_dynamic_quantize_linear(_p(d), _sz(d.size), _p(y), C.byref(s), C.byref(z))
    return y, np.float32(s.value), np.float32(z.value)


def dequantize_linear(q, scale, zp) -> np.ndarray:
    d = _c(q, np.float32)
    out = np.empty(d.shape, np.float32)
    orc().orc_dequantize_linear(_p(d), _sz(d.size), C.c_float(scale), C.c_float(zp), _p(out))
    return out


def exec_matmul_integer(a, b, a_zp, b_zp, m, k, n):
    aa, bb = _c(a, np.float32), _c(b, np.float32)
    out = np.empty((m, n), np.float32)
    fast = orc().orc_exec_matmul_integer(_p(aa), _p(bb), C.c_float(a_zp), C.c_float(b_zp), _sz(m), _sz(k), _sz(n), _p(out))
    return out, bool(fast)


def exec_qlinear_matmul(a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp, m, k, n):
    aa, bb = _c(a, np.float32), _c(b, np.float32)
    out = np.empty((m, n), np.float32)
    fast = orc().orc_exec_qlinear_matmul(_p(aa), C.c_float(a_scale), C.c_float(a_zp), _p(bb), C.c_float(b_scale),
                                         C.c_float(b_zp), C.c_float(y_scale), C.c_float(y_zp),
                                         _sz(m), _sz(k), _sz(n), _p(out))
    return out, bool(fast)


def should_use_prepacked_i8_b(m, k, n) -> bool:
    return bool(orc().orc_should_use_prepacked_i8_b(_sz(m), _sz(k), _sz(n)))


def should_prepack_i8_b(k, n) -> bool:
    return bool(orc().orc_should_prepack_i8_b(_sz(k), _sz(n)))


def kv_i8_quantize_rows(src, rows, kv_dim):
    s = _c(src, np.float32)
    data = np.empty(rows * kv_dim, np.int8)
    scales = np.empty(rows, np.float32)
    orc().orc_kv_i8_quantize_rows(_p(s), _sz(rows), _sz(kv_dim), _p(data), _p(scales))
    return data, scales


def argmax_last(logits) -> int:
    v = _c(logits, np.float32)
    return int(orc().orc_argmax_last(_p(v), _sz(v.size)))


def lcg_i8(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, np.int8)
    orc().orc_lcg_i8(C.c_uint64(seed), _sz(n), _p(out))
    return out


def lcg_f32(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, np.float32)
    orc().orc_lcg_f32(C.c_uint64(seed), _sz(n), _p(out))
    return out


# ---- SIMD restatement (timed CPU baseline) ----------------------------------------

def simd_packed_int4_gemv_dispatch(w, s, x, m_w, k, g, threads: int = 1) -> np.ndarray:
    ww, ss, xx = _c(w, np.uint8), _c(s, np.float32), _c(x, np.float32)
    out = np.empty(m_w, np.float32)
    if threads <= 1:
        simd().simd_packed_int4_gemv_dispatch(_p(ww), _p(ss), _p(xx), _p(out), _sz(m_w), _sz(k), _sz(g))
    else:
        simd().simd_packed_int4_gemv_dispatch_mt(_p(ww), _p(ss), _p(xx), _p(out), _sz(m_w), _sz(k), _sz(g), C.c_int(threads))
    return out


def simd_packed_int4_gemm_dispatch(w, s, x, m, n, k, g, threads: int = 1) -> np.ndarray:
    ww, ss, xx = _c(w, np.uint8), _c(s, np.float32), _c(x, np.float32)
    out = np.empty((m, n), np.float32)
    if threads <= 1:
        simd().simd_packed_int4_gemm_dispatch(_p(ww), _p(ss), _p(xx), _p(out), _sz(m), _sz(n), _sz(k), _sz(g))
    else:
        simd().simd_packed_int4_gemm_dispatch_mt(_p(ww), _p(ss), _p(xx), _p(out), _sz(m), _sz(n), _sz(k), _sz(g), C.c_int(threads))
    return out


def simd_int8_matmul_dispatch(a, b, m, k, n) -> np.ndarray:
    aa, bb = _c(a, np.int8), _c(b, np.int8)
    out = np.empty((m, n), np.int32)
    simd().simd_int8_matmul_dispatch(_p(aa), _p(bb), _sz(m), _sz(k), _sz(n), _p(out))
    return out


class SimdPackedI8B:
    """pack_i8_b_for_matmul handle of the SIMD restatement."""

    def __init__(self, b, k, n):
        self.b = _c(b, np.int8)
        self.k, self.n = k, n
        self.h = C.c_void_p(simd().simd_pack_i8_b_for_matmul(_p(self.b), _sz(k), _sz(n)))

    def matmul(self, a, m, threads: int = 1) -> np.ndarray:
        aa = _c(a, np.int8)
        out = np.empty((m, self.n), np.int32)
        if threads <= 1:
            simd().simd_int8_matmul_prepacked_dispatch(_p(aa), self.h, _p(self.b), _sz(m), _p(out))
        else:
            simd().simd_int8_matmul_prepacked_dispatch_mt(_p(aa), self.h, _p(self.b), _sz(m), _p(out), C.c_int(threads))
        return out

    def __del__(self):
        try:
            simd().simd_packed_i8b_free(self.h)
        except Exception:
            pass


def simd_paths(group_size: int = 32) -> dict:
    names = {0: "scalar", 1: "avx2", 2: "avx512", 3: "avx512-vnni"}
    s = simd()
    return {
        "int4_gemv": names[s.simd_int4_gemv_path(_sz(group_size))],
        "int4_gemm": names[s.simd_int4_gemm_path(_sz(group_size))],
        "int8": names[s.simd_int8_path()],
        "omp_max_threads": s.simd_max_threads(),
    }
