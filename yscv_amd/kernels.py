"""Host-side mirror of the yscv-kernels entry points for this path, over the C ABI.

Names and argument order follow crates/yscv-kernels/src/core.rs:173-186.  The host-slice
functions take numpy arrays (the Rust ``&[T]`` / ``&mut [T]`` slices); the handle classes own
device memory and take torch CUDA tensors, which are used only as device buffers -- every
computation happens inside libyscv_hip.so.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from .capi import (BF16, EPILOGUE_ADD_F32, EPILOGUE_STORE, EPILOGUE_SWIGLU, F16, F32, NIBBLE_SIGNED, NIBBLE_UNSIGNED,
                   ROUND_HALF_AWAY, ROUND_TIES_EVEN, lib)

_sz = C.c_size_t


def _np(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _torch_dtype_code(t) -> int:
    import torch

    return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}[t.dtype]


def _stream_ptr():
    import torch

    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


# ---- host-slice entry points (exact Rust argument lists) ---------------------------------

def packed_int4_gemv_dispatch(weight_packed, scales, activation, output, m_w, k, group_size) -> None:
    """int4_matmul.rs:310 -- output[m_w] = W[m_w][k] . activation[k]."""
    w, s, x = _np(weight_packed, np.uint8), _np(scales, np.float32), _np(activation, np.float32)
    assert isinstance(output, np.ndarray) and output.dtype == np.float32 and output.flags.c_contiguous
    if w.size != m_w * k // 2 or s.size != m_w * (k // max(group_size, 1)) or x.size != k or output.size != m_w:
        raise ValueError("slice lengths do not match m_w, k, group_size")
    lib().packed_int4_gemv_dispatch(_ptr(w), _ptr(s), _ptr(x), _ptr(output), _sz(m_w), _sz(k), _sz(group_size))


def packed_int4_gemm_dispatch(weight_packed, scales, activation, output, m, n, k, group_size) -> None:
    """int4_matmul.rs:548 -- output[m][n] = activation[m][k] . W[n][k]^T."""
    w, s, x = _np(weight_packed, np.uint8), _np(scales, np.float32), _np(activation, np.float32)
    assert isinstance(output, np.ndarray) and output.dtype == np.float32 and output.flags.c_contiguous
    if w.size != n * k // 2 or s.size != n * (k // max(group_size, 1)) or x.size != m * k or output.size != m * n:
        raise ValueError("slice lengths do not match m, n, k, group_size")
    lib().packed_int4_gemm_dispatch(_ptr(w), _ptr(s), _ptr(x), _ptr(output), _sz(m), _sz(n), _sz(k), _sz(group_size))


def pack_int4_symmetric_per_group(weights, m_w, k, group_size):
    """int4_matmul.rs:611 -- returns (packed u8[m_w*k/2], scales f32[m_w*k/group_size])."""
    w = _np(weights, np.float32)
    if w.size != m_w * k:
        raise ValueError("weights length != m_w * k")
    packed = np.empty(m_w * k // 2, np.uint8)
    scales = np.empty(m_w * (k // group_size), np.float32)
    lib().pack_int4_symmetric_per_group(_ptr(w), _sz(m_w), _sz(k), _sz(group_size), _ptr(packed), _ptr(scales))
    return packed, scales


def dequantize_int4_to_f32(packed, scale, zero_point, output) -> None:
    """ops/quantize.rs:18."""
    p = _np(packed, np.uint8)
    assert output.dtype == np.float32 and output.size >= 2 * p.size
    lib().dequantize_int4_to_f32(_ptr(p), _sz(p.size), C.c_float(scale), C.c_int8(zero_point), _ptr(output))


def quantize_f32_to_int4(data, scale, zero_point, output) -> None:
    """ops/quantize.rs:69 -- output holds (len + 1) / 2 bytes."""
    d = _np(data, np.float32)
    assert output.dtype == np.uint8 and output.size >= (d.size + 1) // 2
    lib().quantize_f32_to_int4(_ptr(d), _sz(d.size), C.c_float(scale), C.c_int8(zero_point), _ptr(output))


def int8_matmul_dispatch(a, b, m, k, n, out) -> None:
    """int8_matmul.rs:2407 -- b is row-major [k][n]."""
    aa, bb = _np(a, np.int8), _np(b, np.int8)
    assert out.dtype == np.int32 and out.flags.c_contiguous
    if aa.size != m * k or bb.size != k * n or out.size != m * n:
        raise ValueError("slice lengths do not match m, k, n")
    lib().int8_matmul_dispatch(_ptr(aa), _ptr(bb), _sz(m), _sz(k), _sz(n), _ptr(out))


def quantize_linear_f32_to_i8_dispatch(data, scale, zero_point, output) -> None:
    """ops/quantize.rs:154."""
    d = _np(data, np.float32)
    assert output.dtype == np.int8 and output.size == d.size
    lib().quantize_linear_f32_to_i8_dispatch(_ptr(d), _sz(d.size), C.c_float(scale), C.c_float(zero_point), _ptr(output))


def requant_i8_per_channel_dispatch(acc, corr, composite, y_zp, out, c) -> None:
    """ops/int8_requant.rs:401."""
    a, co, cp = _np(acc, np.int32), _np(corr, np.int32), _np(composite, np.float32)
    assert out.dtype == np.int8 and out.size == a.size
    lib().requant_i8_per_channel_dispatch(_ptr(a), _sz(a.size), _ptr(co), _ptr(cp), C.c_float(y_zp), _ptr(out), _sz(c))


def requant_i32_row_to_i8_dispatch(acc, bias, composite, y_zp, relu, out, c) -> None:
    """ops/int8_requant.rs:81 -- bias may be None."""
    a = _np(acc, np.int32)
    b = None if bias is None else _np(bias, np.int32)
    assert out.dtype == np.int8 and out.size == a.size
    lib().requant_i32_row_to_i8_dispatch(_ptr(a), _sz(a.size), _ptr(b) if b is not None else None,
                                         C.c_float(composite), C.c_float(y_zp), C.c_int32(int(bool(relu))), _ptr(out), _sz(c))


def dynamic_quantize_linear(x):
    """runner/misc.rs:241 -- returns (y uint8, scale f32, zero_point f32)."""
    d = _np(x, np.float32)
    y = np.empty(d.shape, np.uint8)
    s, z = C.c_float(), C.c_float()
    lib().dynamic_quantize_linear_host(_ptr(d), _sz(d.size), _ptr(y), C.byref(s), C.byref(z))
    return y, np.float32(s.value), np.float32(z.value)


def kv_i8_quantize_rows(src):
    """KvCache int8 append (runner/kv_cache.rs:45-61): src CUDA f32 [rows][kv_dim] -> (int8 [rows][kv_dim], f32 [rows])."""
    import torch

    assert src.is_cuda and src.dtype == torch.float32 and src.dim() == 2
    src = src.contiguous()
    rows, kv_dim = int(src.shape[0]), int(src.shape[1])
    data = torch.empty(rows, kv_dim, device=src.device, dtype=torch.int8)
    scales = torch.empty(rows, device=src.device, dtype=torch.float32)
    lib().kv_i8_quantize_rows(C.c_void_p(src.data_ptr()), _sz(rows), _sz(kv_dim), C.c_void_p(data.data_ptr()),
                              C.c_void_p(scales.data_ptr()), _stream_ptr())
    return data, scales


def kv_i8_dequantize_rows(data, scales):
    """KvCache int8 read (runner/kv_cache.rs:64-79)."""
    import torch

    assert data.is_cuda and data.dtype == torch.int8 and data.dim() == 2 and scales.dtype == torch.float32
    rows, kv_dim = int(data.shape[0]), int(data.shape[1])
    out = torch.empty(rows, kv_dim, device=data.device, dtype=torch.float32)
    lib().kv_i8_dequantize_rows(C.c_void_p(data.contiguous().data_ptr()), C.c_void_p(scales.contiguous().data_ptr()), _sz(rows),
                                _sz(kv_dim), C.c_void_p(out.data_ptr()), _stream_ptr())
    return out


# ---- packed int4 weight files (host only; the reference has no on-disk form of PackedInt4Weight) ----------

def int4_file_write(path, packed, scales, group_size, m_w, k, zero_points=None, nibble_format=NIBBLE_SIGNED) -> None:
    """Stores the arguments of PackedInt4Weight(...) behind the 64-byte header of the packed-int4 file format."""
    p = _np(packed, np.uint8)
    s = np.ascontiguousarray(scales)
    if s.dtype not in (np.float32, np.float16):
        raise TypeError("scales must be float32 or float16")
    zp = None if zero_points is None else _np(zero_points, np.uint8)
    if group_size <= 0 or p.size != m_w * k // 2 or s.size != m_w * (k // group_size):
        raise ValueError("slice lengths do not match m_w, k, group_size")
    lib().int4_file_write(str(path).encode(), _ptr(p), _ptr(s), F32 if s.dtype == np.float32 else F16,
                          _ptr(zp) if zp is not None else None, nibble_format, _sz(m_w), _sz(k), _sz(group_size))


def int4_file_read_header(path):
    h = capi.Int4FileHeader()
    lib().int4_file_read_header(str(path).encode(), C.byref(h))
    return h


def int4_file_read(path):
    """-> (packed u8, scales f32|f16, zero_points u8|None, header); the checksum is verified."""
    h = int4_file_read_header(path)
    packed = np.empty(h.packed_bytes, np.uint8)
    sdt = np.float32 if h.scale_dtype == F32 else np.float16
    scales = np.empty(h.scales_bytes // np.dtype(sdt).itemsize, sdt)
    zps = np.empty(h.zero_points_bytes, np.uint8) if h.has_zero_points else None
    lib().int4_file_read(str(path).encode(), _ptr(packed), _sz(packed.size), _ptr(scales), _sz(scales.nbytes),
                         _ptr(zps) if zps is not None else None, _sz(0 if zps is None else zps.size))
    return packed, scales, zps, h


# ---- device handles ---------------------------------------------------------------------------

class PackedInt4Weight:
    """Device-resident PackedInt4Weight (quantize/packed_int4.rs:29-39): packed nibbles + scales
    (+ optional uint4 zero points for the MatMulNBits form), re-tiled for the MFMA kernels."""

    def __init__(self, packed, scales, group_size, m_w, k, zero_points=None, nibble_format=NIBBLE_SIGNED):
        p = _np(packed, np.uint8)
        s = np.ascontiguousarray(scales)
        if s.dtype == np.float32:
            sd = F32
        elif s.dtype == np.float16:
            sd = F16
        else:
            raise TypeError("scales must be float32 or float16")
        zp = None if zero_points is None else _np(zero_points, np.uint8)
        if group_size <= 0 or p.size != m_w * k // 2 or s.size != m_w * (k // group_size):
            raise ValueError("slice lengths do not match m_w, k, group_size")
        h = C.c_void_p()
        lib().int4_weight_create(_ptr(p), _ptr(s), sd, _ptr(zp) if zp is not None else None, nibble_format,
                                 _sz(m_w), _sz(k), _sz(group_size), C.byref(h))
        self._h = h
        self.m_w, self.k, self.group_size = m_w, k, group_size

    @classmethod
    def from_f32(cls, weight, group_size, transposed_nk=False):
        """quantize_matmul_weights_int4_packed (quantize/packed_int4.rs:50-128) for one initialiser: weight is a CUDA
        f32 tensor of shape [K, N] (MatMul, Gemm transB=0) or, with transposed_nk, [N, K] (Gemm transB=1).
        Returns None for a weight the reference skips (K % group_size != 0 or K * N < 32)."""
        import torch

        assert weight.is_cuda and weight.dtype == torch.float32 and weight.dim() == 2
        weight = weight.contiguous()
        d0, d1 = int(weight.shape[0]), int(weight.shape[1])
        h = C.c_void_p()
        lib().int4_weight_from_f32(C.c_void_p(weight.data_ptr()), _sz(d0), _sz(d1), 1 if transposed_nk else 0,
                                   _sz(group_size), _stream_ptr(), C.byref(h))
        if not h:
            return None
        self = cls.__new__(cls)
        self._h = h
        self.m_w, self.k = (d0, d1) if transposed_nk else (d1, d0)
        self.group_size = group_size
        return self

    @classmethod
    def load(cls, path):
        """Reads a packed-int4 weight file (int4_file_write) and uploads it."""
        hdr = int4_file_read_header(path)
        h = C.c_void_p()
        lib().int4_weight_load(str(path).encode(), C.byref(h))
        self = cls.__new__(cls)
        self._h = h
        self.m_w, self.k, self.group_size = int(hdr.n), int(hdr.k), int(hdr.group_size)
        return self

    @property
    def handle(self):
        return self._h

    def device_bytes(self) -> int:
        n, k, g, b = _sz(), _sz(), _sz(), _sz()
        lib().int4_weight_dims(self._h, C.byref(n), C.byref(k), C.byref(g), C.byref(b))
        return b.value

    def workspace_bytes(self, m: int, x_dtype) -> int:
        """Scratch yscv_hip_int4_matmul_ws needs for m rows of activations of torch dtype x_dtype (0 = none)."""
        import torch

        code = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}[x_dtype]
        b = _sz()
        lib().int4_workspace_bytes(self._h, _sz(m), code, C.byref(b))
        return b.value

    def matmul(self, x, out=None, out_dtype=None, mode: str = "auto", workspace=None):
        """x: CUDA tensor [..., k] (f32/f16/bf16).  mode: auto | gemv | gemm.  Output shape is
        x.shape[:-1] + [m_w], like exec_matmul's int4 branch (runner/linear.rs:269-270).  With `workspace` (a CUDA
        uint8 tensor of at least workspace_bytes(m, x.dtype), 256-byte aligned) the call allocates nothing
        (yscv_hip_int4_matmul_ws, mode auto only)."""
        import torch

        assert x.is_cuda and x.shape[-1] == self.k
        x = x.contiguous()
        m = x.numel() // self.k
        odt = out_dtype or x.dtype
        if out is None:
            out = torch.empty(*x.shape[:-1], self.m_w, device=x.device, dtype=odt)
        if workspace is not None:
            assert mode == "auto" and workspace.is_cuda and workspace.dtype == torch.uint8
            lib().int4_matmul_ws(self._h, C.c_void_p(x.data_ptr()), _torch_dtype_code(x), C.c_void_p(out.data_ptr()),
                                 _torch_dtype_code(out), _sz(m), C.c_void_p(workspace.data_ptr()),
                                 _sz(workspace.numel()), _stream_ptr())
            return out
        fn = {"auto": lib().int4_matmul, "gemv": lib().int4_gemv, "gemm": lib().int4_gemm}[mode]
        fn(self._h, C.c_void_p(x.data_ptr()), _torch_dtype_code(x), C.c_void_p(out.data_ptr()),
           _torch_dtype_code(out), _sz(m), _stream_ptr())
        return out

    def matmul_static(self, x, out):
        """yscv_hip_int4_matmul_static: scratch in the library's static device array, nothing allocated by the call
        (`out` comes from the caller for the same reason)."""
        assert x.is_cuda and out.is_cuda and x.is_contiguous() and out.is_contiguous() and x.shape[-1] == self.k
        m = x.numel() // self.k
        assert out.numel() == m * self.m_w
        lib().int4_matmul_static(self._h, C.c_void_p(x.data_ptr()), _torch_dtype_code(x), C.c_void_p(out.data_ptr()),
                                 _torch_dtype_code(out), _sz(m), _stream_ptr())
        return out

    def matmul_fused(self, x, out, epilogue: int):
        """yscv_hip_int4_matmul_fused: the int4 matmul with the epilogue fused (skinny kernel up to 16 rows, the LDS-ring GEMM
        above with 16-bit activations).  EPILOGUE_ADD_F32 adds into the
        f32 tensor `out` [m, m_w]; EPILOGUE_SWIGLU writes silu(gate) * up into `out` [m, m_w / 2]."""
        assert x.is_cuda and out.is_cuda and x.shape[-1] == self.k
        x = x.contiguous()
        m = x.numel() // self.k
        assert out.is_contiguous() and out.numel() == m * (self.m_w // 2 if epilogue == 2 else self.m_w)
        lib().int4_matmul_fused(self._h, C.c_void_p(x.data_ptr()), _torch_dtype_code(x), C.c_void_p(out.data_ptr()),
                                _torch_dtype_code(out), _sz(m), int(epilogue), _stream_ptr())
        return out

    def close(self):
        if self._h:
            lib().int4_weight_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class PackedI8B:
    """Device-resident PackedI8B (int8_matmul.rs:128-160)."""

    def __init__(self, b, k, n):
        bb = _np(b, np.int8)
        if bb.size != k * n:
            raise ValueError("b length != k * n")
        h = C.c_void_p()
        lib().pack_i8_b_for_matmul(_ptr(bb), _sz(k), _sz(n), C.byref(h))
        self._h = h
        self._k, self._n = k, n

    def k(self) -> int:
        return self._k

    def n(self) -> int:
        return self._n

    @property
    def handle(self):
        return self._h

    def matmul_host(self, a, m, out) -> None:
        """int8_matmul_prepacked_dispatch (int8_matmul.rs:2420), host slices."""
        aa = _np(a, np.int8)
        assert out.dtype == np.int32 and out.size == m * self._n and aa.size == m * self._k
        lib().int8_matmul_prepacked_dispatch(_ptr(aa), self._h, _sz(m), _ptr(out))

    def matmul(self, a, a_zp: int = 0, out=None):
        """a: CUDA tensor [m][k] int8 or uint8 -> int32 [m][n] (exact)."""
        import torch

        assert a.is_cuda and a.dim() == 2 and a.shape[1] == self._k and a.dtype in (torch.int8, torch.uint8)
        a = a.contiguous()
        m = a.shape[0]
        if out is None:
            out = torch.empty(m, self._n, device=a.device, dtype=torch.int32)
        lib().int8_matmul(C.c_void_p(a.data_ptr()), int(a.dtype == torch.uint8), int(a_zp), self._h, _sz(m),
                          C.c_void_p(out.data_ptr()), _stream_ptr())
        return out

    def matmul_requant(self, a, a_zp, composite, y_zp, round_mode, clamp_lo, clamp_hi, corr=None, out=None):
        """Fused GEMM + requantize.  composite: float or CUDA f32 tensor [n]; corr: CUDA i32 [n] or None."""
        import torch

        assert a.is_cuda and a.dim() == 2 and a.shape[1] == self._k and a.dtype in (torch.int8, torch.uint8)
        a = a.contiguous()
        m = a.shape[0]
        if out is None:
            out = torch.empty(m, self._n, device=a.device, dtype=torch.int8 if clamp_lo < 0 else torch.uint8)
        comp_v, comp_s = (None, float(composite)) if not hasattr(composite, "data_ptr") else (composite, 0.0)
        lib().int8_matmul_requant(C.c_void_p(a.data_ptr()), int(a.dtype == torch.uint8), int(a_zp), self._h, _sz(m),
                                  C.c_void_p(corr.data_ptr()) if corr is not None else None,
                                  C.c_void_p(comp_v.data_ptr()) if comp_v is not None else None,
                                  C.c_float(comp_s), C.c_float(y_zp), int(round_mode), int(clamp_lo), int(clamp_hi),
                                  C.c_void_p(out.data_ptr()), _stream_ptr())
        return out

    def close(self):
        if self._h:
            lib().i8_weight_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def pack_i8_b_for_matmul(b, k, n) -> PackedI8B:
    """int8_matmul.rs:163."""
    return PackedI8B(b, k, n)


def int8_matmul_prepacked_dispatch(a, b: PackedI8B, m, out) -> None:
    """int8_matmul.rs:2420."""
    b.matmul_host(a, m, out)


def sample_token(logits, top_k, top_p, rng_state):
    """sample_token (crates/yscv-onnx/src/generate.rs:121-208) on a host float32 array, modified in place like the
    Rust `&mut [f32]`.  Returns (token, new_rng_state)."""
    assert isinstance(logits, np.ndarray) and logits.dtype == np.float32 and logits.flags.c_contiguous
    rng = C.c_uint64(rng_state)
    tok = C.c_uint32(0)
    lib().sample_token(_ptr(logits), _sz(logits.size), _sz(top_k), C.c_float(top_p), C.byref(rng), C.byref(tok))
    return tok.value, rng.value
