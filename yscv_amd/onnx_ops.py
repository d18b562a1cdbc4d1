"""Host-side mirror of the reference runner's quantised operators over the C ABI.

Function names and argument meaning follow crates/yscv-onnx/src/runner/linear.rs (exec_matmul_integer :648,
exec_qlinear_matmul :438), crates/yscv-onnx/src/runner/misc.rs (exec_quantize_linear :42, exec_dequantize_linear
:110, exec_dynamic_quantize_linear :241) and crates/yscv-onnx/src/runner/quant_stats.rs.  Tensors are torch CUDA
f32 tensors used as device buffers (the reference keeps every quantised value in an f32 tensor as well); all
arithmetic happens inside libyscv_hip.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from .capi import PATH_FALLBACK_EXACT, PATH_FALLBACK_F32, PATH_FAST, QuantStats, lib  # noqa: F401

_sz = C.c_size_t


def _stream_ptr():
    import torch

    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev_f32(t, name):
    import torch

    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32):
        raise TypeError(f"{name}: expected a CUDA float32 tensor")
    return t.contiguous()


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


@dataclass(frozen=True)
class QuantRuntimeStats:
    """quant_stats.rs:6-22, restricted to the matmul path, plus the int4 and MatMulInteger splits."""

    qlinear_matmul_fast: int = 0
    qlinear_matmul_fallback: int = 0
    matmul_integer_fast: int = 0
    matmul_integer_fallback: int = 0
    int4_fast: int = 0
    int4_fallback: int = 0


def quant_runtime_stats() -> QuantRuntimeStats:
    s = QuantStats()
    lib().quant_runtime_stats(C.byref(s))
    return QuantRuntimeStats(**{n: int(getattr(s, n)) for n, _ in QuantStats._fields_})


def reset_quant_runtime_stats() -> None:
    lib().reset_quant_runtime_stats()


def quant_int8_fast_enabled() -> bool:
    return bool(lib().quant_int8_fast_enabled())


def should_use_prepacked_i8_b(m: int, k: int, n: int) -> bool:
    return bool(lib().should_use_prepacked_i8_b(m, k, n))


def should_prepack_i8_b(k: int, n: int) -> bool:
    return bool(lib().should_prepack_i8_b(k, n))


class PrepackedI8B:
    """Load-time prepack of a weight initialiser given as an f32 carrier [k][n] (plan/build.rs:1367-1454)."""

    def __init__(self, b):
        b = _dev_f32(b, "b")
        if b.dim() != 2:
            raise ValueError("prepack takes a rank-2 weight")
        self.k, self.n = int(b.shape[0]), int(b.shape[1])
        h = C.c_void_p()
        lib().i8_weight_from_f32(_p(b), _sz(self.k), _sz(self.n), _stream_ptr(), C.byref(h))
        self._h = h

    @property
    def handle(self):
        return self._h

    def close(self):
        if self._h:
            lib().i8_weight_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _matmul_operands(a, b, prepacked):
    import torch

    a = _dev_f32(a, "a")
    if a.dim() != 2:
        raise ValueError("a must be rank 2 (flatten leading dimensions into m)")
    m, k = int(a.shape[0]), int(a.shape[1])
    if b is not None:
        b = _dev_f32(b, "b")
        if b.dim() != 2 or int(b.shape[0]) != k:
            raise ValueError("b must be [k][n] with k = a.shape[1]")
        n = int(b.shape[1])
    elif prepacked is not None:
        n = prepacked.n
    else:
        raise ValueError("neither b nor a prepacked weight given")
    out = torch.empty(m, n, device=a.device, dtype=torch.float32)
    return a, b, m, k, n, out


def exec_matmul_integer(a, b=None, a_zp: float = 0.0, b_zp: float = 0.0, prepacked: PrepackedI8B | None = None):
    """linear.rs:648-737.  Returns (out [m][n] f32, path)."""
    a, b, m, k, n, out = _matmul_operands(a, b, prepacked)
    path = C.c_int32(-1)
    lib().exec_matmul_integer(_p(a), _p(b), prepacked.handle if prepacked is not None else None, C.c_float(a_zp),
                              C.c_float(b_zp), _sz(m), _sz(k), _sz(n), _p(out), C.byref(path), _stream_ptr())
    return out, path.value


def exec_qlinear_matmul(a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp, prepacked: PrepackedI8B | None = None):
    """linear.rs:438-538.  Returns (out [m][n] f32 holding values in [-128, 127], path)."""
    a, b, m, k, n, out = _matmul_operands(a, b, prepacked)
    path = C.c_int32(-1)
    lib().exec_qlinear_matmul(_p(a), C.c_float(a_scale), C.c_float(a_zp), _p(b),
                              prepacked.handle if prepacked is not None else None, C.c_float(b_scale),
                              C.c_float(b_zp), C.c_float(y_scale), C.c_float(y_zp), _sz(m), _sz(k), _sz(n), _p(out),
                              C.byref(path), _stream_ptr())
    return out, path.value


def exec_qdq_matmul(x, a_scale, prepacked: PrepackedI8B, b_scale, y_scale, y_zp: float = 0.0):
    """QuantizeLinear -> QLinearMatMul -> DequantizeLinear (quantize/rewriter.rs:586-673) in one call, f32 in / out."""
    import torch

    x = _dev_f32(x, "x")
    if x.dim() != 2 or int(x.shape[1]) != prepacked.k:
        raise ValueError("x must be [m][k] with k matching the prepacked weight")
    out = torch.empty(int(x.shape[0]), prepacked.n, device=x.device, dtype=torch.float32)
    lib().exec_qdq_matmul(_p(x), _sz(int(x.shape[0])), C.c_float(a_scale), prepacked.handle, C.c_float(b_scale),
                          C.c_float(y_scale), C.c_float(y_zp), _p(out), _stream_ptr())
    return out


def exec_dql_matmul_integer(x, prepacked: PrepackedI8B):
    """DynamicQuantizeLinear -> MatMulInteger (b_zero_point 0) in one call.  Returns (out [m][n] f32, y_scale [1], y_zp [1])."""
    import torch

    x = _dev_f32(x, "x")
    if x.dim() != 2 or int(x.shape[1]) != prepacked.k:
        raise ValueError("x must be [m][k] with k matching the prepacked weight")
    out = torch.empty(int(x.shape[0]), prepacked.n, device=x.device, dtype=torch.float32)
    sz = torch.empty(2, device=x.device, dtype=torch.float32)
    lib().exec_dql_matmul_integer(_p(x), _sz(int(x.shape[0])), prepacked.handle, _p(out), _p(sz[0:1]), _p(sz[1:2]), _stream_ptr())
    return out, sz[0:1], sz[1:2]


class MatMulNBitsWeight:
    """The initialisers of one MatMulNBits node (com.microsoft) uploaded once: B [N][K/block][block/2] uint8 (element 2i
    in the low nibble), scales [N * K/block] float32 or float16, optional packed uint4 zero_points [N][ceil(K/block/2)]
    (default 8).  Same byte order as the reference's PackedInt4Weight (int4_matmul.rs:12-14) with unsigned nibbles."""

    def __init__(self, b, scales, zero_points, K: int, N: int, bits: int = 4, block_size: int = 32):
        from .kernels import NIBBLE_UNSIGNED, PackedInt4Weight

        if bits != 4:
            raise ValueError("MatMulNBits: only bits = 4 is supported")
        self.K, self.N, self.bits, self.block_size = int(K), int(N), int(bits), int(block_size)
        self.weight = PackedInt4Weight(b, scales, block_size, N, K, zero_points=zero_points, nibble_format=NIBBLE_UNSIGNED)

    def close(self):
        self.weight.close()


def exec_matmul_nbits(a, w: MatMulNBitsWeight, bias=None, out_dtype=None, *, K=None, N=None, bits=None, block_size=None):
    """MatMulNBits executor: Y = A x dequant(B)^T (+ bias).  a: CUDA tensor [..., K] f32 / f16 / bf16; the attributes
    default to the ones the weight was built with (a graph executor passes the node's own).  Output [..., N]."""
    import torch

    from .kernels import _torch_dtype_code

    if not a.is_cuda or a.shape[-1] != w.K:
        raise ValueError("a must be a CUDA tensor whose last dimension is K")
    a = a.contiguous()
    m = a.numel() // w.K
    out = torch.empty(*a.shape[:-1], w.N, device=a.device, dtype=out_dtype or a.dtype)
    if bias is not None:
        bias = _dev_f32(bias, "bias")
        if bias.numel() != w.N:
            raise ValueError("bias must hold N values")
    lib().exec_matmul_nbits(_p(a), _torch_dtype_code(a), _sz(m), w.weight.handle, _p(bias),
                            C.c_int64(w.K if K is None else K), C.c_int64(w.N if N is None else N),
                            C.c_int64(w.bits if bits is None else bits),
                            C.c_int64(w.block_size if block_size is None else block_size), _p(out), _torch_dtype_code(out),
                            _stream_ptr())
    return out


def exec_gemm_int4(a, w, c=None, alpha: float = 1.0, beta: float = 1.0):
    """Gemm (transA = 0) whose weight the int4 packing pass quantised: alpha * (a x W^T) + beta * c on f32 carriers.
    w: kernels.PackedInt4Weight (from_f32 of the Gemm's B in either layout); c: None, [N], [1][N] or [M][N]."""
    import torch

    a = _dev_f32(a, "a")
    if a.dim() != 2 or int(a.shape[1]) != w.k:
        raise ValueError("a must be [m][K]")
    m = int(a.shape[0])
    c_rows = 0
    if c is not None:
        c = _dev_f32(c, "c")
        if c.numel() == w.m_w:
            c_rows = 1
        elif c.numel() == m * w.m_w:
            c_rows = m
        else:
            raise ValueError("c must hold N or M * N values")
    out = torch.empty(m, w.m_w, device=a.device, dtype=torch.float32)
    lib().exec_gemm_int4(_p(a), _sz(m), w.handle, _p(c), _sz(c_rows), C.c_float(alpha), C.c_float(beta), _p(out), _stream_ptr())
    return out


def exec_quantize_linear(x, scale: float, zero_point: float = 0.0):
    """misc.rs:42-80 (f32-carrier arm): clamp(round_ties_even(x / scale + zp), -128, 127) as f32."""
    import torch

    x = _dev_f32(x, "x")
    out = torch.empty_like(x)
    lib().exec_quantize_linear(_p(x), _sz(x.numel()), C.c_float(scale), C.c_float(zero_point), _p(out), _stream_ptr())
    return out


def exec_dequantize_linear(q, scale, zero_point=None, axis: int = 1):
    """misc.rs:110-239: (q - zp) * scale, per tensor (one scale) or per channel along `axis`."""
    import torch

    q = _dev_f32(q, "q")
    scale = _dev_f32(scale.reshape(-1) if hasattr(scale, "reshape") else torch.tensor([scale], device=q.device), "scale")
    if zero_point is not None:
        zero_point = _dev_f32(zero_point.reshape(-1) if hasattr(zero_point, "reshape")
                              else torch.tensor([zero_point], device=q.device, dtype=torch.float32), "zero_point")
    if scale.numel() == 1:
        outer, chan, inner = 1, 1, q.numel()
    else:
        ax = axis + q.dim() if axis < 0 else axis
        shape = list(q.shape)
        outer = 1
        for d in shape[:ax]:
            outer *= d
        chan = shape[ax]
        inner = 1
        for d in shape[ax + 1:]:
            inner *= d
    out = torch.empty_like(q)
    lib().exec_dequantize_linear(_p(q), _sz(outer), _sz(chan), _sz(inner), _p(scale), _p(zero_point),
                                 _sz(scale.numel()), _p(out), _stream_ptr())
    return out


def exec_dynamic_quantize_linear(x):
    """misc.rs:241-289.  Returns (y f32 in [0, 255], y_scale [1], y_zp [1]) as device tensors."""
    import torch

    x = _dev_f32(x, "x")
    y = torch.empty_like(x)
    sz = torch.empty(2, device=x.device, dtype=torch.float32)
    lib().exec_dynamic_quantize_linear(_p(x), _sz(x.numel()), _p(y), _p(sz[0:1]), _p(sz[1:2]), _stream_ptr())
    return y, sz[0:1], sz[1:2]


# ---- the operators between the MatMuls of an LLM graph (device tensors in, device tensors out) ----------------------
def rms_norm(x, gamma, eps: float):
    """rms_norm_last_dim (crates/yscv-kernels/src/ops/norm.rs:1431-1518) over the last axis of a CUDA f32 tensor."""
    import torch

    x = _dev_f32(x, "x")
    gamma = _dev_f32(gamma, "gamma")
    d = x.shape[-1]
    if gamma.ndim != 1 or gamma.shape[0] != d:
        raise ValueError(f"gamma must be [{d}], got {tuple(gamma.shape)}")
    y = torch.empty_like(x)
    lib().rms_norm_dev(_p(x), _p(gamma), _sz(x.numel() // d if d else 0), _sz(d), C.c_float(eps), _p(y), _stream_ptr())
    return y


def apply_rotary_embedding(q, k, num_q_heads: int, num_kv_heads: int, d_head: int, seq_len: int, seq_offset: int, theta: float):
    """apply_rotary_embedding (crates/yscv-kernels/src/ops/rope.rs:24-117), in place on CUDA f32 tensors
    q [seq_len][num_q_heads][d_head] and k [seq_len][num_kv_heads][d_head]."""
    for t, heads, name in ((q, num_q_heads, "q"), (k, num_kv_heads, "k")):
        if not (t.is_cuda and t.is_contiguous() and t.numel() == seq_len * heads * d_head):
            raise ValueError(f"{name}: expected a contiguous CUDA tensor of {seq_len} x {heads} x {d_head} values")
        _dev_f32(t, name)
    lib().rope_dev(_p(q), _p(k), _sz(num_q_heads), _sz(num_kv_heads), _sz(d_head), _sz(seq_len), _sz(seq_offset), C.c_float(theta),
                   _stream_ptr())


def exec_grouped_query_attention(q, k, v, num_heads: int, kv_num_heads: int | None = None):
    """exec_grouped_query_attention (crates/yscv-onnx/src/runner/linear.rs:552-646): q [B][Sq][Hq d], k / v [B][Sk][Hkv d]
    CUDA f32 tensors -> [B][Sq][Hq d]."""
    import torch

    q, k, v = _dev_f32(q, "q"), _dev_f32(k, "k"), _dev_f32(v, "v")
    kv_num_heads = num_heads if kv_num_heads is None else kv_num_heads
    B, Sq, Sk = q.shape[0], q.shape[1], k.shape[1]
    d_head = q.shape[2] // num_heads
    if k.shape != (B, Sk, kv_num_heads * d_head) or v.shape != k.shape or q.shape[2] != num_heads * d_head:
        raise ValueError("GroupQueryAttention: inconsistent shapes")
    out = torch.empty_like(q)
    lib().gqa_attention_dev(_p(q), _p(k), _p(v), _sz(B), _sz(Sq), _sz(Sk), _sz(num_heads), _sz(kv_num_heads), _sz(d_head), _p(out),
                            _stream_ptr())
    return out
