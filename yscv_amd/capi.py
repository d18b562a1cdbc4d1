"""ctypes binding of include/yscv_hip.h.  Loading fails loudly when the library is missing."""
from __future__ import annotations

import ctypes as C
import os

F32, F16, BF16 = 0, 1, 2
NIBBLE_SIGNED, NIBBLE_UNSIGNED = 0, 1
ROUND_HALF_AWAY, ROUND_TIES_EVEN = 0, 1
EPILOGUE_STORE, EPILOGUE_ADD_F32, EPILOGUE_SWIGLU = 0, 1, 2
STATIC_SCRATCH_BYTES = 32 << 20

_HERE = os.path.dirname(os.path.abspath(__file__))
# YSCV_HIP_LIB points at another build of the same library (e.g. one with stage timestamps compiled in)
_LIB_PATH = os.environ.get("YSCV_HIP_LIB") or os.path.join(_HERE, "lib", "libyscv_hip.so")

STATUS_NAMES = {0: "OK", -1: "INVALID_ARG", -2: "DEVICE", -3: "OOM", -4: "UNSUPPORTED", -5: "NO_DEVICE"}


class DecoderConfig(C.Structure):
    """yscv_hip_decoder_config."""

    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d_model", "n_heads", "n_kv_heads", "head_dim", "d_ff", "vocab",
                                         "group_size", "max_batch", "max_ctx", "max_steps")] + \
               [("rope_theta", C.c_float), ("rms_eps", C.c_float)]


class GenerateConfig(C.Structure):
    """yscv_hip_generate_config (GenerateConfig, crates/yscv-onnx/src/generate.rs:9-35)."""

    _fields_ = [("max_tokens", C.c_size_t), ("temperature", C.c_float), ("top_k", C.c_size_t), ("top_p", C.c_float),
                ("has_eos", C.c_int32), ("eos_token_id", C.c_uint32), ("repetition_penalty", C.c_float)]


class Int4FileHeader(C.Structure):
    """yscv_hip_int4_file_header"""
    _fields_ = [("n", C.c_uint64), ("k", C.c_uint64), ("group_size", C.c_uint64), ("scale_dtype", C.c_int32),
                ("nibble_format", C.c_int32), ("has_zero_points", C.c_int32), ("packed_bytes", C.c_uint64),
                ("scales_bytes", C.c_uint64), ("zero_points_bytes", C.c_uint64), ("checksum", C.c_uint64)]


class QuantStats(C.Structure):
    """yscv_hip_quant_stats."""

    _fields_ = [(n, C.c_uint64) for n in ("qlinear_matmul_fast", "qlinear_matmul_fallback", "matmul_integer_fast",
                                          "matmul_integer_fallback", "int4_fast", "int4_fallback")]


PATH_FAST, PATH_FALLBACK_EXACT, PATH_FALLBACK_F32 = 0, 1, 2


class YscvHipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"yscv_hip status {code} ({STATUS_NAMES.get(code, '?')}): {message}")
        self.code = code
        self.message = message


def library_path() -> str:
    return _LIB_PATH


_sz, _vp, _i32, _f32 = C.c_size_t, C.c_void_p, C.c_int32, C.c_float

# name -> argtypes; every function returns int32 status unless listed in _SPECIAL
_SIGNATURES = {
    "yscv_hip_init": [_i32],
    "yscv_hip_shutdown": [],
    "yscv_hip_device_info": [C.c_char_p, _sz],
    "yscv_hip_measure_peaks": [C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "yscv_hip_measure_fill": [C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "yscv_hip_launch_empty": [_vp],
    "yscv_hip_malloc": [C.POINTER(_vp), _sz],
    "yscv_hip_free": [_vp],
    "yscv_hip_memcpy_h2d": [_vp, _vp, _sz, _vp],
    "yscv_hip_memcpy_d2h": [_vp, _vp, _sz, _vp],
    "yscv_hip_stream_synchronize": [_vp],
    "yscv_hip_int4_weight_create": [_vp, _vp, _i32, _vp, _i32, _sz, _sz, _sz, C.POINTER(_vp)],
    "yscv_hip_int4_weight_destroy": [_vp],
    "yscv_hip_int4_file_write": [C.c_char_p, _vp, _vp, _i32, _vp, _i32, _sz, _sz, _sz],
    "yscv_hip_int4_file_read_header": [C.c_char_p, _vp],
    "yscv_hip_int4_file_read": [C.c_char_p, _vp, _sz, _vp, _sz, _vp, _sz],
    "yscv_hip_int4_weight_load": [C.c_char_p, C.POINTER(_vp)],
    "yscv_hip_int4_weight_dims": [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)],
    "yscv_hip_int4_matmul": [_vp, _vp, _i32, _vp, _i32, _sz, _vp],
    "yscv_hip_int4_gemv": [_vp, _vp, _i32, _vp, _i32, _sz, _vp],
    "yscv_hip_int4_gemm": [_vp, _vp, _i32, _vp, _i32, _sz, _vp],
    "yscv_hip_int4_matmul_fused": [_vp, _vp, _i32, _vp, _i32, _sz, _i32, _vp],
    "yscv_hip_int4_matmul_static": [_vp, _vp, _i32, _vp, _i32, _sz, _vp],
    "yscv_hip_int4_workspace_bytes": [_vp, _sz, _i32, C.POINTER(_sz)],
    "yscv_hip_int4_matmul_ws": [_vp, _vp, _i32, _vp, _i32, _sz, _vp, _sz, _vp],
    "yscv_hip_packed_int4_gemv_dispatch": [_vp, _vp, _vp, _vp, _sz, _sz, _sz],
    "yscv_hip_packed_int4_gemm_dispatch": [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz],
    "yscv_hip_pack_int4_symmetric_per_group": [_vp, _sz, _sz, _sz, _vp, _vp],
    "yscv_hip_dequantize_int4_to_f32": [_vp, _sz, _f32, C.c_int8, _vp],
    "yscv_hip_quantize_f32_to_int4": [_vp, _sz, _f32, C.c_int8, _vp],
    "yscv_hip_quantize_f32_to_int4_dev": [_vp, _sz, _f32, C.c_int8, _vp, _vp],
    "yscv_hip_pack_i8_b_for_matmul": [_vp, _sz, _sz, C.POINTER(_vp)],
    "yscv_hip_i8_weight_destroy": [_vp],
    "yscv_hip_i8_weight_dims": [_vp, C.POINTER(_sz), C.POINTER(_sz)],
    "yscv_hip_int8_matmul": [_vp, _i32, _i32, _vp, _sz, _vp, _vp],
    "yscv_hip_int8_matmul_requant": [_vp, _i32, _i32, _vp, _sz, _vp, _vp, _f32, _f32, _i32, _i32, _i32, _vp, _vp],
    "yscv_hip_int8_matmul_dispatch": [_vp, _vp, _sz, _sz, _sz, _vp],
    "yscv_hip_int8_matmul_prepacked_dispatch": [_vp, _vp, _sz, _vp],
    "yscv_hip_quantize_linear_f32_to_i8": [_vp, _sz, _f32, _f32, _vp, _vp],
    "yscv_hip_requant_i8_per_channel": [_vp, _sz, _vp, _vp, _f32, _vp, _sz, _vp],
    "yscv_hip_requant_i32_row_to_i8": [_vp, _sz, _vp, _f32, _f32, _i32, _vp, _sz, _vp],
    "yscv_hip_dynamic_quantize_linear": [_vp, _sz, _vp, _vp, _vp],
    "yscv_hip_quantize_linear_f32_to_i8_dispatch": [_vp, _sz, _f32, _f32, _vp],
    "yscv_hip_requant_i8_per_channel_dispatch": [_vp, _sz, _vp, _vp, _f32, _vp, _sz],
    "yscv_hip_requant_i32_row_to_i8_dispatch": [_vp, _sz, _vp, _f32, _f32, _i32, _vp, _sz],
    "yscv_hip_dynamic_quantize_linear_host": [_vp, _sz, _vp, C.POINTER(_f32), C.POINTER(_f32)],
    "yscv_hip_quant_runtime_stats": [_vp],
    "yscv_hip_reset_quant_runtime_stats": [],
    "yscv_hip_i8_weight_from_f32": [_vp, _sz, _sz, _vp, C.POINTER(_vp)],
    "yscv_hip_exec_matmul_integer": [_vp, _vp, _vp, _f32, _f32, _sz, _sz, _sz, _vp, C.POINTER(_i32), _vp],
    "yscv_hip_exec_qlinear_matmul": [_vp, _f32, _f32, _vp, _vp, _f32, _f32, _f32, _f32, _sz, _sz, _sz, _vp,
                                     C.POINTER(_i32), _vp],
    "yscv_hip_exec_qdq_matmul": [_vp, _sz, _f32, _vp, _f32, _f32, _f32, _vp, _vp],
    "yscv_hip_exec_dql_matmul_integer": [_vp, _sz, _vp, _vp, _vp, _vp, _vp],
    "yscv_hip_exec_matmul_nbits": [_vp, _i32, _sz, _vp, _vp, C.c_int64, C.c_int64, C.c_int64, C.c_int64, _vp, _i32, _vp],
    "yscv_hip_exec_gemm_int4": [_vp, _sz, _vp, _vp, _sz, _f32, _f32, _vp, _vp],
    "yscv_hip_exec_quantize_linear": [_vp, _sz, _f32, _f32, _vp, _vp],
    "yscv_hip_exec_dequantize_linear": [_vp, _sz, _sz, _sz, _vp, _vp, _sz, _vp, _vp],
    "yscv_hip_exec_dynamic_quantize_linear": [_vp, _sz, _vp, _vp, _vp, _vp],
    "yscv_hip_int4_weight_from_f32": [_vp, _sz, _sz, _i32, _sz, _vp, C.POINTER(_vp)],
    "yscv_hip_kv_i8_quantize_rows": [_vp, _sz, _sz, _vp, _vp, _vp],
    "yscv_hip_kv_i8_dequantize_rows": [_vp, _vp, _sz, _sz, _vp, _vp],
    "yscv_hip_decoder_create": [_vp, C.POINTER(_vp)],
    "yscv_hip_decoder_create_kv": [_vp, _i32, C.POINTER(_vp)],
    "yscv_hip_decoder_destroy": [_vp],
    "yscv_hip_decoder_set_linear": [_vp, _i32, _i32, _vp, _vp, _sz, _sz],
    "yscv_hip_decoder_set_norm": [_vp, _i32, _i32, _vp],
    "yscv_hip_decoder_set_embedding": [_vp, _vp],
    "yscv_hip_decoder_finalize": [_vp],
    "yscv_hip_decoder_init_random": [_vp, C.c_uint64],
    "yscv_hip_decoder_init_random_range": [_vp, C.c_uint64, _i32, _i32],
    "yscv_hip_decoder_fill_kv_random": [_vp, C.c_uint64],
    "yscv_hip_decoder_set_kv": [_vp, _i32, _vp, _vp, _i32, _i32],
    "yscv_hip_decoder_get_kv": [_vp, _i32, _vp, _vp, _i32, _i32, _i32],
    "yscv_hip_decoder_reset": [_vp, _i32, _i32, _vp],
    "yscv_hip_decoder_run": [_vp, _i32, _i32, _vp],
    "yscv_hip_decoder_last_path": [_vp, _vp],
    "yscv_hip_decoder_set_prefill_rows": [_vp, _i32],
    "yscv_hip_decoder_prefill": [_vp, _vp, _i32, _i32, _vp],
    "yscv_hip_decoder_set_qkv_bias": [_vp, _i32, _vp],
    "yscv_hip_rms_norm_dev": [_vp, _vp, _sz, _sz, C.c_float, _vp, _vp],
    "yscv_hip_rope_dev": [_vp, _vp, _sz, _sz, _sz, _sz, _sz, C.c_float, _vp],
    "yscv_hip_gqa_attention_dev": [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _vp, _vp],
    "yscv_hip_decoder_run_projections": [_vp, _i32, _vp],
    "yscv_hip_decoder_read_tokens": [_vp, _i32, _i32, _vp],
    "yscv_hip_decoder_read_logits": [_vp, _vp],
    "yscv_hip_decoder_read_activation": [_vp, _i32, _vp, _sz],
    "yscv_hip_decoder_debug_set_tag_epoch": [_vp, C.c_uint32],
    "yscv_hip_decoder_debug_set_fused_attention": [_vp, C.c_int32],
    "yscv_hip_decoder_debug_set_folded_norm": [_vp, C.c_int32],
    "yscv_hip_decoder_weight_bytes": [_vp, C.POINTER(_sz)],
    "yscv_hip_decoder_vocab": [_vp, C.POINTER(_sz)],
    "yscv_hip_sample_token": [_vp, _sz, _sz, _f32, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)],
    "yscv_hip_decoder_generate": [_vp, _vp, _sz, _vp, _vp, C.POINTER(_sz)],
}
_SPECIAL = {
    "yscv_hip_abi_version": ([], C.c_uint32),
    "yscv_hip_last_error": ([], C.c_char_p),
    # predicates: the return value is the answer, not a status
    "yscv_hip_quant_int8_fast_enabled": ([], _i32),
    "yscv_hip_should_use_prepacked_i8_b": ([_sz, _sz, _sz], _i32),
    "yscv_hip_should_prepack_i8_b": ([_sz, _sz], _i32),
}

EXPORTED_SYMBOLS = sorted(list(_SIGNATURES) + list(_SPECIAL))

_lib = None


class _Checked:
    """Wraps the CDLL so that every status-returning call raises YscvHipError on failure."""

    def __init__(self, cdll: C.CDLL):
        self._cdll = cdll
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(cdll, name)
            fn.argtypes = argtypes
            fn.restype = _i32
            setattr(self, name[len("yscv_hip_"):], self._wrap(fn))
        for name, (argtypes, restype) in _SPECIAL.items():
            fn = getattr(cdll, name)
            fn.argtypes = argtypes
            fn.restype = restype
            setattr(self, name[len("yscv_hip_"):], fn)

    def _wrap(self, fn):
        def call(*args):
            st = fn(*args)
            if st != 0:
                msg = self._cdll.yscv_hip_last_error()
                raise YscvHipError(st, msg.decode() if msg else "")
            return st

        call.raw = fn
        return call


def lib() -> _Checked:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `make -C yscv_amd/csrc -j8` "
                "(or __graft_entry__.build()); there is no fallback path"
            )
        # torch ships its own HIP runtime under the same soname as /opt/rocm's; a process can hold
        # only one, and torch's must be the one that is loaded first or torch loses the GPU.
        import torch  # noqa: F401

        _lib = _Checked(C.CDLL(_LIB_PATH))
    return _lib
