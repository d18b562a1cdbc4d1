/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the YSCV quantized-matmul path.
 *
 * This file is the parity checker for the HIP backend.  It is never linked into,
 * loaded by, or called from the shipped library; only the test-suite, the smoke
 * check and the benchmark's CPU-baseline leg may use it.
 *
 * Every function restates, in plain C, the *scalar* function of the Rust
 * reference that it cites (paths relative to the reference checkout).  The Rust
 * guarantees the restatement relies on:
 *   - f32 `+ - * /` are IEEE-754 single operations, never contracted into FMA
 *     (build this file with -ffp-contract=off -fno-fast-math, no -march flags);
 *   - `x as i8` / `x as i32` on a float saturates and maps NaN to 0;
 *   - `f32::round` rounds half away from zero (C roundf);
 *   - `f32::round_ties_even` rounds half to even (C rintf in the default mode);
 *   - `f32::clamp` propagates NaN;
 *   - `f32::max/min` return the non-NaN operand;
 *   - `i32::wrapping_add` is two's-complement addition.
 *
 * Parity status: every function below is pinned by a golden vector or
 * known-answer test taken from the reference's own unit tests, or by a closed
 * form / brute-force check (see tests/test_oracle_*.py).  The f32 kernels are
 * sequential recurrences without transcendental functions, so their results are
 * fixed by the source text; what no test in this repository can show is
 * last-ulp identity with rustc's code generation, because no Rust toolchain is
 * available to run the reference.  The decoder glue (RMSNorm, RoPE, softmax)
 * depends on libm and is tolerance-checked only.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))
#define F32_EPSILON 1.1920929e-7f

/* ---- Rust cast / rounding semantics ------------------------------------ */

/* `v as i8` for f32: saturating, NaN -> 0. */
static inline int8_t rust_f32_as_i8(float v) {
  if (v != v) return 0;
  if (v <= -128.0f) return -128;
  if (v >= 127.0f) return 127;
  return (int8_t)v; /* truncation toward zero, in range */
}

/* `v as i32` for f32: saturating, NaN -> 0. */
static inline int32_t rust_f32_as_i32(float v) {
  if (v != v) return 0;
  if (v <= -2147483648.0f) return INT32_MIN;
  if (v >= 2147483648.0f) return INT32_MAX;
  return (int32_t)v;
}

/* `f32::clamp(lo, hi)`: NaN stays NaN. */
static inline float rust_clampf(float v, float lo, float hi) {
  if (v < lo) return lo;
  if (v > hi) return hi;
  return v;
}

/* `f32::max`: if one operand is NaN, the other is returned. */
static inline float rust_maxf(float a, float b) {
  if (a != a) return b;
  if (b != b) return a;
  return a > b ? a : b;
}
static inline float rust_minf(float a, float b) {
  if (a != a) return b;
  if (b != b) return a;
  return a < b ? a : b;
}

static inline int32_t wrapping_add_i32(int32_t a, int32_t b) {
  return (int32_t)((uint32_t)a + (uint32_t)b);
}

/* ---- fp16 / bf16 bit conversions ---------------------------------------- */
/* crates/yscv-tensor/src/tensor.rs:711-735 -- f32 -> fp16 TRUNCATES the mantissa. */
ORC_API uint16_t orc_f32_to_fp16_bits(float val) {
  uint32_t bits;
  memcpy(&bits, &val, 4);
  uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
  int32_t exponent = (int32_t)((bits >> 23) & 0xFFu);
  uint32_t mantissa = bits & 0x007FFFFFu;
  if (exponent == 0xFF) return (uint16_t)(sign | 0x7C00u | (mantissa != 0 ? 0x0200u : 0u));
  int32_t unbiased = exponent - 127;
  if (unbiased < -24) return sign;
  if (unbiased < -14) {
    int32_t shift = -1 - unbiased;
    uint16_t sub = (uint16_t)((mantissa | 0x00800000u) >> (shift + 13));
    return (uint16_t)(sign | sub);
  }
  if (unbiased > 15) return (uint16_t)(sign | 0x7C00u);
  uint16_t e = (uint16_t)((uint16_t)(unbiased + 15) << 10);
  uint16_t m = (uint16_t)(mantissa >> 13);
  return (uint16_t)(sign | e | m);
}

/* crates/yscv-tensor/src/tensor.rs:737-762 -- exact widening. */
ORC_API float orc_fp16_bits_to_f32(uint16_t half) {
  uint32_t sign = ((uint32_t)(half & 0x8000u)) << 16;
  uint32_t exponent = (half >> 10) & 0x1Fu;
  uint32_t mantissa = half & 0x03FFu;
  uint32_t out;
  if (exponent == 0) {
    if (mantissa == 0) {
      out = sign;
    } else {
      int32_t e = 0;
      uint32_t m = mantissa;
      while ((m & 0x0400u) == 0) {
        m <<= 1;
        e += 1;
      }
      out = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x03FFu) << 13);
    }
  } else if (exponent == 31) {
    out = sign | 0x7F800000u | (mantissa != 0 ? 0x00400000u : 0u);
  } else {
    out = sign | ((exponent + 112u) << 23) | (mantissa << 13);
  }
  float f;
  memcpy(&f, &out, 4);
  return f;
}

/* crates/yscv-tensor/src/tensor.rs:764-769 -- round to nearest even, no NaN case. */
ORC_API uint16_t orc_f32_to_bf16_bits(float val) {
  uint32_t bits;
  memcpy(&bits, &val, 4);
  uint32_t bias = 0x7FFFu + ((bits >> 16) & 1u);
  return (uint16_t)((bits + bias) >> 16);
}

/* crates/yscv-tensor/src/tensor.rs:771-773 */
ORC_API float orc_bf16_bits_to_f32(uint16_t b) {
  uint32_t bits = ((uint32_t)b) << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

ORC_API void orc_fp16_to_f32_array(const uint16_t *src, float *dst, size_t n) {
  for (size_t i = 0; i < n; i++) dst[i] = orc_fp16_bits_to_f32(src[i]);
}
ORC_API void orc_bf16_to_f32_array(const uint16_t *src, float *dst, size_t n) {
  for (size_t i = 0; i < n; i++) dst[i] = orc_bf16_bits_to_f32(src[i]);
}
ORC_API void orc_f32_to_bf16_array(const float *src, uint16_t *dst, size_t n) {
  for (size_t i = 0; i < n; i++) dst[i] = orc_f32_to_bf16_bits(src[i]);
}
ORC_API void orc_f32_to_fp16_array(const float *src, uint16_t *dst, size_t n) {
  for (size_t i = 0; i < n; i++) dst[i] = orc_f32_to_fp16_bits(src[i]);
}

/* ---- int4 nibble decode -------------------------------------------------- */
/* crates/yscv-kernels/src/ops/int4_matmul.rs:29-40 */
ORC_API int8_t orc_unpack_low(uint8_t byte) {
  int8_t v = (int8_t)(uint8_t)(byte << 4);
  return (int8_t)(v >> 4);
}
ORC_API int8_t orc_unpack_high(uint8_t byte) { return (int8_t)(((int8_t)byte) >> 4); }

/* crates/yscv-kernels/src/ops/quantize.rs:201-213 -- the other spelling of the same decode. */
ORC_API int8_t orc_nibble_lo(uint8_t byte) {
  int8_t v = (int8_t)(byte & 0x0F);
  return v >= 8 ? (int8_t)(v - 16) : v;
}
ORC_API int8_t orc_nibble_hi(uint8_t byte) {
  int8_t v = (int8_t)((byte >> 4) & 0x0F);
  return v >= 8 ? (int8_t)(v - 16) : v;
}

/* ---- packed int4 GEMV / GEMM --------------------------------------------- */
/* crates/yscv-kernels/src/ops/int4_matmul.rs:44-81 (packed_int4_gemv_scalar) */
ORC_API void orc_packed_int4_gemv_scalar(const uint8_t *weight_packed, const float *scales,
                                         const float *activation, float *output, size_t m_w,
                                         size_t k, size_t group_size) {
  size_t groups = k / group_size;
  for (size_t row = 0; row < m_w; row++) {
    const uint8_t *row_bytes = weight_packed + row * k / 2;
    const float *row_scales = scales + row * groups;
    float acc = 0.0f;
    for (size_t g = 0; g < groups; g++) {
      float scale = row_scales[g];
      float group_acc = 0.0f;
      size_t byte_base = g * group_size / 2;
      size_t act_base = g * group_size;
      for (size_t i = 0; i < group_size / 2; i++) {
        uint8_t byte = row_bytes[byte_base + i];
        float q_lo = (float)orc_unpack_low(byte);
        float q_hi = (float)orc_unpack_high(byte);
        group_acc += q_lo * activation[act_base + 2 * i];
        group_acc += q_hi * activation[act_base + 2 * i + 1];
      }
      acc += scale * group_acc;
    }
    output[row] = acc;
  }
}

/* crates/yscv-kernels/src/ops/int4_matmul.rs:387-435 (packed_int4_gemm_scalar) */
ORC_API void orc_packed_int4_gemm_scalar(const uint8_t *weight_packed, const float *scales,
                                         const float *activation, float *output, size_t m,
                                         size_t n, size_t k, size_t group_size) {
  size_t groups = k / group_size;
  for (size_t i = 0; i < m * n; i++) output[i] = 0.0f;
  int8_t *unpacked = (int8_t *)malloc(group_size > 256 ? group_size : 256);
  for (size_t nn = 0; nn < n; nn++) {
    const uint8_t *row_bytes = weight_packed + nn * k / 2;
    const float *row_scales = scales + nn * groups;
    for (size_t g = 0; g < groups; g++) {
      float scale = row_scales[g];
      size_t byte_base = g * group_size / 2;
      size_t act_base = g * group_size;
      for (size_t i = 0; i < group_size / 2; i++) {
        uint8_t byte = row_bytes[byte_base + i];
        unpacked[2 * i] = orc_unpack_low(byte);
        unpacked[2 * i + 1] = orc_unpack_high(byte);
      }
      for (size_t mi = 0; mi < m; mi++) {
        float sum = 0.0f;
        const float *row_act = activation + mi * k + act_base;
        for (size_t j = 0; j < group_size; j++) sum += ((float)unpacked[j]) * row_act[j];
        output[mi * n + nn] += scale * sum;
      }
    }
  }
  free(unpacked);
}

/* crates/yscv-kernels/src/ops/int4_matmul.rs:611-646 (pack_int4_symmetric_per_group) */
ORC_API void orc_pack_int4_symmetric_per_group(const float *weights, size_t m_w, size_t k,
                                               size_t group_size, uint8_t *packed,
                                               float *scales) {
  size_t groups = k / group_size;
  for (size_t row = 0; row < m_w; row++) {
    for (size_t g = 0; g < groups; g++) {
      const float *slice = weights + row * k + g * group_size;
      float abs_max = 0.0f;
      for (size_t i = 0; i < group_size; i++) abs_max = rust_maxf(abs_max, fabsf(slice[i]));
      float scale = (abs_max <= F32_EPSILON) ? 1.0f : abs_max / 7.0f;
      scales[row * groups + g] = scale;
      float inv = 1.0f / scale;
      for (size_t i = 0; i < group_size / 2; i++) {
        int8_t v0 = rust_f32_as_i8(rust_clampf(rintf(slice[2 * i] * inv), -8.0f, 7.0f));
        int8_t v1 = rust_f32_as_i8(rust_clampf(rintf(slice[2 * i + 1] * inv), -8.0f, 7.0f));
        uint8_t byte = (uint8_t)(((uint8_t)v0 & 0x0F) | (((uint8_t)v1 & 0x0F) << 4));
        packed[row * k / 2 + g * group_size / 2 + i] = byte;
      }
    }
  }
}

/* ---- int4 quantize / dequantize with zero point -------------------------- */
/* crates/yscv-kernels/src/ops/quantize.rs:215-222 (dequantize_int4_to_f32_scalar) */
ORC_API void orc_dequantize_int4_to_f32(const uint8_t *packed, size_t n_bytes, float scale,
                                        int8_t zero_point, float *output) {
  float zp = (float)zero_point;
  for (size_t i = 0; i < n_bytes; i++) {
    uint8_t byte = packed[i];
    output[i * 2] = ((float)orc_nibble_lo(byte) - zp) * scale;
    output[i * 2 + 1] = ((float)orc_nibble_hi(byte) - zp) * scale;
  }
}

/* crates/yscv-kernels/src/ops/quantize.rs:69-95 (quantize_f32_to_int4) */
ORC_API void orc_quantize_f32_to_int4(const float *data, size_t n, float scale,
                                      int8_t zero_point, uint8_t *output) {
  float inv_scale = (fabsf(scale) > F32_EPSILON) ? 1.0f / scale : 0.0f;
  int32_t zp = (int32_t)zero_point;
  size_t out_n = (n + 1) / 2;
  for (size_t o = 0; o < out_n; o++) {
    /* `as i32` saturates; the sum with zp cannot overflow after saturation in
       practice, Rust would wrap in release -- keep plain wrapping add. */
    int32_t q0 = wrapping_add_i32(rust_f32_as_i32(rintf(data[2 * o] * inv_scale)), zp);
    q0 = q0 < -8 ? -8 : (q0 > 7 ? 7 : q0);
    int32_t q1 = 0;
    if (2 * o + 1 < n) {
      q1 = wrapping_add_i32(rust_f32_as_i32(rintf(data[2 * o + 1] * inv_scale)), zp);
      q1 = q1 < -8 ? -8 : (q1 > 7 ? 7 : q1);
    }
    output[o] = (uint8_t)(((uint8_t)q0 & 0x0F) | (((uint8_t)q1 & 0x0F) << 4));
  }
}

/*
 * MatMulNBits bridge (the reference has no MatMulNBits executor; this composes
 * two reference functions).  ONNX stores unsigned nibbles q in [0,15] with a
 * per-group unsigned zero point zp (default 8) and value (q - zp) * scale.  The
 * reference nibble is the signed two's-complement s = q - 8, i.e. byte ^ 0x88,
 * and (q - zp) = (s - (zp - 8)).  Per group the weights are dequantised with
 * dequantize_int4_to_f32 (quantize.rs:215-222) using zero_point = zp - 8, then
 * dotted with the activation row in the element order of
 * packed_int4_gemm_scalar (int4_matmul.rs:425-431), accumulating
 * `out += sum` from 0.0 over groups.  With zp == 8 and scale applied after the
 * dot this is NOT bit-identical to packed_int4_gemv_scalar (scale is applied
 * per element here); it is the definition used for asymmetric weights only.
 *   b:      [n][k/2] bytes, element 2i in the low nibble
 *   scales: [n][k/group] f32
 *   zps:    [n][ceil((k/group)/2)] bytes, group 2j in the low nibble; NULL => 8
 */
ORC_API void orc_matmul_nbits_dequant_dot(const uint8_t *b, const float *scales,
                                          const uint8_t *zps, const float *activation,
                                          float *output, size_t m, size_t n, size_t k,
                                          size_t group_size) {
  size_t groups = k / group_size;
  size_t zp_row_bytes = (groups + 1) / 2;
  float *deq = (float *)malloc(sizeof(float) * group_size);
  uint8_t *tmp = (uint8_t *)malloc(group_size / 2);
  for (size_t i = 0; i < m * n; i++) output[i] = 0.0f;
  for (size_t nn = 0; nn < n; nn++) {
    for (size_t g = 0; g < groups; g++) {
      int32_t zp = 8;
      if (zps) {
        uint8_t zb = zps[nn * zp_row_bytes + g / 2];
        zp = (g & 1) ? (zb >> 4) : (zb & 0x0F);
      }
      const uint8_t *src = b + nn * k / 2 + g * group_size / 2;
      for (size_t i = 0; i < group_size / 2; i++) tmp[i] = src[i] ^ 0x88;
      orc_dequantize_int4_to_f32(tmp, group_size / 2, scales[nn * groups + g],
                                 (int8_t)(zp - 8), deq);
      for (size_t mi = 0; mi < m; mi++) {
        const float *row_act = activation + mi * k + g * group_size;
        float sum = 0.0f;
        for (size_t j = 0; j < group_size; j++) sum += deq[j] * row_act[j];
        output[mi * n + nn] += sum;
      }
    }
  }
  free(deq);
  free(tmp);
}

/* ---- int8 GEMM ------------------------------------------------------------ */
/* crates/yscv-kernels/src/ops/int8_matmul.rs:195-208 (int8_matmul_scalar); b is [k][n]. */
ORC_API void orc_int8_matmul_scalar(const int8_t *a, const int8_t *b, size_t m, size_t k,
                                    size_t n, int32_t *out) {
  for (size_t i = 0; i < m; i++) {
    for (size_t j = 0; j < n; j++) {
      int32_t acc = 0;
      for (size_t kk = 0; kk < k; kk++)
        acc = wrapping_add_i32(acc, (int32_t)a[i * k + kk] * (int32_t)b[kk * n + j]);
      out[i * n + j] = acc;
    }
  }
}

/* crates/yscv-kernels/src/ops/int8_matmul.rs:90-117 (transpose_b): [k][n] -> [n][k]. */
ORC_API void orc_transpose_b(const int8_t *b, size_t k, size_t n, int8_t *bt) {
  for (size_t kk = 0; kk < k; kk++)
    for (size_t j = 0; j < n; j++) bt[j * k + kk] = b[kk * n + j];
}

/* crates/yscv-kernels/src/ops/int8_matmul.rs:212-227 (int8_matmul_prepacked_scalar); bt is [n][k]. */
ORC_API void orc_int8_matmul_prepacked_scalar(const int8_t *a, const int8_t *bt, size_t m,
                                              size_t k, size_t n, int32_t *out) {
  for (size_t i = 0; i < m; i++) {
    for (size_t j = 0; j < n; j++) {
      int32_t acc = 0;
      for (size_t kk = 0; kk < k; kk++)
        acc = wrapping_add_i32(acc, (int32_t)a[i * k + kk] * (int32_t)bt[j * k + kk]);
      out[i * n + j] = acc;
    }
  }
}

/* crates/yscv-kernels/src/ops/int8_matmul.rs:168-175 (column sums kept beside the packed B). */
ORC_API void orc_i8_col_sums(const int8_t *b, size_t k, size_t n, int32_t *col_sum) {
  for (size_t j = 0; j < n; j++) {
    int32_t s = 0;
    for (size_t kk = 0; kk < k; kk++) s = wrapping_add_i32(s, (int32_t)b[kk * n + j]);
    col_sum[j] = s;
  }
}

/*
 * u8 x i8 GEMM with an activation zero point: out = sum_k (a[i,k] - a_zp) * b[k,j].
 * Definition: int8_matmul_scalar (int8_matmul.rs:195-208) applied to
 * a' = a - a_zp, computed directly in i32 (a' may not fit i8 for general a_zp;
 * for a_zp = 128 it is exactly `(a ^ 0x80) as i8`, the bias shift of
 * int8_matmul.rs:1866-1868).  The algebra acc - a_zp * colsum is
 * crates/yscv-onnx/src/runner/conv/quantized.rs:119-147.
 */
ORC_API void orc_u8i8_matmul_zp(const uint8_t *a, int32_t a_zp, const int8_t *b, size_t m,
                                size_t k, size_t n, int32_t *out) {
  for (size_t i = 0; i < m; i++) {
    for (size_t j = 0; j < n; j++) {
      int32_t acc = 0;
      for (size_t kk = 0; kk < k; kk++)
        acc = wrapping_add_i32(acc, ((int32_t)a[i * k + kk] - a_zp) * (int32_t)b[kk * n + j]);
      out[i * n + j] = acc;
    }
  }
}

/* ---- QuantizeLinear / requantize ------------------------------------------ */
/* crates/yscv-kernels/src/ops/quantize.rs:242-254 (quantize_linear_f32_to_i8_scalar) */
ORC_API void orc_quantize_linear_f32_to_i8(const float *data, size_t n, float scale,
                                           float zero_point, int8_t *output) {
  for (size_t i = 0; i < n; i++)
    output[i] = rust_f32_as_i8(rust_clampf(rintf(data[i] / scale + zero_point), -128.0f, 127.0f));
}

/* crates/yscv-kernels/src/ops/quantize.rs:226-238 (quantize_linear_f32_to_f32_i8_scalar) */
ORC_API void orc_quantize_linear_f32_to_f32_i8(const float *data, size_t n, float scale,
                                               float zero_point, float *output) {
  for (size_t i = 0; i < n; i++)
    output[i] = rust_clampf(rintf(data[i] / scale + zero_point), -128.0f, 127.0f);
}

/* crates/yscv-kernels/src/ops/int8_requant.rs:143-169 (requant_scalar); bias may be NULL. */
ORC_API void orc_requant_i32_row_to_i8(const int32_t *acc, size_t len, const int32_t *bias,
                                       float composite, float y_zp, int relu, int8_t *out,
                                       size_t c) {
  size_t pixels = len / c;
  for (size_t p = 0; p < pixels; p++) {
    for (size_t ch = 0; ch < c; ch++) {
      int32_t a = acc[p * c + ch];
      if (bias) a = wrapping_add_i32(a, bias[ch]);
      float v = (float)a * composite + y_zp;
      int8_t q = rust_f32_as_i8(rust_clampf(rintf(v), -128.0f, 127.0f));
      if (relu && q < 0) q = 0;
      out[p * c + ch] = q;
    }
  }
}

/* crates/yscv-kernels/src/ops/int8_requant.rs:537-555 (requant_i8_per_channel_scalar) */
ORC_API void orc_requant_i8_per_channel(const int32_t *acc, size_t len, const int32_t *corr,
                                        const float *composite, float y_zp, int8_t *out,
                                        size_t c) {
  size_t pixels = len / c;
  for (size_t p = 0; p < pixels; p++) {
    for (size_t ch = 0; ch < c; ch++) {
      int32_t a = wrapping_add_i32(acc[p * c + ch], corr[ch]);
      float v = (float)a * composite[ch] + y_zp;
      out[p * c + ch] = rust_f32_as_i8(rust_clampf(rintf(v), -128.0f, 127.0f));
    }
  }
}

/*
 * General requantize epilogue with a selectable rounding rule and clamp range,
 * out as i32 so both the i8 and the u8 range fit:
 *   round_mode 0: half away from zero -- QLinearMatMul fast path,
 *                 crates/yscv-onnx/src/runner/linear.rs:481-485
 *   round_mode 1: ties to even -- int8_requant.rs:161-162 / :550-552
 * corr / composite_v may be NULL (then corr = 0 and the scalar composite is
 * used).  [lo,hi] = [-128,127] reproduces the reference; [0,255] is the uint8
 * extension BASELINE config 2 asks for.
 */
ORC_API void orc_requant_general(const int32_t *acc, size_t len, size_t c, const int32_t *corr,
                                 const float *composite_v, float composite_s, float y_zp,
                                 int round_mode, float lo, float hi, int32_t *out) {
  for (size_t i = 0; i < len; i++) {
    size_t ch = i % c;
    int32_t a = acc[i];
    if (corr) a = wrapping_add_i32(a, corr[ch]);
    float comp = composite_v ? composite_v[ch] : composite_s;
    float v = (float)a * comp + y_zp;
    float r = round_mode == 0 ? roundf(v) : rintf(v);
    out[i] = rust_f32_as_i32(rust_clampf(r, lo, hi));
  }
}

/* crates/yscv-onnx/src/runner/misc.rs:241-289 (exec_dynamic_quantize_linear).
 * y holds the uint8 values as f32 carriers, exactly like the reference tensor. */
ORC_API void orc_dynamic_quantize_linear(const float *data, size_t n, float *y, float *y_scale,
                                         float *y_zp) {
  float min_val = 3.40282347e+38f;
  float max_val = -3.40282347e+38f;
  for (size_t i = 0; i < n; i++) {
    float v = data[i];
    if (v < min_val) min_val = v;
    if (v > max_val) max_val = v;
  }
  const float qmin = 0.0f, qmax = 255.0f;
  min_val = rust_minf(min_val, 0.0f);
  max_val = rust_maxf(max_val, 0.0f);
  float scale = (fabsf(max_val - min_val) < F32_EPSILON) ? 1.0f : (max_val - min_val) / (qmax - qmin);
  float zero_point = rust_clampf(roundf(qmin - min_val / scale), qmin, qmax);
  for (size_t i = 0; i < n; i++) y[i] = rust_clampf(roundf(data[i] / scale + zero_point), qmin, qmax);
  *y_scale = scale;
  *y_zp = zero_point;
}

/* crates/yscv-onnx/src/runner/misc.rs:184-188 (DequantizeLinear, per tensor, f32 carrier in). */
ORC_API void orc_dequantize_linear(const float *q, size_t n, float scale, float zp, float *out) {
  for (size_t i = 0; i < n; i++) out[i] = (q[i] - zp) * scale;
}

/* ---- ONNX operator semantics (f32 carriers, as the reference runner) ------ */
/* Sequential-k f32 matmul used by the operator fallbacks below.  The reference
 * routes the fallback through its blocked f32 GEMM whose summation order is not
 * restated here; results agree exactly whenever every partial sum is an
 * integer below 2^24, which is the case for all fixtures that pin it. */
static void f32_matmul_seq(const float *a, const float *b, size_t m, size_t k, size_t n,
                           float *out) {
  for (size_t i = 0; i < m; i++)
    for (size_t j = 0; j < n; j++) {
      float acc = 0.0f;
      for (size_t kk = 0; kk < k; kk++) acc += a[i * k + kk] * b[kk * n + j];
      out[i * n + j] = acc;
    }
}

/* crates/yscv-onnx/src/runner/linear.rs:648-737 (exec_matmul_integer), rank 2.
 * Returns 1 when the integer fast path was taken, 0 for the f32 fallback. */
ORC_API int orc_exec_matmul_integer(const float *a, const float *b, float a_zp, float b_zp,
                                    size_t m, size_t k, size_t n, float *out) {
  if (a_zp == 0.0f && b_zp == 0.0f) {
    int8_t *a8 = (int8_t *)malloc(m * k), *b8 = (int8_t *)malloc(k * n);
    int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * m * n);
    for (size_t i = 0; i < m * k; i++) a8[i] = rust_f32_as_i8(a[i]);
    for (size_t i = 0; i < k * n; i++) b8[i] = rust_f32_as_i8(b[i]);
    orc_int8_matmul_scalar(a8, b8, m, k, n, acc);
    for (size_t i = 0; i < m * n; i++) out[i] = (float)acc[i];
    free(a8);
    free(b8);
    free(acc);
    return 1;
  }
  float *da = (float *)malloc(sizeof(float) * m * k), *db = (float *)malloc(sizeof(float) * k * n);
  for (size_t i = 0; i < m * k; i++) da[i] = a[i] - a_zp;
  for (size_t i = 0; i < k * n; i++) db[i] = b[i] - b_zp;
  f32_matmul_seq(da, db, m, k, n, out);
  for (size_t i = 0; i < m * n; i++) out[i] = roundf(out[i]);
  free(da);
  free(db);
  return 0;
}

/* crates/yscv-onnx/src/runner/linear.rs:438-538 (exec_qlinear_matmul), rank 2.
 * Returns 1 for the fast path, 0 for the fallback. */
ORC_API int orc_exec_qlinear_matmul(const float *a, float a_scale, float a_zp, const float *b,
                                    float b_scale, float b_zp, float y_scale, float y_zp,
                                    size_t m, size_t k, size_t n, float *out) {
  if (a_zp == 0.0f && b_zp == 0.0f) {
    int8_t *a8 = (int8_t *)malloc(m * k), *b8 = (int8_t *)malloc(k * n);
    int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * m * n);
    for (size_t i = 0; i < m * k; i++) a8[i] = rust_f32_as_i8(a[i]);
    for (size_t i = 0; i < k * n; i++) b8[i] = rust_f32_as_i8(b[i]);
    orc_int8_matmul_scalar(a8, b8, m, k, n, acc);
    float composite = (a_scale * b_scale) / y_scale;
    for (size_t i = 0; i < m * n; i++)
      out[i] = rust_clampf(roundf((float)acc[i] * composite + y_zp), -128.0f, 127.0f);
    free(a8);
    free(b8);
    free(acc);
    return 1;
  }
  float *da = (float *)malloc(sizeof(float) * m * k), *db = (float *)malloc(sizeof(float) * k * n);
  for (size_t i = 0; i < m * k; i++) da[i] = (a[i] - a_zp) * a_scale;
  for (size_t i = 0; i < k * n; i++) db[i] = (b[i] - b_zp) * b_scale;
  f32_matmul_seq(da, db, m, k, n, out);
  for (size_t i = 0; i < m * n; i++)
    out[i] = rust_clampf(roundf(out[i] / y_scale + y_zp), -128.0f, 127.0f);
  free(da);
  free(db);
  return 0;
}

/* crates/yscv-onnx/src/runner/layout.rs:6-11 */
ORC_API int orc_should_use_prepacked_i8_b(size_t m, size_t k, size_t n) {
  return (m >= 4 && k >= 4 && n >= 32 && n % 16 == 0) || (m <= 64 && k >= 512 && n >= 1024);
}
/* crates/yscv-onnx/src/plan/build.rs:1371-1377 */
ORC_API int orc_should_prepack_i8_b(size_t k, size_t n) {
  return (k >= 4 && n % 16 == 0) || (k >= 512 && n >= 1024);
}

/* ---- KV cache int8 row quantisation --------------------------------------- */
/* crates/yscv-onnx/src/runner/kv_cache.rs:45-61 (LayerStorage::append, I8 arm) */
ORC_API void orc_kv_i8_quantize_rows(const float *src, size_t rows, size_t kv_dim, int8_t *data,
                                     float *scales) {
  for (size_t r = 0; r < rows; r++) {
    const float *row = src + r * kv_dim;
    float abs_max = 0.0f;
    for (size_t i = 0; i < kv_dim; i++) abs_max = rust_maxf(abs_max, fabsf(row[i]));
    float scale = (abs_max <= F32_EPSILON) ? 1.0f : abs_max / 127.0f;
    float inv = 1.0f / scale;
    scales[r] = scale;
    for (size_t i = 0; i < kv_dim; i++)
      data[r * kv_dim + i] = rust_f32_as_i8(rust_clampf(roundf(row[i] * inv), -127.0f, 127.0f));
  }
}

/* apps/llm-bench/src/main.rs:538-543 -- greedy pick: Iterator::max_by returns
 * the LAST of several equal maxima; incomparable (NaN) pairs count as equal. */
ORC_API uint32_t orc_argmax_last(const float *logits, size_t n) {
  if (n == 0) return 0;
  size_t best = 0;
  for (size_t i = 1; i < n; i++) {
    /* max_by keeps the new element when compare(best, new) != Greater */
    int greater = logits[best] > logits[i];
    if (!greater) best = i;
  }
  return (uint32_t)best;
}

/* ---- seeded inputs ---------------------------------------------------------- */
/* apps/llm-bench/src/bin/kernel_bench.rs:28-50 (pseudo_i8 / pseudo_f32) */
ORC_API void orc_lcg_i8(uint64_t seed, size_t n, int8_t *out) {
  uint64_t s = seed;
  for (size_t i = 0; i < n; i++) {
    s = s * 6364136223846793005ULL + 1442695040888963407ULL;
    out[i] = (int8_t)((int64_t)(s >> 33) % 256 - 128);
  }
}
ORC_API void orc_lcg_f32(uint64_t seed, size_t n, float *out) {
  uint64_t s = seed;
  for (size_t i = 0; i < n; i++) {
    s = s * 6364136223846793005ULL + 1442695040888963407ULL;
    out[i] = (float)((int64_t)(s >> 33) % 2001 - 1000) * 0.001f;
  }
}
