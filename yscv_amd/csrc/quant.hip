// Elementwise quantisation kernels, bit-exact with the reference's scalar definitions:
//   quantize_linear_f32_to_i8_scalar     crates/yscv-kernels/src/ops/quantize.rs:242-254
//   requant_scalar                       crates/yscv-kernels/src/ops/int8_requant.rs:143-169
//   requant_i8_per_channel_scalar        crates/yscv-kernels/src/ops/int8_requant.rs:537-555
//   exec_dynamic_quantize_linear         crates/yscv-onnx/src/runner/misc.rs:241-289
// All of them are one pass over HBM; the arithmetic uses explicitly rounded single
// operations (no FMA contraction, IEEE division) because the Rust source never fuses.
#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

__device__ __forceinline__ float round_half_away_f(float v) {
  float t = truncf(v);
  float d = fabsf(__fsub_rn(v, t));
  return (d >= 0.5f) ? __fadd_rn(t, copysignf(1.0f, v)) : t;
}

// clamp that keeps NaN, then the saturating NaN->0 integer cast of Rust's `as`
__device__ __forceinline__ int clamp_cast(float r, float lo, float hi) {
  if (r != r) return 0;
  return (int)fminf(fmaxf(r, lo), hi);
}

__global__ void quantize_linear_i8_kernel(const float *__restrict__ x, size_t len, float scale, float zp,
                                          int8_t *__restrict__ out) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < len;
       i += (size_t)gridDim.x * blockDim.x) {
    float v = __fadd_rn(__fdiv_rn(x[i], scale), zp);
    out[i] = (int8_t)clamp_cast(rintf(v), -128.0f, 127.0f);
  }
}

int32_t launch_quantize_linear_i8(const float *x, size_t len, float scale, float zp, int8_t *out,
                                  hipStream_t s) {
  size_t blocks = ceil_div(len, (size_t)256);
  if (blocks > 16384) blocks = 16384;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(quantize_linear_i8_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, len, scale,
                     zp, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// quantize_f32_to_int4 (crates/yscv-kernels/src/ops/quantize.rs:69-95): q = clamp(round_ties_even(x * inv_scale) as
// i32 + zp, -8, 7) with inv_scale = 1 / scale, or 0 when |scale| <= f32::EPSILON; element 2i in the low nibble, the
// high nibble of an odd tail is 0.  `as i32` saturates and maps NaN to 0; the addition of zp wraps.
__device__ __forceinline__ int quant_int4_one(float x, float inv_scale, int zp) {
  const float r = rintf(__fmul_rn(x, inv_scale));
  int32_t q;
  if (r != r) q = 0;
  else if (r >= 2147483648.0f) q = INT32_MAX;
  else if (r <= -2147483648.0f) q = INT32_MIN;
  else q = (int32_t)r;
  q = (int32_t)((uint32_t)q + (uint32_t)zp);
  return q < -8 ? -8 : (q > 7 ? 7 : q);
}
__global__ void quantize_int4_kernel(const float *__restrict__ x, size_t len, float inv_scale, int zp,
                                     uint8_t *__restrict__ out) {
  const size_t n_out = (len + 1) / 2;
  for (size_t o = blockIdx.x * (size_t)blockDim.x + threadIdx.x; o < n_out; o += (size_t)gridDim.x * blockDim.x) {
    const int q0 = quant_int4_one(x[2 * o], inv_scale, zp);
    const int q1 = (2 * o + 1 < len) ? quant_int4_one(x[2 * o + 1], inv_scale, zp) : 0;
    out[o] = (uint8_t)((q0 & 0x0F) | ((q1 & 0x0F) << 4));
  }
}

int32_t launch_quantize_f32_to_int4(const float *x, size_t len, float scale, int zp, uint8_t *out, hipStream_t s) {
  if (len == 0) return YSCV_HIP_OK;
  const float inv_scale = fabsf(scale) > 1.1920929e-7f ? 1.0f / scale : 0.0f;  // host IEEE division, as the reference's
  size_t blocks = ceil_div((len + 1) / 2, (size_t)256);
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(quantize_int4_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, len, inv_scale, zp, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

__global__ void requant_kernel(const int32_t *__restrict__ acc, size_t len, size_t c,
                               const int32_t *__restrict__ corr, const float *__restrict__ composite_v,
                               float composite, float y_zp, int round_mode, float lo, float hi, int relu,
                               uint8_t *__restrict__ out) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < len;
       i += (size_t)gridDim.x * blockDim.x) {
    size_t ch = i % c;
    int32_t a = acc[i];
    if (corr) a = (int32_t)((uint32_t)a + (uint32_t)corr[ch]);
    float comp = composite_v ? composite_v[ch] : composite;
    float v = __fadd_rn(__fmul_rn((float)a, comp), y_zp);
    float r = round_mode == YSCV_HIP_ROUND_HALF_AWAY ? round_half_away_f(v) : rintf(v);
    int q = clamp_cast(r, lo, hi);
    if (relu && q < 0) q = 0;
    out[i] = (uint8_t)q;
  }
}

int32_t launch_requant(const int32_t *acc, size_t len, size_t c, const int32_t *corr,
                       const float *composite_v, float composite, float y_zp, int round_mode, int lo,
                       int hi, int relu, void *out, hipStream_t s) {
  size_t blocks = ceil_div(len, (size_t)256);
  if (blocks > 16384) blocks = 16384;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(requant_kernel, dim3((unsigned)blocks), dim3(256), 0, s, acc, len, c, corr,
                     composite_v, composite, y_zp, round_mode, (float)lo, (float)hi, relu,
                     static_cast<uint8_t *>(out));
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// ---- DynamicQuantizeLinear ---------------------------------------------------------------
// Pass 1: every workgroup writes its min / max to minmax[2*block].  Pass 2: every workgroup
// re-reduces those few hundred partials (cheaper than a third launch), derives scale and
// zero point exactly as the reference does, and quantises its share.
constexpr int DQL_BLOCKS = 1024;

__global__ void __launch_bounds__(256) dql_minmax_kernel(const float *__restrict__ x, size_t len,
                                                         float *__restrict__ minmax) {
  __shared__ float smin[4], smax[4];
  float mn = 3.40282347e+38f, mx = -3.40282347e+38f;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < len;
       i += (size_t)gridDim.x * blockDim.x) {
    float v = x[i];
    if (v < mn) mn = v;  // comparisons, not fmin: NaN never wins, as in misc.rs:250-256
    if (v > mx) mx = v;
  }
  for (int off = 32; off > 0; off >>= 1) {
    float a = __shfl_xor(mn, off, 64), b = __shfl_xor(mx, off, 64);
    if (a < mn) mn = a;
    if (b > mx) mx = b;
  }
  if ((threadIdx.x & 63) == 0) {
    smin[threadIdx.x >> 6] = mn;
    smax[threadIdx.x >> 6] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++) {
      if (smin[w] < mn) mn = smin[w];
      if (smax[w] > mx) mx = smax[w];
    }
    minmax[2 * blockIdx.x] = mn;
    minmax[2 * blockIdx.x + 1] = mx;
  }
}

__global__ void __launch_bounds__(256) dql_quantize_kernel(const float *__restrict__ x, size_t len,
                                                           const float *__restrict__ minmax, int nparts,
                                                           uint8_t *__restrict__ y,
                                                           float *__restrict__ scale_zp) {
  __shared__ float smin[4], smax[4];
  float mn = 3.40282347e+38f, mx = -3.40282347e+38f;
  for (int i = threadIdx.x; i < nparts; i += blockDim.x) {
    float a = minmax[2 * i], b = minmax[2 * i + 1];
    if (a < mn) mn = a;
    if (b > mx) mx = b;
  }
  for (int off = 32; off > 0; off >>= 1) {
    float a = __shfl_xor(mn, off, 64), b = __shfl_xor(mx, off, 64);
    if (a < mn) mn = a;
    if (b > mx) mx = b;
  }
  if ((threadIdx.x & 63) == 0) {
    smin[threadIdx.x >> 6] = mn;
    smax[threadIdx.x >> 6] = mx;
  }
  __syncthreads();
  mn = smin[0];
  mx = smax[0];
  for (int w = 1; w < 4; w++) {
    if (smin[w] < mn) mn = smin[w];
    if (smax[w] > mx) mx = smax[w];
  }
  mn = fminf(mn, 0.0f);  // f32::min / f32::max: range always contains 0 (misc.rs:260-261)
  mx = fmaxf(mx, 0.0f);
  const float range = __fsub_rn(mx, mn);
  const float scale = (fabsf(range) < 1.1920929e-7f) ? 1.0f : __fdiv_rn(range, 255.0f);
  float zp = round_half_away_f(__fsub_rn(0.0f, __fdiv_rn(mn, scale)));
  if (zp == zp) zp = fminf(fmaxf(zp, 0.0f), 255.0f);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    scale_zp[0] = scale;
    scale_zp[1] = zp;
  }
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < len;
       i += (size_t)gridDim.x * blockDim.x) {
    float v = __fadd_rn(__fdiv_rn(x[i], scale), zp);
    y[i] = (uint8_t)clamp_cast(round_half_away_f(v), 0.0f, 255.0f);
  }
}

int32_t launch_dynamic_quantize_linear(const float *x, size_t len, uint8_t *y, float *scale_zp,
                                       hipStream_t s) {
  int blocks = (int)ceil_div(len, (size_t)1024);
  if (blocks > DQL_BLOCKS) blocks = DQL_BLOCKS;
  if (blocks < 1) blocks = 1;
  float *minmax = nullptr;
  YSCV_HIP_TRY(hipMallocAsync(reinterpret_cast<void **>(&minmax), sizeof(float) * 2 * blocks, s));
  hipLaunchKernelGGL(dql_minmax_kernel, dim3(blocks), dim3(256), 0, s, x, len, minmax);
  hipError_t e1 = hipGetLastError();
  hipLaunchKernelGGL(dql_quantize_kernel, dim3(blocks), dim3(256), 0, s, x, len, minmax, blocks, y,
                     scale_zp);
  hipError_t e2 = hipGetLastError();
  hipError_t e3 = hipFreeAsync(minmax, s);
  YSCV_HIP_TRY(e1);
  YSCV_HIP_TRY(e2);
  YSCV_HIP_TRY(e3);
  return YSCV_HIP_OK;
}

// ---- KV-cache int8 storage: per-row symmetric quantisation (crates/yscv-onnx/src/runner/kv_cache.rs:45-61) ----
// One wavefront per appended row: abs-max (f32::max ignores NaN), scale = abs_max / 127 (1.0 when abs_max <=
// EPSILON), q = clamp(round_half_away(v * (1 / scale)), -127, 127) as i8.
__global__ void __launch_bounds__(256) kv_i8_quantize_rows_kernel(const float *__restrict__ src, size_t rows, size_t kv_dim,
                                                                  int8_t *__restrict__ data, float *__restrict__ scales) {
  const size_t row = blockIdx.x * (size_t)(blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const float *x = src + row * kv_dim;
  float amax = 0.0f;
  for (size_t i = lane; i < kv_dim; i += 64) amax = fmaxf(amax, fabsf(x[i]));  // fmaxf drops NaN like f32::max
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  const float scale = (amax <= 1.1920929e-7f) ? 1.0f : __fdiv_rn(amax, 127.0f);
  const float inv = __fdiv_rn(1.0f, scale);
  if (lane == 0) scales[row] = scale;
  for (size_t i = lane; i < kv_dim; i += 64)
    data[row * kv_dim + i] = (int8_t)clamp_cast(round_half_away_f(__fmul_rn(x[i], inv)), -127.0f, 127.0f);
}

// LayerStorage::dequantise_to_vec (kv_cache.rs:64-79): q as f32 * scale of its row
__global__ void kv_i8_dequantize_rows_kernel(const int8_t *__restrict__ data, const float *__restrict__ scales, size_t rows,
                                             size_t kv_dim, float *__restrict__ out) {
  const size_t total = rows * kv_dim;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    out[i] = __fmul_rn((float)data[i], scales[i / kv_dim]);
}

int32_t launch_kv_i8_quantize_rows(const float *src, size_t rows, size_t kv_dim, int8_t *data, float *scales, hipStream_t s) {
  hipLaunchKernelGGL(kv_i8_quantize_rows_kernel, dim3((unsigned)ceil_div(rows, (size_t)4)), dim3(256), 0, s, src, rows, kv_dim,
                     data, scales);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_kv_i8_dequantize_rows(const int8_t *data, const float *scales, size_t rows, size_t kv_dim, float *out,
                                     hipStream_t s) {
  size_t blocks = ceil_div(rows * kv_dim, (size_t)256);
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(kv_i8_dequantize_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, s, data, scales, rows, kv_dim, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

}  // namespace yscv
