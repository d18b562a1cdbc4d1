// ONNX operator entry points of the quantised matmul path.  Tensors are device-resident f32
// "carriers" exactly as the reference runner keeps them (every quantised value is an f32 holding an
// integer), so a graph executor can call these where the reference calls
//   exec_matmul_integer          crates/yscv-onnx/src/runner/linear.rs:648-737
//   exec_qlinear_matmul          crates/yscv-onnx/src/runner/linear.rs:438-538
//   exec_quantize_linear         crates/yscv-onnx/src/runner/misc.rs:42-108 (f32-carrier arm)
//   exec_dequantize_linear       crates/yscv-onnx/src/runner/misc.rs:110-239
//   exec_dynamic_quantize_linear crates/yscv-onnx/src/runner/misc.rs:241-289
// and read the same fast/fallback counters (crates/yscv-onnx/src/runner/quant_stats.rs:6-92).
//
// Fast path (both zero points 0): operands are cast with Rust's saturating `as i8`, the product runs on the
// int8 MFMA kernel, the epilogue follows the reference expression by expression.
//
// Fallback (a zero point is non-zero): the reference dequantises to f32 and calls its float matmul.  When
// every operand value is an integer that fits 8 bits the same quantity is computed exactly here,
//   sum_k (a - a_zp)(b - b_zp) = sum_k A'B' - a_zp' colsum(B')[j] - b_zp' (rowsum(A')[i] - K a_zp'),
// with A' the operand shifted into u8, B' shifted into i8 and the zero points shifted alike, on the
// same MFMA kernel.  That equals the reference's f32 result whenever the latter is exact (all partial
// sums below 2^24) and is the correctly rounded value otherwise.  Operands that are not 8-bit integers
// take a plain f32 kernel that adds the products in k order with separately rounded multiply and add.
#include <atomic>
#include <cstdlib>

#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {
namespace {

std::atomic<uint64_t> g_qlinear_fast{0}, g_qlinear_fallback{0}, g_mmi_fast{0}, g_mmi_fallback{0},
    g_int4_fast{0}, g_int4_fallback{0};

__device__ __forceinline__ float round_half_away(float v) {
  float t = truncf(v);
  float d = fabsf(__fsub_rn(v, t));
  return (d >= 0.5f) ? __fadd_rn(t, copysignf(1.0f, v)) : t;
}
// f32::clamp: NaN stays NaN
__device__ __forceinline__ float clamp_keep_nan(float r, float lo, float hi) {
  return (r != r) ? r : fminf(fmaxf(r, lo), hi);
}
// Rust `v as i8`: NaN -> 0, saturating, truncation toward zero
__device__ __forceinline__ int8_t f32_as_i8(float v) {
  if (v != v) return 0;
  if (v <= -128.0f) return -128;
  if (v >= 127.0f) return 127;
  return (int8_t)(int)v;
}

inline unsigned grid_for(size_t len, unsigned per_block = 256) {
  size_t blocks = ceil_div(len, (size_t)per_block);
  if (blocks > 16384) blocks = 16384;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

#define GRID_STRIDE(i, len) \
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < (len); i += (size_t)gridDim.x * blockDim.x)

// round_first: `v.round() as i8` (load-time prepack), else `v as i8` (per-call cast)
__global__ void cast_as_i8_kernel(const float *__restrict__ x, size_t len, int round_first, int8_t *__restrict__ out) {
  GRID_STRIDE(i, len) out[i] = f32_as_i8(round_first ? round_half_away(x[i]) : x[i]);
}

// info[0] = min, info[1] = max (as integers), info[2] != 0 when a value is not an integer in [-1024, 1024]
__global__ void scan_int_range_kernel(const float *__restrict__ x, size_t len, int *__restrict__ info) {
  int lo = 1 << 20, hi = -(1 << 20), bad = 0;
  GRID_STRIDE(i, len) {
    float v = x[i];
    if (!(fabsf(v) <= 1024.0f) || truncf(v) != v) {
      bad = 1;
    } else {
      int q = (int)v;
      lo = min(lo, q);
      hi = max(hi, q);
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    lo = min(lo, __shfl_xor(lo, o));
    hi = max(hi, __shfl_xor(hi, o));
    bad |= __shfl_xor(bad, o);
  }
  if ((threadIdx.x & 63) == 0) {
    atomicMin(&info[0], lo);
    atomicMax(&info[1], hi);
    if (bad) atomicOr(&info[2], 1);
  }
}
__global__ void init_range_kernel(int *info) {
  if (threadIdx.x < 2) {
    info[threadIdx.x * 4 + 0] = 1 << 20;
    info[threadIdx.x * 4 + 1] = -(1 << 20);
    info[threadIdx.x * 4 + 2] = 0;
    info[threadIdx.x * 4 + 3] = 0;
  }
}

__global__ void cast_shift_kernel(const float *__restrict__ x, size_t len, int shift, uint8_t *__restrict__ out) {
  GRID_STRIDE(i, len) out[i] = (uint8_t)((int)x[i] + shift);
}

// one wavefront per row of the u8 matrix
__global__ void row_sum_u8_kernel(const uint8_t *__restrict__ a, size_t m, size_t k, int32_t *__restrict__ rs) {
  const size_t row = blockIdx.x * (size_t)(blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= m) return;
  const int lane = threadIdx.x & 63;
  int s = 0;
  for (size_t c = lane; c < k; c += 64) s += a[row * k + c];
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) rs[row] = s;
}

// mode 0: out = f32(acc')                 (MatMulInteger)
// mode 1: out = clamp(round(f32(acc') * composite + y_zp))       (QLinearMatMul fast path)
// mode 2: out = clamp(round(f32(acc' * ab_scale) / y_scale + y_zp))  (QLinearMatMul, asymmetric)
// acc' = acc - b_zp * (rs[i] - k_azp) when rs != null
__global__ void mm_post_kernel(const int32_t *__restrict__ acc, const int32_t *__restrict__ rs, int b_zp, int k_azp,
                               size_t m, size_t n, int mode, float composite, double ab_scale, float y_scale,
                               float y_zp, float *__restrict__ out) {
  GRID_STRIDE(i, m * n) {
    int32_t a = acc[i];
    if (rs) a = (int32_t)((uint32_t)a - (uint32_t)b_zp * ((uint32_t)rs[i / n] - (uint32_t)k_azp));  // wraps like the sum itself
    float r;
    if (mode == 0) {
      r = (float)a;
    } else if (mode == 1) {
      r = clamp_keep_nan(round_half_away(__fadd_rn(__fmul_rn((float)a, composite), y_zp)), -128.0f, 127.0f);
    } else {
      float v = (float)((double)a * ab_scale);
      r = clamp_keep_nan(round_half_away(__fadd_rn(__fdiv_rn(v, y_scale), y_zp)), -128.0f, 127.0f);
    }
    out[i] = r;
  }
}

// Plain f32 product of the dequantised operands in k order; mode as in mm_post_kernel (0 rounds the sum,
// 2 requantises it).  One output element per lane, B read coalesced along n.
__global__ void f32_fallback_kernel(const float *__restrict__ a, const float *__restrict__ b, size_t m, size_t k,
                                    size_t n, float a_zp, float a_scale, float b_zp, float b_scale, int mode,
                                    float y_scale, float y_zp, float *__restrict__ out) {
  const size_t j = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  const size_t i = blockIdx.y;
  if (j >= n || i >= m) return;
  float s = 0.0f;
  for (size_t kk = 0; kk < k; kk++) {
    float av = __fsub_rn(a[i * k + kk], a_zp);
    float bv = __fsub_rn(b[kk * n + j], b_zp);
    if (mode == 2) {
      av = __fmul_rn(av, a_scale);
      bv = __fmul_rn(bv, b_scale);
    }
    s = __fadd_rn(s, __fmul_rn(av, bv));
  }
  out[i * n + j] = (mode == 0)
                       ? round_half_away(s)
                       : clamp_keep_nan(round_half_away(__fadd_rn(__fdiv_rn(s, y_scale), y_zp)), -128.0f, 127.0f);
}

__global__ void quantize_linear_f32_kernel(const float *__restrict__ x, size_t len, float scale, float zp,
                                           float *__restrict__ out) {
  GRID_STRIDE(i, len) out[i] = clamp_keep_nan(rintf(__fadd_rn(__fdiv_rn(x[i], scale), zp)), -128.0f, 127.0f);
}

// scales / zps: one entry (chan == 1) or one per index of the quantisation axis
__global__ void dequantize_linear_f32_kernel(const float *__restrict__ q, size_t len, size_t chan, size_t inner,
                                             const float *__restrict__ scales, const float *__restrict__ zps,
                                             float *__restrict__ out) {
  GRID_STRIDE(i, len) {
    const size_t c = chan == 1 ? 0 : (i / inner) % chan;
    const float zp = zps ? zps[c] : 0.0f;
    out[i] = __fmul_rn(__fsub_rn(q[i], zp), scales[c]);
  }
}

__global__ void u8_to_f32_kernel(const uint8_t *__restrict__ q, size_t len, const float *__restrict__ scale_zp,
                                 float *__restrict__ y, float *__restrict__ scale_out, float *__restrict__ zp_out) {
  GRID_STRIDE(i, len) y[i] = (float)q[i];
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *scale_out = scale_zp[0];
    *zp_out = scale_zp[1];
  }
}

// [d0][d1] -> [d1][d0]
__global__ void transpose_f32_kernel(const float *__restrict__ in, size_t d0, size_t d1, float *__restrict__ out) {
  __shared__ float tile[32][33];
  const size_t x = blockIdx.x * 32 + threadIdx.x, y0 = blockIdx.y * 32;
  for (int j = threadIdx.y; j < 32; j += blockDim.y)
    if (x < d1 && y0 + j < d0) tile[j][threadIdx.x] = in[(y0 + j) * d1 + x];
  __syncthreads();
  const size_t ox = blockIdx.y * 32 + threadIdx.x, oy0 = blockIdx.x * 32;
  for (int j = threadIdx.y; j < 32; j += blockDim.y)
    if (ox < d0 && oy0 + j < d1) out[(oy0 + j) * d0 + ox] = tile[threadIdx.x][j];
}

struct Operand8 {
  DevBuf buf;
  int shift = 0;    // added to every value
  bool ok = false;  // values are integers that fit the 8-bit target after the shift
};

bool is_int_in(float v, int lo, int hi) { return v == (float)(int)v && (int)v >= lo && (int)v <= hi; }

// y[m][n] (f32) = (alpha != 1 ? y * alpha : y) + (beta != 1 ? c * beta : c), each multiply and add rounded on its own
// like Tensor::scale followed by kernel_add in exec_gemm (crates/yscv-onnx/src/runner/linear.rs:54-66); c is null,
// one row [n] broadcast over the rows, or [m][n].  c_rows: 0 none, 1 broadcast, m full.
__global__ void gemm_post_kernel(float *__restrict__ y, size_t m, size_t n, const float *__restrict__ c, size_t c_rows,
                                 float alpha, int use_alpha, float beta, int use_beta) {
  const size_t total = m * n;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    float v = y[i];
    if (use_alpha) v = __fmul_rn(v, alpha);
    if (c) {
      float a = c[c_rows == 1 ? i % n : i];
      if (use_beta) a = __fmul_rn(a, beta);
      v = __fadd_rn(v, a);
    }
    y[i] = v;
  }
}
// out[m][n] (f32 / f16 / bf16) = acc[m][n] (f32) + bias[n]: the f32 sum is rounded once to the output type
__global__ void bias_cast_kernel(const float *__restrict__ acc, size_t m, size_t n, const float *__restrict__ bias,
                                 void *__restrict__ out, int out_dtype) {
  const size_t total = m * n;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const float v = __fadd_rn(acc[i], bias[i % n]);
    if (out_dtype == YSCV_HIP_F32) static_cast<float *>(out)[i] = v;
    else if (out_dtype == YSCV_HIP_F16) static_cast<_Float16 *>(out)[i] = (_Float16)v;
    else static_cast<uint16_t *>(out)[i] = float_to_bf16_bits(v);
  }
}

int32_t free_weight(yscv_hip_i8_weight *w) {
  if (!w) return YSCV_HIP_OK;
  if (w->frag) (void)hipFree(w->frag);
  if (w->col_sum) (void)hipFree(w->col_sum);
  delete w;
  return YSCV_HIP_OK;
}

// device i8 [k][n] -> fragment layout + column sums
int32_t pack_device_i8(const int8_t *b_kn, size_t k, size_t n, hipStream_t s, yscv_hip_i8_weight **out) {
  auto *b = new yscv_hip_i8_weight();
  b->k = k;
  b->n = n;
  b->kp = round_up(k, 64);
  b->np = round_up(n, 16);
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&b->frag), b->kp * b->np);
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&b->col_sum), b->np * sizeof(int32_t));
  int32_t st = YSCV_HIP_OK;
  if (e == hipSuccess) st = launch_i8_pack_b(b_kn, k, n, b->kp, b->np, b->frag, b->col_sum, s);
  if (e != hipSuccess || st != YSCV_HIP_OK) {
    free_weight(b);
    if (st != YSCV_HIP_OK) return st;
    return set_error(e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE, "packing B failed: %s",
                     hipGetErrorString(e));
  }
  b->device_bytes = b->kp * b->np + b->np * sizeof(int32_t);
  *out = b;
  return YSCV_HIP_OK;
}

struct TempWeight {
  yscv_hip_i8_weight *w = nullptr;
  ~TempWeight() { free_weight(w); }
};

enum : int { OP_MATMUL_INTEGER = 0, OP_QLINEAR = 1 };

struct MatmulArgs {
  int op;
  const float *a;
  const float *b;                     // [k][n] carrier or null
  const yscv_hip_i8_weight *b_packed;  // or null
  size_t m, k, n;
  float a_scale, a_zp, b_scale, b_zp, y_scale, y_zp;
  float *out;
  hipStream_t s;
};

int32_t run_fast(const MatmulArgs &g) {
  if (g.b_packed) {
    // the usual case, a weight packed at load time: cast kernel + GEMM whose epilogue writes the f32 carriers, the
    // int8 copy of A in stream-ordered scratch -- nothing here waits for the device
    StreamBuf a8;
    YSCV_TRY(a8.alloc(g.m * g.k, g.s));
    hipLaunchKernelGGL(cast_as_i8_kernel, dim3(grid_for(g.m * g.k)), dim3(256), 0, g.s, g.a, g.m * g.k, 0, a8.as<int8_t>());
    YSCV_HIP_TRY(hipGetLastError());
    I8Epilogue ep{};
    if (g.op == OP_QLINEAR) {
      ep.mode = 4;
      ep.composite = (g.a_scale * g.b_scale) / g.y_scale;
      ep.y_zp = g.y_zp;
      ep.round_mode = YSCV_HIP_ROUND_HALF_AWAY;
      ep.lo = -128;
      ep.hi = 127;
    } else {
      ep.mode = 3;
    }
    return launch_i8_gemm(a8.p, 0, 0, g.b_packed, g.m, g.out, ep, g.s);
  }
  DevBuf a8, b8, acc;
  YSCV_TRY(a8.alloc(g.m * g.k));
  YSCV_TRY(acc.alloc(g.m * g.n * sizeof(int32_t)));
  hipLaunchKernelGGL(cast_as_i8_kernel, dim3(grid_for(g.m * g.k)), dim3(256), 0, g.s, g.a, g.m * g.k, 0, a8.as<int8_t>());
  TempWeight tmp;
  YSCV_TRY(b8.alloc(g.k * g.n));
  hipLaunchKernelGGL(cast_as_i8_kernel, dim3(grid_for(g.k * g.n)), dim3(256), 0, g.s, g.b, g.k * g.n, 0,
                     b8.as<int8_t>());
  YSCV_TRY(pack_device_i8(b8.as<int8_t>(), g.k, g.n, g.s, &tmp.w));
  const yscv_hip_i8_weight *w = tmp.w;
  I8Epilogue ep{};
  ep.mode = 0;
  YSCV_TRY(launch_i8_gemm(a8.p, 0, 0, w, g.m, acc.p, ep, g.s));
  const float composite = g.op == OP_QLINEAR ? (g.a_scale * g.b_scale) / g.y_scale : 0.0f;
  hipLaunchKernelGGL(mm_post_kernel, dim3(grid_for(g.m * g.n)), dim3(256), 0, g.s, acc.as<int32_t>(),
                     (const int32_t *)nullptr, 0, 0, g.m, g.n, g.op == OP_QLINEAR ? 1 : 0, composite, 0.0, g.y_scale,
                     g.y_zp, g.out);
  YSCV_HIP_TRY(hipGetLastError());
  YSCV_HIP_TRY(hipStreamSynchronize(g.s));  // the scratch buffers and the temporary weight are released on return
  return YSCV_HIP_OK;
}

int32_t run_fallback(const MatmulArgs &g, int *took_integer_route) {
  *took_integer_route = 0;
  // operand ranges decide whether the exact integer route applies
  DevBuf info;
  YSCV_TRY(info.alloc(8 * sizeof(int)));
  int h[8] = {0};
  bool integer_route = g.k * (size_t)65025 < ((size_t)1 << 31) && is_int_in(g.a_zp, -128, 255) &&
                       is_int_in(g.b_zp, -128, 255);
  if (integer_route && !g.b) integer_route = g.b_zp == 0.0f;  // a packed B was cast without a shift
  if (integer_route) {
    hipLaunchKernelGGL(init_range_kernel, dim3(1), dim3(64), 0, g.s, info.as<int>());
    hipLaunchKernelGGL(scan_int_range_kernel, dim3(grid_for(g.m * g.k)), dim3(256), 0, g.s, g.a, g.m * g.k,
                       info.as<int>());
    if (g.b)
      hipLaunchKernelGGL(scan_int_range_kernel, dim3(grid_for(g.k * g.n)), dim3(256), 0, g.s, g.b, g.k * g.n,
                         info.as<int>() + 4);
    YSCV_HIP_TRY(hipMemcpyAsync(h, info.p, sizeof(h), hipMemcpyDeviceToHost, g.s));
    YSCV_HIP_TRY(hipStreamSynchronize(g.s));
  }
  // shift A into u8 (by 0 or 128) so that its zero point fits as well; shift B into i8 (by 0 or -128)
  int sa = 0, sb = 0;
  if (integer_route) {
    const int zp = (int)g.a_zp;
    auto fits = [&](int sh) { return h[0] + sh >= 0 && h[1] + sh <= 255 && zp + sh >= 0 && zp + sh <= 255; };
    if (h[2] || (g.m * g.k > 0 && !fits(0) && !fits(128))) integer_route = false;
    else sa = fits(0) ? 0 : 128;
  }
  if (integer_route && g.b) {
    if (h[6]) integer_route = false;
    else if (h[4] >= -128 && h[5] <= 127) sb = 0;
    else if (h[4] >= 0 && h[5] <= 255) sb = -128;
    else integer_route = false;
  }
  const int azp = (int)g.a_zp + sa, bzp = (int)g.b_zp + sb;

  if (!integer_route) {
    YSCV_REQUIRE(g.b != nullptr,
                 "operands are not 8-bit integers (or the zero points do not fit); the f32 route needs the unpacked B");
    dim3 grid((unsigned)ceil_div(g.n, (size_t)256), (unsigned)g.m);
    YSCV_REQUIRE(g.m <= 65535, "f32 route: m=%zu exceeds 65535 rows", g.m);
    hipLaunchKernelGGL(f32_fallback_kernel, grid, dim3(256), 0, g.s, g.a, g.b, g.m, g.k, g.n, g.a_zp, g.a_scale,
                       g.b_zp, g.b_scale, g.op == OP_QLINEAR ? 2 : 0, g.y_scale, g.y_zp, g.out);
    YSCV_HIP_TRY(hipGetLastError());
    return YSCV_HIP_OK;
  }

  *took_integer_route = 1;
  DevBuf a8, b8, acc, rs;
  YSCV_TRY(a8.alloc(g.m * g.k));
  YSCV_TRY(acc.alloc(g.m * g.n * sizeof(int32_t)));
  YSCV_TRY(rs.alloc(g.m * sizeof(int32_t)));
  hipLaunchKernelGGL(cast_shift_kernel, dim3(grid_for(g.m * g.k)), dim3(256), 0, g.s, g.a, g.m * g.k, sa,
                     a8.as<uint8_t>());
  TempWeight tmp;
  const yscv_hip_i8_weight *w = g.b_packed;
  if (g.b) {
    YSCV_TRY(b8.alloc(g.k * g.n));
    hipLaunchKernelGGL(cast_shift_kernel, dim3(grid_for(g.k * g.n)), dim3(256), 0, g.s, g.b, g.k * g.n, sb,
                       b8.as<uint8_t>());
    YSCV_TRY(pack_device_i8(b8.as<int8_t>(), g.k, g.n, g.s, &tmp.w));
    w = tmp.w;
  }
  const bool need_rs = bzp != 0;
  if (need_rs)
    hipLaunchKernelGGL(row_sum_u8_kernel, dim3((unsigned)ceil_div(g.m, (size_t)4)), dim3(256), 0, g.s,
                       a8.as<uint8_t>(), g.m, g.k, rs.as<int32_t>());
  I8Epilogue ep{};
  ep.mode = 0;
  YSCV_TRY(launch_i8_gemm(a8.p, 1, azp, w, g.m, acc.p, ep, g.s));
  hipLaunchKernelGGL(mm_post_kernel, dim3(grid_for(g.m * g.n)), dim3(256), 0, g.s, acc.as<int32_t>(),
                     need_rs ? rs.as<int32_t>() : (const int32_t *)nullptr, bzp, (int)g.k * azp, g.m, g.n,
                     g.op == OP_QLINEAR ? 2 : 0, 0.0f, (double)g.a_scale * (double)g.b_scale, g.y_scale, g.y_zp,
                     g.out);
  YSCV_HIP_TRY(hipGetLastError());
  YSCV_HIP_TRY(hipStreamSynchronize(g.s));
  return YSCV_HIP_OK;
}

int32_t run_matmul(const MatmulArgs &g, int32_t *path_out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(g.b || g.b_packed, "neither an unpacked nor a packed B given");
  YSCV_REQUIRE(g.k > 0 && g.n > 0, "bad shape k=%zu n=%zu", g.k, g.n);
  if (g.b_packed)
    YSCV_REQUIRE(g.b_packed->k == g.k && g.b_packed->n == g.n, "prepacked weight shape mismatch: packed %zux%zu, op %zux%zu",
                 g.b_packed->k, g.b_packed->n, g.k, g.n);
  const bool fast = g.a_zp == 0.0f && g.b_zp == 0.0f;
  auto &fast_ctr = g.op == OP_QLINEAR ? g_qlinear_fast : g_mmi_fast;
  auto &fb_ctr = g.op == OP_QLINEAR ? g_qlinear_fallback : g_mmi_fallback;
  int32_t path = fast ? YSCV_HIP_PATH_FAST : YSCV_HIP_PATH_FALLBACK_F32;
  if (g.m > 0) {
    YSCV_REQUIRE(g.a && g.out, "null a / out pointer");
    if (fast) {
      YSCV_TRY(run_fast(g));
    } else {
      int integer_route = 0;
      YSCV_TRY(run_fallback(g, &integer_route));
      if (integer_route) path = YSCV_HIP_PATH_FALLBACK_EXACT;
    }
  }
  (fast ? fast_ctr : fb_ctr).fetch_add(1, std::memory_order_relaxed);
  if (path_out) *path_out = path;
  return YSCV_HIP_OK;
}

}  // namespace

void note_int4_fast() { g_int4_fast.fetch_add(1, std::memory_order_relaxed); }
void note_int4_fallback() { g_int4_fallback.fetch_add(1, std::memory_order_relaxed); }

}  // namespace yscv

using namespace yscv;

extern "C" {

int32_t yscv_hip_quant_runtime_stats(yscv_hip_quant_stats *out) {
  YSCV_REQUIRE(out != nullptr, "null stats pointer");
  out->qlinear_matmul_fast = g_qlinear_fast.load(std::memory_order_relaxed);
  out->qlinear_matmul_fallback = g_qlinear_fallback.load(std::memory_order_relaxed);
  out->matmul_integer_fast = g_mmi_fast.load(std::memory_order_relaxed);
  out->matmul_integer_fallback = g_mmi_fallback.load(std::memory_order_relaxed);
  out->int4_fast = g_int4_fast.load(std::memory_order_relaxed);
  out->int4_fallback = g_int4_fallback.load(std::memory_order_relaxed);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_reset_quant_runtime_stats(void) {
  for (auto *c : {&g_qlinear_fast, &g_qlinear_fallback, &g_mmi_fast, &g_mmi_fallback, &g_int4_fast, &g_int4_fallback})
    c->store(0, std::memory_order_relaxed);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_quant_int8_fast_enabled(void) {
  const char *v = std::getenv("YSCV_QUANT_INT8_FAST");
  return (v != nullptr && v[0] == '0' && v[1] == '\0') ? 0 : 1;
}

int32_t yscv_hip_should_use_prepacked_i8_b(size_t m, size_t k, size_t n) {
  return ((m >= 4 && k >= 4 && n >= 32 && n % 16 == 0) || (m <= 64 && k >= 512 && n >= 1024)) ? 1 : 0;
}

int32_t yscv_hip_should_prepack_i8_b(size_t k, size_t n) {
  return ((k >= 4 && n % 16 == 0) || (k >= 512 && n >= 1024)) ? 1 : 0;
}

int32_t yscv_hip_i8_weight_from_f32(const float *b_dev, size_t k, size_t n, void *stream, yscv_hip_i8_weight **out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(out != nullptr, "null output handle pointer");
  *out = nullptr;
  YSCV_REQUIRE(b_dev != nullptr, "null b");
  YSCV_REQUIRE(k > 0 && n > 0 && k < (1u << 30) && n < (1u << 30), "bad shape k=%zu n=%zu", k, n);
  hipStream_t s = as_stream(stream);
  DevBuf b8;
  YSCV_TRY(b8.alloc(k * n));
  hipLaunchKernelGGL(cast_as_i8_kernel, dim3(grid_for(k * n)), dim3(256), 0, s, b_dev, k * n, 1, b8.as<int8_t>());
  YSCV_TRY(pack_device_i8(b8.as<int8_t>(), k, n, s, out));
  hipError_t e = hipStreamSynchronize(s);
  if (e != hipSuccess) {
    free_weight(*out);
    *out = nullptr;
    return set_error(YSCV_HIP_ERR_DEVICE, "packing B failed: %s", hipGetErrorString(e));
  }
  return YSCV_HIP_OK;
}

int32_t yscv_hip_int4_weight_from_f32(const float *w_dev, size_t d0, size_t d1, int32_t layout, size_t group_size,
                                      void *stream, yscv_hip_int4_weight **out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(out != nullptr, "null output handle pointer");
  *out = nullptr;
  YSCV_REQUIRE(group_size != 0 && (group_size & 1) == 0, "group_size must be even and > 0, got %zu", group_size);
  YSCV_REQUIRE(layout == YSCV_HIP_WEIGHT_KN || layout == YSCV_HIP_WEIGHT_NK, "unknown weight layout %d", layout);
  YSCV_REQUIRE(w_dev != nullptr && d0 > 0 && d1 > 0, "null weight / empty shape");
  const size_t m_w = layout == YSCV_HIP_WEIGHT_KN ? d1 : d0, k = layout == YSCV_HIP_WEIGHT_KN ? d0 : d1;
  if (k % group_size != 0 || k * m_w < 32) return YSCV_HIP_OK;  // the reference skips these weights silently
  if (!(group_size == 32 || group_size == 64 || group_size % 128 == 0))
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "device-side packing needs group size 32, 64 or a multiple of 128, got %zu",
                     group_size);
  hipStream_t s = as_stream(stream);
  DevBuf t, packed, scales;
  const float *src = w_dev;
  if (layout == YSCV_HIP_WEIGHT_KN) {
    YSCV_TRY(t.alloc(d0 * d1 * sizeof(float)));
    dim3 grid((unsigned)ceil_div(d1, (size_t)32), (unsigned)ceil_div(d0, (size_t)32));
    YSCV_REQUIRE(grid.y <= 65535, "weight too tall to transpose in one launch");
    hipLaunchKernelGGL(transpose_f32_kernel, grid, dim3(32, 8), 0, s, w_dev, d0, d1, t.as<float>());
    YSCV_HIP_TRY(hipGetLastError());
    src = t.as<float>();
  }
  YSCV_TRY(packed.alloc(m_w * k / 2));
  YSCV_TRY(scales.alloc(m_w * (k / group_size) * sizeof(float)));
  YSCV_TRY(launch_pack_int4_symmetric(src, m_w, k, group_size, packed.as<uint8_t>(), scales.as<float>(), s));
  YSCV_HIP_TRY(hipStreamSynchronize(s));
  return int4_create_from_device(packed.as<uint8_t>(), scales.p, YSCV_HIP_F32, YSCV_HIP_NIBBLE_SIGNED, m_w, k, group_size, out);
}

int32_t yscv_hip_kv_i8_quantize_rows(const float *src_dev, size_t rows, size_t kv_dim, int8_t *data_dev, float *scales_dev,
                                     void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  if (rows == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(src_dev && data_dev && scales_dev && kv_dim > 0, "null pointer / empty row");
  return launch_kv_i8_quantize_rows(src_dev, rows, kv_dim, data_dev, scales_dev, as_stream(stream));
}

int32_t yscv_hip_kv_i8_dequantize_rows(const int8_t *data_dev, const float *scales_dev, size_t rows, size_t kv_dim,
                                       float *out_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  if (rows == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(data_dev && scales_dev && out_dev && kv_dim > 0, "null pointer / empty row");
  return launch_kv_i8_dequantize_rows(data_dev, scales_dev, rows, kv_dim, out_dev, as_stream(stream));
}

int32_t yscv_hip_exec_matmul_integer(const float *a_dev, const float *b_dev, const yscv_hip_i8_weight *b_packed,
                                     float a_zp, float b_zp, size_t m, size_t k, size_t n, float *out_dev,
                                     int32_t *path_out, void *stream) {
  MatmulArgs g{OP_MATMUL_INTEGER, a_dev, b_dev, b_packed, m, k, n, 1.0f, a_zp, 1.0f, b_zp, 1.0f, 0.0f, out_dev,
               as_stream(stream)};
  return run_matmul(g, path_out);
}

int32_t yscv_hip_exec_qlinear_matmul(const float *a_dev, float a_scale, float a_zp, const float *b_dev,
                                     const yscv_hip_i8_weight *b_packed, float b_scale, float b_zp, float y_scale,
                                     float y_zp, size_t m, size_t k, size_t n, float *out_dev, int32_t *path_out,
                                     void *stream) {
  MatmulArgs g{OP_QLINEAR, a_dev, b_dev, b_packed, m, k, n, a_scale, a_zp, b_scale, b_zp, y_scale, y_zp, out_dev,
               as_stream(stream)};
  return run_matmul(g, path_out);
}

int32_t yscv_hip_exec_qdq_matmul(const float *x_dev, size_t m, float a_scale, const yscv_hip_i8_weight *b, float b_scale,
                                 float y_scale, float y_zp, float *out_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(b != nullptr, "null int8 weight handle");
  if (m == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(x_dev && out_dev, "null x / out pointer");
  hipStream_t s = as_stream(stream);
  // QuantizeLinear (zero point 0) into a scratch int8 matrix, then the GEMM whose epilogue requantises with the
  // QLinearMatMul fast-path expression and dequantises again
  int8_t *a8 = nullptr;
  YSCV_HIP_TRY(hipMallocAsync(reinterpret_cast<void **>(&a8), m * b->k, s));
  int32_t st = launch_quantize_linear_i8(x_dev, m * b->k, a_scale, 0.0f, a8, s);
  if (st == YSCV_HIP_OK) {
    I8Epilogue ep{};
    ep.mode = 2;
    ep.composite = (a_scale * b_scale) / y_scale;
    ep.y_zp = y_zp;
    ep.round_mode = YSCV_HIP_ROUND_HALF_AWAY;
    ep.lo = -128;
    ep.hi = 127;
    ep.dq_scale = y_scale;
    st = launch_i8_gemm(a8, 0, 0, b, m, out_dev, ep, s);
  }
  const hipError_t fe = hipFreeAsync(a8, s);
  YSCV_TRY(st);
  YSCV_HIP_TRY(fe);
  g_qlinear_fast.fetch_add(1, std::memory_order_relaxed);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_exec_dql_matmul_integer(const float *x_dev, size_t m, const yscv_hip_i8_weight *b, float *out_dev,
                                         float *y_scale_dev, float *y_zp_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(b != nullptr, "null int8 weight handle");
  YSCV_REQUIRE(y_scale_dev && y_zp_dev, "null scale / zero-point pointer");
  if (m == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(x_dev && out_dev, "null x / out pointer");
  hipStream_t s = as_stream(stream);
  const size_t len = m * b->k;
  // uint8 A and {scale, zero point} in one stream-ordered scratch block; nothing returns to the host
  uint8_t *scratch = nullptr;
  const size_t a_bytes = round_up(len, 256);
  YSCV_HIP_TRY(hipMallocAsync(reinterpret_cast<void **>(&scratch), a_bytes + 256, s));
  float *scale_zp = reinterpret_cast<float *>(scratch + a_bytes);
  int32_t st = launch_dynamic_quantize_linear(x_dev, len, scratch, scale_zp, s);
  if (st == YSCV_HIP_OK) {
    I8Epilogue ep{};
    ep.mode = 3;                   // f32(acc): MatMulInteger's output carrier (linear.rs:693-697)
    ep.a_zp_dev = scale_zp + 1;    // the zero point stays on the device: the GEMM folds (128 - zp) * colsum(b) itself
    st = launch_i8_gemm(scratch, 1, 0, b, m, out_dev, ep, s);
  }
  hipError_t e1 = hipSuccess, e2 = hipSuccess;
  if (st == YSCV_HIP_OK) {
    e1 = hipMemcpyAsync(y_scale_dev, scale_zp, sizeof(float), hipMemcpyDeviceToDevice, s);
    e2 = hipMemcpyAsync(y_zp_dev, scale_zp + 1, sizeof(float), hipMemcpyDeviceToDevice, s);
  }
  const hipError_t fe = hipFreeAsync(scratch, s);
  YSCV_TRY(st);
  YSCV_HIP_TRY(e1);
  YSCV_HIP_TRY(e2);
  YSCV_HIP_TRY(fe);
  g_mmi_fallback.fetch_add(1, std::memory_order_relaxed);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_exec_matmul_nbits(const void *a_dev, int32_t a_dtype, size_t m, const yscv_hip_int4_weight *b,
                                   const float *bias_dev, int64_t attr_k, int64_t attr_n, int64_t attr_bits,
                                   int64_t attr_block_size, void *y_dev, int32_t y_dtype, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(b != nullptr, "MatMulNBits: null weight handle");
  if (attr_bits != 4) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "MatMulNBits: bits=%lld, only 4 is supported", (long long)attr_bits);
  size_t n = 0, k = 0, g = 0;
  YSCV_TRY(yscv_hip_int4_weight_dims(b, &n, &k, &g, nullptr));
  YSCV_REQUIRE(attr_k > 0 && attr_n > 0 && (size_t)attr_k == k && (size_t)attr_n == n,
               "MatMulNBits: attributes K=%lld N=%lld but the packed weight is [N=%zu][K=%zu]", (long long)attr_k,
               (long long)attr_n, n, k);
  YSCV_REQUIRE(attr_block_size > 0 && (size_t)attr_block_size == g,
               "MatMulNBits: block_size=%lld but the packed weight has group size %zu", (long long)attr_block_size, g);
  if (m == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(a_dev && y_dev, "MatMulNBits: null A / Y pointer");
  hipStream_t s = as_stream(stream);
  if (bias_dev == nullptr) return yscv_hip_int4_matmul(b, a_dev, a_dtype, y_dev, y_dtype, m, stream);
  // with a bias the product is kept in f32 until the bias is added, then rounded once to the output type
  float *acc = nullptr;
  const bool in_place = y_dtype == YSCV_HIP_F32;
  if (in_place) acc = static_cast<float *>(y_dev);
  else YSCV_HIP_TRY(hipMallocAsync(reinterpret_cast<void **>(&acc), m * n * sizeof(float), s));
  int32_t st = yscv_hip_int4_matmul(b, a_dev, a_dtype, acc, YSCV_HIP_F32, m, stream);
  if (st == YSCV_HIP_OK) {
    hipLaunchKernelGGL(bias_cast_kernel, dim3(grid_for(m * n)), dim3(256), 0, s, acc, m, n, bias_dev, y_dev, y_dtype);
    if (hipGetLastError() != hipSuccess) st = set_error(YSCV_HIP_ERR_DEVICE, "MatMulNBits: bias kernel launch failed");
  }
  if (!in_place) {
    const hipError_t fe = hipFreeAsync(acc, s);
    YSCV_TRY(st);
    YSCV_HIP_TRY(fe);
  }
  return st;
}

int32_t yscv_hip_exec_gemm_int4(const float *a_dev, size_t m, const yscv_hip_int4_weight *b, const float *c_dev,
                                size_t c_rows, float alpha, float beta, float *y_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(b != nullptr, "Gemm: null weight handle");
  size_t n = 0, k = 0, g = 0;
  YSCV_TRY(yscv_hip_int4_weight_dims(b, &n, &k, &g, nullptr));
  YSCV_REQUIRE(c_dev == nullptr ? c_rows == 0 : (c_rows == 1 || c_rows == m),
               "Gemm: C must be absent, one row of N values or [M][N] (c_rows = %zu, m = %zu)", c_rows, m);
  if (m == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(a_dev && y_dev, "Gemm: null A / Y pointer");
  YSCV_TRY(yscv_hip_int4_matmul(b, a_dev, YSCV_HIP_F32, y_dev, YSCV_HIP_F32, m, stream));
  // exec_gemm scales only when |alpha - 1| (|beta - 1|) exceeds f32::EPSILON (linear.rs:54,58)
  const int use_alpha = fabsf(alpha - 1.0f) > 1.1920929e-7f, use_beta = fabsf(beta - 1.0f) > 1.1920929e-7f;
  if (!use_alpha && c_dev == nullptr) return YSCV_HIP_OK;
  hipLaunchKernelGGL(gemm_post_kernel, dim3(grid_for(m * n)), dim3(256), 0, as_stream(stream), y_dev, m, n, c_dev, c_rows,
                     alpha, use_alpha, beta, use_beta);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t yscv_hip_exec_quantize_linear(const float *x_dev, size_t len, float scale, float zero_point, float *out_dev,
                                      void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  if (len == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(x_dev && out_dev, "null pointer");
  hipLaunchKernelGGL(quantize_linear_f32_kernel, dim3(grid_for(len)), dim3(256), 0, as_stream(stream), x_dev, len,
                     scale, zero_point, out_dev);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t yscv_hip_exec_dequantize_linear(const float *q_dev, size_t outer, size_t chan, size_t inner,
                                        const float *scales_dev, const float *zps_dev, size_t n_scales,
                                        float *out_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(scales_dev != nullptr, "null scale pointer");
  YSCV_REQUIRE(n_scales == 1 || n_scales == chan, "DequantizeLinear: scale len=%zu but axis dim=%zu", n_scales, chan);
  const size_t len = outer * chan * inner;
  if (len == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(q_dev && out_dev, "null pointer");
  hipLaunchKernelGGL(dequantize_linear_f32_kernel, dim3(grid_for(len)), dim3(256), 0, as_stream(stream), q_dev, len,
                     n_scales == 1 ? (size_t)1 : chan, inner, scales_dev, zps_dev, out_dev);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t yscv_hip_exec_dynamic_quantize_linear(const float *x_dev, size_t len, float *y_dev, float *y_scale_dev,
                                              float *y_zp_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(y_scale_dev && y_zp_dev, "null scale / zero-point pointer");
  YSCV_REQUIRE(len == 0 || (x_dev && y_dev), "null pointer");
  hipStream_t s = as_stream(stream);
  StreamBuf q, sz;  // released in stream order: the call does not wait for the device
  YSCV_TRY(q.alloc(len, s));
  YSCV_TRY(sz.alloc(2 * sizeof(float), s));
  YSCV_TRY(launch_dynamic_quantize_linear(x_dev, len, q.as<uint8_t>(), sz.as<float>(), s));
  hipLaunchKernelGGL(u8_to_f32_kernel, dim3(grid_for(len)), dim3(256), 0, s, q.as<uint8_t>(), len, sz.as<float>(),
                     y_dev, y_scale_dev, y_zp_dev);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

}  // extern "C"
