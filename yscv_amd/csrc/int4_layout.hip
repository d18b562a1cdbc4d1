// Load-time and per-call layout kernels of the int4 path: weight re-tiling, scale /
// zero-point re-tiling, activation preparation, and the GPU forms of
// pack_int4_symmetric_per_group and dequantize_int4_to_f32.
#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

// ---- weight re-tiling ----------------------------------------------------------------
// One thread per output word.  Source: caller's [n][k/2] bytes (element 2i in the low
// nibble, int4_matmul.rs:12-14).  See int4_common.hpp for the destination layout.
__global__ void int4_retile_kernel(const uint8_t *__restrict__ raw, int is_signed, size_t n, size_t k,
                                   size_t nt_count, size_t kt_count, uint32_t *__restrict__ tiles) {
  size_t total = nt_count * kt_count * 256;  // words
  for (size_t w = blockIdx.x * (size_t)blockDim.x + threadIdx.x; w < total;
       w += (size_t)gridDim.x * blockDim.x) {
    size_t j = w & 3;
    size_t lane = (w >> 2) & 63;
    size_t tile = w >> 8;
    size_t kt = tile % kt_count, nt = tile / kt_count;
    size_t r = lane & 15, c = lane >> 4;
    size_t row = nt * 16 + r;
    size_t k0 = kt * 128 + j * 32 + c * 8;
    uint32_t e[8];
    for (int i = 0; i < 8; i++) {
      size_t kk = k0 + i;
      uint32_t q = 8;  // padding: value 0 under the implicit zero point 8
      if (row < n && kk < k) {
        uint8_t byte = raw[row * (k / 2) + kk / 2];
        q = (kk & 1) ? (byte >> 4) : (byte & 15);
        if (is_signed) q ^= 8;  // two's complement nibble s -> s + 8
      }
      e[i] = q;
    }
    uint32_t word = e[0] | (e[2] << 4) | (e[4] << 8) | (e[6] << 12) | (e[1] << 16) | (e[3] << 20) |
                    (e[5] << 24) | (e[7] << 28);
    tiles[w] = word;
  }
}

int32_t launch_int4_retile(const uint8_t *raw_in, int nibble_format, size_t n, size_t k, size_t nt,
                           size_t kt, uint8_t *tiles, hipStream_t s) {
  size_t total = nt * kt * 256;
  int blocks = (int)((total + 255) / 256 < 65535 * 4 ? (total + 255) / 256 : 65535 * 4);
  hipLaunchKernelGGL(int4_retile_kernel, dim3(blocks), dim3(256), 0, s, raw_in,
                     nibble_format == YSCV_HIP_NIBBLE_SIGNED ? 1 : 0, n, k, nt, kt,
                     reinterpret_cast<uint32_t *>(tiles));
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

template <typename T>
__global__ void int4_retile_scales_kernel(const T *__restrict__ scales, const uint8_t *__restrict__ zps,
                                          size_t n, size_t groups, size_t g, int spt, size_t nt_count,
                                          size_t chunks, T *__restrict__ tscales,
                                          uint8_t *__restrict__ tzps) {
  size_t total = nt_count * chunks * 16 * (size_t)spt;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    size_t sj = idx % spt;
    size_t r = (idx / spt) % 16;
    size_t ch = (idx / spt / 16) % chunks;
    size_t nt = idx / spt / 16 / chunks;
    size_t row = nt * 16 + r;
    size_t grp = ch * spt + sj;  // spt > 1: chunk = 128-k tile; spt == 1: chunk = group
    T sv = (T)0;
    uint8_t zv = 8;
    if (row < n && grp < groups) {
      sv = scales[row * groups + grp];
      if (zps) zv = zps[row * groups + grp];
    }
    tscales[idx] = sv;
    if (tzps) tzps[idx] = zv;
  }
  (void)g;
}

int32_t launch_int4_retile_scales(const void *scales_in, int scale_dtype, const uint8_t *zps_in,
                                  size_t n, size_t k, size_t g, int gm, size_t nt, size_t chunks,
                                  void *tscales, uint8_t *tzps, hipStream_t s) {
  int spt = scales_per_chunk(gm);
  size_t groups = k / g;
  size_t total = nt * chunks * 16 * (size_t)spt;
  int blocks = (int)((total + 255) / 256 < 262140 ? (total + 255) / 256 : 262140);
  if (blocks < 1) blocks = 1;
  if (scale_dtype == YSCV_HIP_F32) {
    hipLaunchKernelGGL(int4_retile_scales_kernel<float>, dim3(blocks), dim3(256), 0, s,
                       static_cast<const float *>(scales_in), zps_in, n, groups, g, spt, nt, chunks,
                       static_cast<float *>(tscales), tzps);
  } else {
    hipLaunchKernelGGL(int4_retile_scales_kernel<_Float16>, dim3(blocks), dim3(256), 0, s,
                       static_cast<const _Float16 *>(scales_in), zps_in, n, groups, g, spt, nt,
                       chunks, static_cast<_Float16 *>(tscales), tzps);
  }
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

__global__ void unpack_zps_kernel(const uint8_t *__restrict__ packed, size_t n, size_t groups,
                                  uint8_t *__restrict__ out) {
  size_t row_bytes = (groups + 1) / 2;
  size_t total = n * groups;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    size_t row = idx / groups, grp = idx % groups;
    uint8_t b = packed[row * row_bytes + grp / 2];
    out[idx] = (grp & 1) ? (b >> 4) : (b & 15);
  }
}

int32_t launch_unpack_zps(const uint8_t *zps_packed, size_t n, size_t groups, uint8_t *out,
                          hipStream_t s) {
  size_t total = n * groups;
  int blocks = (int)((total + 255) / 256 < 262140 ? (total + 255) / 256 : 262140);
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(unpack_zps_kernel, dim3(blocks), dim3(256), 0, s, zps_packed, n, groups, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

__global__ void xor88_kernel(uint8_t *buf, size_t bytes) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < bytes;
       i += (size_t)gridDim.x * blockDim.x)
    buf[i] ^= 0x88;
}
int32_t launch_xor88(uint8_t *buf, size_t bytes, hipStream_t s) {
  int blocks = (int)((bytes + 255) / 256 < 262140 ? (bytes + 255) / 256 : 262140);
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(xor88_kernel, dim3(blocks), dim3(256), 0, s, buf, bytes);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// ---- activation preparation -------------------------------------------------------------
// One workgroup per activation row.  The row is divided by a power of two so that its
// largest magnitude lands in [2^14, 2^15) -- the top of the fp16 range -- then written as
// fp16 `hi` and, for f32 input, a second fp16 `lo` = x' - hi.  hi + lo carries ~22
// significant bits, f16/bf16 inputs are represented exactly by hi alone.  The power of
// two is returned so the GEMV/GEMM epilogue can multiply it back (exactly).
// load 8 consecutive activations starting at element `idx` (idx % 8 == 0 when VEC)
template <bool VEC>
__device__ __forceinline__ void load8(const void *x, size_t idx, int dtype, size_t limit, float v[8]) {
  if constexpr (VEC) {
    if (dtype == YSCV_HIP_F32) {
      const float4_t *p = reinterpret_cast<const float4_t *>(reinterpret_cast<const float *>(x) + idx);
      float4_t a = p[0], b = p[1];
      v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3];
      v[4] = b[0]; v[5] = b[1]; v[6] = b[2]; v[7] = b[3];
    } else if (dtype == YSCV_HIP_F16) {
      half8_t h = *reinterpret_cast<const half8_t *>(reinterpret_cast<const _Float16 *>(x) + idx);
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = (float)h[i];
    } else {
      uint4_t u = *reinterpret_cast<const uint4_t *>(reinterpret_cast<const uint16_t *>(x) + idx);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        v[2 * i] = __uint_as_float(u[i] << 16);
        v[2 * i + 1] = __uint_as_float(u[i] & 0xFFFF0000u);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = (idx + i < limit) ? load_in(x, idx + i, dtype) : 0.0f;
  }
}

template <bool VEC>
__global__ void __launch_bounds__(1024) x_prep_kernel(const void *__restrict__ x, int x_dtype, size_t k,
                                                      size_t k_pad, int split, _Float16 *__restrict__ xh,
                                                      _Float16 *__restrict__ xl,
                                                      float *__restrict__ row_scale) {
  __shared__ float red[16];
  const size_t row = blockIdx.x;
  const size_t base = row * k;
  const size_t chunks = k_pad / 8;
  // pass 1: abs-max of the row.  The first sweep's values stay in registers for pass 2 (a row of up to 8 blockDim
  // elements is read from memory once); longer rows re-read the rest.
  float amax = 0.0f;
  float v0[8];
  const size_t ch0 = threadIdx.x;
  const bool have0 = ch0 < chunks && ch0 * 8 < k;
  if (have0) {
    load8<VEC>(x, base + ch0 * 8, x_dtype, base + k, v0);
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) v0[i] = 0.0f;
  }
#pragma unroll
  for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v0[i]));  // NaN is ignored here, kept in the values
  for (size_t ch = ch0 + blockDim.x; ch < chunks; ch += blockDim.x) {
    if (ch * 8 < k) {
      float v[8];
      load8<VEC>(x, base + ch * 8, x_dtype, base + k, v);
#pragma unroll
      for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v[i]));
    }
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = 0.0f;
  for (unsigned w = 0; w < (blockDim.x >> 6); w++) amax = fmaxf(amax, red[w]);
  int e = 14;
  if (amax > 0.0f && amax < 3.0e38f) {
    (void)frexpf(amax, &e);  // amax = f * 2^e, f in [0.5, 1)
    e -= 1;                  // amax in [2^e, 2^(e+1))
  }  // else: all-zero or non-finite row, leave the values alone
  int shift = 14 - e;
  shift = shift > 100 ? 100 : (shift < -100 ? -100 : shift);
  const float up = ldexpf(1.0f, shift);
  if (threadIdx.x == 0) row_scale[row] = ldexpf(1.0f, -shift);
  const size_t obase = row * k_pad;
  for (size_t ch = ch0; ch < chunks; ch += blockDim.x) {
    float v[8];
    if (ch == ch0) {
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = v0[i];
    } else if (ch * 8 < k) {
      load8<VEC>(x, base + ch * 8, x_dtype, base + k, v);
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = 0.0f;
    }
    half8_t h, l;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float s = v[i] * up;
      h[i] = (_Float16)s;
      l[i] = (_Float16)(s - (float)h[i]);
    }
    *reinterpret_cast<half8_t *>(xh + obase + ch * 8) = h;
    if (split == 2) *reinterpret_cast<half8_t *>(xl + obase + ch * 8) = l;
  }
}

// Rows of at most 4096 padded elements, aligned: one wavefront per row, eight 8-element chunks per lane held in
// registers from the abs-max sweep to the conversion; no LDS, no barrier, and every load is unconditional (lanes
// past the end of the row re-read its last chunk and drop it), so a row costs one memory round trip.
template <int DT>
__global__ void __launch_bounds__(256) x_prep_wave_kernel(const void *__restrict__ x, size_t m, size_t k, size_t k_pad,
                                                          int split, _Float16 *__restrict__ xh,
                                                          _Float16 *__restrict__ xl, float *__restrict__ row_scale) {
  const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= m) return;
  const int lane = threadIdx.x & 63;
  const size_t base = row * k;
  const int chunks = (int)(k_pad / 8), data_chunks = (int)(k / 8);  // k % 8 == 0 on this path
  float v[8][8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int ch = lane + 64 * i;
    load8<true>(x, base + (size_t)min(ch, data_chunks - 1) * 8, DT, base + k, v[i]);
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const bool have = lane + 64 * i < data_chunks;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      v[i][e] = have ? v[i][e] : 0.0f;
      amax = fmaxf(amax, fabsf(v[i][e]));  // NaN is ignored here, kept in the values
    }
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  int e2 = 14;
  if (amax > 0.0f && amax < 3.0e38f) {
    (void)frexpf(amax, &e2);
    e2 -= 1;
  }
  int shift = 14 - e2;
  shift = shift > 100 ? 100 : (shift < -100 ? -100 : shift);
  const float up = ldexpf(1.0f, shift);
  if (lane == 0) row_scale[row] = ldexpf(1.0f, -shift);
  const size_t obase = row * k_pad;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int ch = lane + 64 * i;
    if (ch < chunks) {
      half8_t h, l;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float sv = v[i][e] * up;
        h[e] = (_Float16)sv;
        l[e] = (_Float16)(sv - (float)h[e]);
      }
      *reinterpret_cast<half8_t *>(xh + obase + (size_t)ch * 8) = h;
      if (split == 2) *reinterpret_cast<half8_t *>(xl + obase + (size_t)ch * 8) = l;
    }
  }
}

int32_t launch_x_prep(const void *x, int x_dtype, size_t m, size_t k, size_t k_pad, int split,
                      _Float16 *xh, _Float16 *xl, float *row_scale, hipStream_t s) {
  const size_t esz = x_dtype == YSCV_HIP_F32 ? 4 : 2;
  const bool vec = (k % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) && ((k * esz) % 16 == 0);
  if (vec && k >= 8 && k_pad <= 4096) {
    const dim3 grid((unsigned)ceil_div(m, (size_t)4));
    if (x_dtype == YSCV_HIP_F32)
      hipLaunchKernelGGL(x_prep_wave_kernel<YSCV_HIP_F32>, grid, dim3(256), 0, s, x, m, k, k_pad, split, xh, xl, row_scale);
    else if (x_dtype == YSCV_HIP_F16)
      hipLaunchKernelGGL(x_prep_wave_kernel<YSCV_HIP_F16>, grid, dim3(256), 0, s, x, m, k, k_pad, split, xh, xl, row_scale);
    else
      hipLaunchKernelGGL(x_prep_wave_kernel<YSCV_HIP_BF16>, grid, dim3(256), 0, s, x, m, k, k_pad, split, xh, xl, row_scale);
    YSCV_HIP_TRY(hipGetLastError());
    return YSCV_HIP_OK;
  }
  size_t chunks = k_pad / 8;
  unsigned threads = chunks >= 1024 ? 1024 : (unsigned)round_up(chunks < 64 ? 64 : chunks, 64);
  if (vec)
    hipLaunchKernelGGL(x_prep_kernel<true>, dim3((unsigned)m), dim3(threads), 0, s, x, x_dtype, k, k_pad, split,
                       xh, xl, row_scale);
  else
    hipLaunchKernelGGL(x_prep_kernel<false>, dim3((unsigned)m), dim3(threads), 0, s, x, x_dtype, k, k_pad,
                       split, xh, xl, row_scale);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// ---- pack_int4_symmetric_per_group (int4_matmul.rs:611-646) ---------------------------------
// One wavefront per (row, group): abs-max, scale = absmax / 7 (1.0 when absmax <= EPSILON),
// q = clamp(round_ties_even(w * (1/scale)), -8, 7), low nibble = even element.
__global__ void __launch_bounds__(256) pack_int4_kernel(const float *__restrict__ w, size_t rows,
                                                        size_t k, size_t g, uint8_t *__restrict__ packed,
                                                        float *__restrict__ scales) {
  size_t groups = k / g;
  size_t wave = (blockIdx.x * (size_t)blockDim.x + threadIdx.x) >> 6;
  int lane = threadIdx.x & 63;
  size_t total = rows * groups;
  size_t nwaves = ((size_t)gridDim.x * blockDim.x) >> 6;
  for (size_t item = wave; item < total; item += nwaves) {
    size_t row = item / groups, grp = item % groups;
    const float *src = w + row * k + grp * g;
    float amax = 0.0f;
    for (size_t i = lane; i < g; i += 64) amax = fmaxf(amax, fabsf(src[i]));
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    float scale = (amax <= 1.1920929e-7f) ? 1.0f : __fdiv_rn(amax, 7.0f);
    float inv = __fdiv_rn(1.0f, scale);
    if (lane == 0) scales[item] = scale;
    for (size_t b = lane; b < g / 2; b += 64) {
      float v0 = rintf(__fmul_rn(src[2 * b], inv));
      float v1 = rintf(__fmul_rn(src[2 * b + 1], inv));
      // clamp keeps NaN and `as i8` maps it to 0 (Rust semantics)
      int q0 = (v0 != v0) ? 0 : (int)fminf(fmaxf(v0, -8.0f), 7.0f);
      int q1 = (v1 != v1) ? 0 : (int)fminf(fmaxf(v1, -8.0f), 7.0f);
      packed[row * (k / 2) + grp * (g / 2) + b] = (uint8_t)((q0 & 15) | ((q1 & 15) << 4));
    }
  }
}

int32_t launch_pack_int4_symmetric(const float *w, size_t m_w, size_t k, size_t g, uint8_t *packed,
                                   float *scales, hipStream_t s) {
  size_t items = m_w * (k / g);
  size_t blocks = (items + 3) / 4;
  if (blocks > 65535 * 8) blocks = 65535 * 8;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(pack_int4_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w, m_w, k, g, packed,
                     scales);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// ---- dequantize_int4_to_f32 (ops/quantize.rs:215-222) ----------------------------------------
__global__ void dequant_int4_kernel(const uint8_t *__restrict__ packed, size_t n_bytes, float scale,
                                    float zp, float *__restrict__ out) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n_bytes;
       i += (size_t)gridDim.x * blockDim.x) {
    int b = packed[i];
    int lo = ((b & 15) ^ 8) - 8, hi = ((b >> 4) ^ 8) - 8;
    out[2 * i] = __fmul_rn(__fsub_rn((float)lo, zp), scale);
    out[2 * i + 1] = __fmul_rn(__fsub_rn((float)hi, zp), scale);
  }
}

int32_t launch_dequantize_int4(const uint8_t *packed, size_t n_bytes, float scale, int zp, float *out,
                               hipStream_t s) {
  size_t blocks = (n_bytes + 255) / 256;
  if (blocks > 262140) blocks = 262140;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(dequant_int4_kernel, dim3((unsigned)blocks), dim3(256), 0, s, packed, n_bytes,
                     scale, (float)zp, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

}  // namespace yscv
