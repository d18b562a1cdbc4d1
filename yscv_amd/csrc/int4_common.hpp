// Device-side pieces shared by the int4 kernels: the tiled weight layout, the
// nibble -> fp16 decode and the vector types the gfx950 MFMA builtins take.
//
// Tiled layout of a packed-int4 weight W[n][k] (n = output row, k = input channel)
// ---------------------------------------------------------------------------------
// The weight is cut into tiles of 16 rows x 128 k.  Tile (nt, kt) is one contiguous
// 1 KiB block at ((nt * KT + kt) * 1024) bytes; inside it lane L = 16*c + r of a
// wavefront owns 16 bytes = four 32-bit words j = 0..3, and word j holds the eight
// weights W[16*nt + r][128*kt + 32*j + 8*c + 0..7].  That is exactly the B operand of
// v_mfma_f32_16x16x32_f16 for the k-block [128*kt + 32*j, +32): one 128-bit coalesced
// load per lane feeds four MFMAs, and each MFMA covers one quantisation group when
// group_size == 32.
// Nibbles are stored unsigned (q in [0,15], value q - zp) and permuted inside the
// word: bits [4i,4i+4) for i = 0..3 hold elements 0,2,4,6 and for i = 4..7 elements
// 1,3,5,7, so that masking with 0x000F000F yields two consecutive k in one register.
// Rows >= n and k >= k are padded with nibble 8 and scale 0.
//
// Scales (and zero points, one byte each) are re-tiled as [nt][chunk][16 rows][SPT]:
// for group_size <= 128 a chunk is one 128-k tile holding SPT = 128/group_size
// values per row; for larger groups a chunk is one group (SPT = 1).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/yscv_hip.h"

namespace yscv {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
typedef int int16_t_v __attribute__((ext_vector_type(16)));

constexpr int kTileRows = 16;
constexpr int kTileK = 128;
constexpr int kTileBytes = 1024;

// group mode of a tiled weight
enum : int { GM32 = 0, GM64 = 1, GM128 = 2 };

__host__ __device__ inline int scales_per_chunk(int gm) { return gm == GM32 ? 4 : (gm == GM64 ? 2 : 1); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global load (s_waitcnt vmcnt(0)), which would drain the software-pipelined weight loads of the
// streaming kernels at every tile; the kernels here exchange data through LDS alone.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

union U32H2 {
  uint32_t u;
  half2_t h;
};

// Decode one tiled word (8 weights) to fp16 (q - zp), in k order.
// c1 = -(1024 + zp), c2 = -(64 + zp), both splat.  Every step is exact in fp16:
// 0x6400 | q is 1024 + q, 0x6400 | (q << 4) is 1024 + 16 q.
__device__ __forceinline__ half8_t decode8(uint32_t s, half2_t c1, half2_t c2) {
  const uint32_t magic = 0x64006400u;
  U32H2 r0, r1, r2, r3;
  r0.u = (s & 0x000F000Fu) | magic;
  r1.u = (s & 0x00F000F0u) | magic;
  uint32_t s2 = s >> 8;
  r2.u = (s2 & 0x000F000Fu) | magic;
  r3.u = (s2 & 0x00F000F0u) | magic;
  const half2_t sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  half2_t h0 = r0.h + c1;
  half2_t h1 = r1.h * sixteenth + c2;
  half2_t h2 = r2.h + c1;
  half2_t h3 = r3.h * sixteenth + c2;
  half8_t out;
  out[0] = h0[0];
  out[1] = h0[1];
  out[2] = h1[0];
  out[3] = h1[1];
  out[4] = h2[0];
  out[5] = h2[1];
  out[6] = h3[0];
  out[7] = h3[1];
  return out;
}

// Constants of the nibble -> fp16 decode, held in registers whose contents the compiler cannot see.  Given literal
// constants it emits v_and_b32 + v_or_b32 per pair of nibbles (a VOP3 encoding cannot hold a literal); with a mask in
// an SGPR and the magic in a VGPR it selects one v_and_or_b32.  The empty asm statements emit no instruction, so
// every real instruction stays visible to the compiler's MFMA hazard handling.
struct NibbleConsts {
  uint32_t lo, hi, magic;  // 0x000F000F, 0x00F000F0, 0x64006400
  __device__ __forceinline__ void init() {
    lo = 0x000F000Fu;
    hi = 0x00F000F0u;
    magic = 0x64006400u;
    asm volatile("" : "+s"(lo), "+s"(hi), "+v"(magic));
  }
};

// raw fp16 forms of the 8 weights of one word: {1024+q0, 1024+q1, 1024+16 q2, 1024+16 q3, ...}
__device__ __forceinline__ half8_t extract8(uint32_t s, const NibbleConsts &nc) {
  U32H2 r0, r1, r2, r3;
  const uint32_t s2 = s >> 8;
  r0.u = (s & nc.lo) | nc.magic;
  r1.u = (s & nc.hi) | nc.magic;
  r2.u = (s2 & nc.lo) | nc.magic;
  r3.u = (s2 & nc.hi) | nc.magic;
  half8_t out;
  out[0] = r0.h[0];
  out[1] = r0.h[1];
  out[2] = r1.h[0];
  out[3] = r1.h[1];
  out[4] = r2.h[0];
  out[5] = r2.h[1];
  out[6] = r3.h[0];
  out[7] = r3.h[1];
  return out;
}

// exact (q - zp) in fp16: c1 = -(1024 + zp), c2 = -(64 + zp)
__device__ __forceinline__ half8_t decode8_exact(uint32_t s, const NibbleConsts &nc, half2_t c1, half2_t c2) {
  U32H2 r0, r1, r2, r3;
  const uint32_t s2 = s >> 8;
  r0.u = (s & nc.lo) | nc.magic;
  r1.u = (s & nc.hi) | nc.magic;
  r2.u = (s2 & nc.lo) | nc.magic;
  r3.u = (s2 & nc.hi) | nc.magic;
  const half2_t sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const half2_t h0 = r0.h + c1;
  const half2_t h1 = r1.h * sixteenth + c2;
  const half2_t h2 = r2.h + c1;
  const half2_t h3 = r3.h * sixteenth + c2;
  half8_t out;
  out[0] = h0[0];
  out[1] = h0[1];
  out[2] = h1[0];
  out[3] = h1[1];
  out[4] = h2[0];
  out[5] = h2[1];
  out[6] = h3[0];
  out[7] = h3[1];
  return out;
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
// round to nearest even, the rule of the reference's f32 -> bf16 narrowing
// (crates/yscv-tensor/src/tensor.rs:764-769)
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t bits = __float_as_uint(f);
  uint32_t bias = 0x7FFFu + ((bits >> 16) & 1u);
  return (uint16_t)((bits + bias) >> 16);
}

// store one result element as f32 / f16 / bf16
__device__ __forceinline__ void store_out(void *y, size_t idx, float v, int dtype) {
  if (dtype == YSCV_HIP_F32) {
    reinterpret_cast<float *>(y)[idx] = v;
  } else if (dtype == YSCV_HIP_F16) {
    reinterpret_cast<_Float16 *>(y)[idx] = (_Float16)v;
  } else {
    reinterpret_cast<uint16_t *>(y)[idx] = float_to_bf16_bits(v);
  }
}

__device__ __forceinline__ float load_in(const void *x, size_t idx, int dtype) {
  if (dtype == YSCV_HIP_F32) return reinterpret_cast<const float *>(x)[idx];
  if (dtype == YSCV_HIP_F16) return (float)reinterpret_cast<const _Float16 *>(x)[idx];
  return bf16_bits_to_float(reinterpret_cast<const uint16_t *>(x)[idx]);
}

// Cross-lane moves without LDS: __shfl_* compiles to ds_bpermute_b32, about a hundred cycles each when one depends
// on the other, and a layer has some ninety of them on its critical path.  Within a row of 16 lanes DPP does the
// same in one vector instruction; v_permlane16_swap / v_permlane32_swap exchange rows and halves of the wave.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E;         // quad_perm [1,0,3,2], [2,3,0,1]
constexpr int DPP_NEXT1 = 0xF5, DPP_NEXT2 = 0xEE;       // quad_perm [1,1,3,3], [2,3,2,3]: lane + 1 / lane + 2 inside a quad
constexpr int DPP_ROR4 = 0x124, DPP_ROR8 = 0x128;       // row_ror:4, row_ror:8 (= lane ^ 8 inside a row)
constexpr int DPP_HALF_MIRROR = 0x141;                  // lane -> 7 - lane inside each group of 8
typedef uint32_t swap_pair_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void xor16_pair(float v, float &x, float &y) {  // {x, y} = {v[lane & ~16], v[lane | 16]}
  const swap_pair_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  x = __uint_as_float(r[0]);
  y = __uint_as_float(r[1]);
}
__device__ __forceinline__ void xor32_pair(float v, float &x, float &y) {  // {x, y} = {v[lane & ~32], v[lane | 32]}
  const swap_pair_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  x = __uint_as_float(r[0]);
  y = __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_xor16_xor32(float v) {  // v + v[lane ^ 16], then the same over lane ^ 32
  float x, y;
  xor16_pair(v, x, y);
  v = x + y;
  xor32_pair(v, x, y);
  return x + y;
}
__device__ __forceinline__ float row_sum16(float v) {  // sum over the 16 lanes of a row, in every lane
  v += dpp_move<DPP_XOR1>(v);
  v += dpp_move<DPP_XOR2>(v);
  v += dpp_move<DPP_ROR4>(v);
  v += dpp_move<DPP_ROR8>(v);
  return v;
}
__device__ __forceinline__ float row_max16(float v) {
  v = fmaxf(v, dpp_move<DPP_XOR1>(v));
  v = fmaxf(v, dpp_move<DPP_XOR2>(v));
  v = fmaxf(v, dpp_move<DPP_HALF_MIRROR>(v));
  v = fmaxf(v, dpp_move<DPP_ROR8>(v));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) { return sum_xor16_xor32(row_sum16(v)); }
__device__ __forceinline__ float max_xor16_xor32(float v) {  // max(v, v[lane ^ 16]), then the same over lane ^ 32
  float x, y;
  xor16_pair(v, x, y);
  v = fmaxf(x, y);
  xor32_pair(v, x, y);
  return fmaxf(x, y);
}
__device__ __forceinline__ float wave_max(float v) { return max_xor16_xor32(row_max16(v)); }

// The power of two at or below 1 / (4 rms), rms = 1 / inv_rms, kept within 2^-40 .. 2^40 (NormFold, kernels.hpp)
__device__ __forceinline__ float norm_fold_prescale(float inv_rms) {
  const float r = fminf(fmaxf(0.25f * inv_rms, 0x1p-40f), 0x1p40f);
  return __uint_as_float(__float_as_uint(r) & 0x7f800000u);
}

}  // namespace yscv
