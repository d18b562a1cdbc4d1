// Wide-M packed-int4 matmul (prefill GEMM): y[m][n] = sum_k x[m][k] * W[n][k].
// Replaces packed_int4_gemm_dispatch (crates/yscv-kernels/src/ops/int4_matmul.rs:548-605).
//
// MFMA-bound design for gfx950, sharing the tiled weight layout of the skinny kernel
// (int4_common.hpp):
//   * a workgroup owns BM = 16*MT rows x 256 columns of y; its 4 waves sit side by side
//     along N (64 columns = 4 weight tiles each), so every weight tile is fetched and
//     decoded by exactly one wave, straight from global memory into registers -- the packed
//     weights never pass through LDS and are never decoded twice inside a workgroup;
//   * the activations (already fp16 hi [+ lo], see x_prep) are staged through LDS in MFMA
//     A-operand order, one 128-k slab per stage, double buffered; every A fetch is a
//     contiguous 1 KiB ds_read_b128;
//   * v_mfma_f32_16x16x32_f16 with exact integer weights; the group scale is applied in
//     fp32 when a quantisation group ends (acc += scale * D), exactly as in the skinny
//     kernel, so both kernels agree to fp32 rounding.
#include <type_traits>

#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

struct GemmArgs {
  const uint8_t *tiles;
  const void *tscales;
  const uint8_t *tzps;
  const _Float16 *xh;
  const _Float16 *xl;
  const float *row_scale;
  void *y;
  int m, n;
  int nt, kt, ktp;
  int chunks, chunk_div;
  int k_pad;
  int y_dtype;
};

template <int GM, bool SF16>
struct GScale {
  static constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  typedef typename std::conditional<SF16, _Float16, float>::type elem_t;
  typedef elem_t vec_t __attribute__((ext_vector_type(SPT)));
  vec_t v;
  __device__ __forceinline__ void load(const void *base, size_t chunk_idx, int r) {
    const elem_t *p = reinterpret_cast<const elem_t *>(base) + (chunk_idx * 16 + r) * SPT;
    v = *reinterpret_cast<const vec_t *>(p);
  }
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
};

__device__ __forceinline__ void gemm_zp_consts(uint32_t zp, half2_t &c1, half2_t &c2) {
  _Float16 z = (_Float16)(float)zp;
  _Float16 a = (_Float16)(-1024.0f) - z;
  _Float16 b = (_Float16)(-64.0f) - z;
  c1 = half2_t{a, a};
  c2 = half2_t{b, b};
}

constexpr int G_NTW = 4;       // weight tiles (16 columns each) per wave
constexpr int G_WAVES = 4;      // G_NTW * G_WAVES * 16 = 256 columns per workgroup

template <int MT, int SPLIT, int GM, bool SF16>
__global__ void __launch_bounds__(256) int4_gemm_kernel(GemmArgs a) {
  constexpr int BM = MT * 16;
  constexpr int STAGE_HALVES = BM * 128;          // one slab of hi (or lo)
  constexpr int PASSES = BM * 16 / 256;           // 16-byte chunks per thread per slab
  extern __shared__ __attribute__((aligned(16))) _Float16 lds[];  // [2][SPLIT][STAGE_HALVES]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int m0 = blockIdx.y * BM;
  const int nt0 = (blockIdx.x * G_WAVES + wave) * G_NTW;  // first weight tile of this wave
  const bool has_zp = a.tzps != nullptr;

  float4_t acc[MT][G_NTW];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < G_NTW; j++) acc[i][j] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

  // ---- activation slab: global -> registers -> LDS (fragment order) -----------------
  uint4_t sreg[SPLIT][PASSES];
  auto slab_load = [&](int kt) {
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
      const int row = p * 16 + (tid >> 4);
      const int chunk = tid & 15;
      // rows past m repeat the last row (never stored): no load sits behind a branch of its own, so all loads of a
      // slab are in flight together
      const int gm = min(m0 + row, a.m - 1);
#pragma unroll
      for (int sp = 0; sp < SPLIT; sp++) {
        const _Float16 *src = (sp == 0 ? a.xh : a.xl) + (size_t)gm * a.k_pad + (size_t)kt * 128 + chunk * 8;
        sreg[sp][p] = *reinterpret_cast<const uint4_t *>(src);
      }
    }
  };
  auto slab_store = [&](int buf) {
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
      const int row = p * 16 + (tid >> 4);
      const int chunk = tid & 15;
      const int mt = row >> 4, rr = row & 15;
      const int j = chunk >> 2, cc = chunk & 3;
      const int off = (((mt * 4 + j) * 64) + cc * 16 + rr) * 8;  // in halves
#pragma unroll
      for (int sp = 0; sp < SPLIT; sp++)
        *reinterpret_cast<uint4_t *>(&lds[((size_t)buf * SPLIT + sp) * STAGE_HALVES + off]) = sreg[sp][p];
    }
  };

  // ---- weight tiles of one k-slab for this wave ----------------------------------------
  uint4_t wraw[2][G_NTW];
  GScale<GM, SF16> wsc[2][G_NTW];
  uint32_t wzp[2][G_NTW];
  // weight tiles past the last one repeat it (their columns are never stored); without zero points the zero-point
  // load reads the scale chunk instead and its value is ignored, so the load count does not depend on the weight
  const uint8_t *zsrc = has_zp ? a.tzps : reinterpret_cast<const uint8_t *>(a.tscales);
  auto w_load = [&](int kt, int slot) {
#pragma unroll
    for (int t = 0; t < G_NTW; t++) {
      const int nt = min(nt0 + t, a.nt - 1);
      wraw[slot][t] = *(reinterpret_cast<const uint4_t *>(a.tiles + ((size_t)nt * a.ktp + kt) * kTileBytes) + lane);
      const size_t chunk = (size_t)nt * a.chunks + (GM == GM128 ? kt / a.chunk_div : kt);
      wsc[slot][t].load(a.tscales, chunk, r);
      constexpr int SPT = GScale<GM, SF16>::SPT;
      const uint8_t *zp = zsrc + (chunk * 16 + r) * SPT;
      wzp[slot][t] = SPT == 4 ? *reinterpret_cast<const uint32_t *>(zp)
                              : (SPT == 2 ? (uint32_t) * reinterpret_cast<const uint16_t *>(zp) : (uint32_t)zp[0]);
    }
  };

  const half2_t c1_default = {(_Float16)(-1032.0f), (_Float16)(-1032.0f)};
  const half2_t c2_default = {(_Float16)(-72.0f), (_Float16)(-72.0f)};

  auto compute = [&](int buf, int slot) {
    // decode this wave's 4 tiles x 4 k-blocks once
    half8_t b[G_NTW][4];
#pragma unroll
    for (int t = 0; t < G_NTW; t++) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        half2_t c1 = c1_default, c2 = c2_default;
        if (has_zp) {
          uint32_t zp = GM == GM32 ? ((wzp[slot][t] >> (8 * j)) & 0xFF)
                                   : (GM == GM64 ? ((wzp[slot][t] >> (8 * (j >> 1))) & 0xFF) : (wzp[slot][t] & 0xFF));
          gemm_zp_consts(zp, c1, c2);
        }
        b[t][j] = decode8(wraw[slot][t][j], c1, c2);
      }
    }
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      half8_t ah[4], al[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int off = (((mt * 4 + j) * 64) + lane) * 8;
        ah[j] = *reinterpret_cast<const half8_t *>(&lds[((size_t)buf * SPLIT + 0) * STAGE_HALVES + off]);
        if constexpr (SPLIT == 2)
          al[j] = *reinterpret_cast<const half8_t *>(&lds[((size_t)buf * SPLIT + 1) * STAGE_HALVES + off]);
      }
#pragma unroll
      for (int t = 0; t < G_NTW; t++) {
        float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
          d = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[j], b[t][j], d, 0, 0, 0);
          if constexpr (SPLIT == 2) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[j], b[t][j], d, 0, 0, 0);
          const bool group_end = GM == GM32 || (GM == GM64 && (j & 1)) || (GM == GM128 && j == 3);
          if (group_end) {
            const float sc = wsc[slot][t].get(GM == GM32 ? j : (GM == GM64 ? (j >> 1) : 0));
#pragma unroll
            for (int i = 0; i < 4; i++) acc[mt][t][i] = fmaf(sc, d[i], acc[mt][t][i]);
            d = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
          }
        }
      }
    }
  };

  slab_load(0);
  w_load(0, 0);
  slab_store(0);
  __syncthreads();
  for (int kt = 0; kt < a.kt; kt += 2) {
    // even step: slot 0 / buffer 0
    if (kt + 1 < a.kt) {
      slab_load(kt + 1);
      w_load(kt + 1, 1);
    }
    compute(0, 0);
    if (kt + 1 < a.kt) slab_store(1);
    __syncthreads();
    if (kt + 1 >= a.kt) break;
    // odd step: slot 1 / buffer 1
    if (kt + 2 < a.kt) {
      slab_load(kt + 2);
      w_load(kt + 2, 0);
    }
    compute(1, 1);
    if (kt + 2 < a.kt) slab_store(0);
    __syncthreads();
  }

  // ---- epilogue ---------------------------------------------------------------------------
  float rsv[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int i = 0; i < 4; i++) rsv[mt][i] = 1.0f;
  if (a.row_scale) {  // one branch around all row scales
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
      for (int i = 0; i < 4; i++) rsv[mt][i] = a.row_scale[min(m0 + mt * 16 + c * 4 + i, a.m - 1)];
  }
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = m0 + mt * 16 + c * 4 + i;
      if (row >= a.m) continue;
      const float rs = rsv[mt][i];
#pragma unroll
      for (int t = 0; t < G_NTW; t++) {
        const int col = (nt0 + t) * 16 + r;
        if (col < a.n) store_out(a.y, (size_t)row * a.n + col, acc[mt][t][i] * rs, a.y_dtype);
      }
    }
  }
}

template <int MT, int SPLIT, int GM, bool SF16>
static int32_t gemm_launch_one(const GemmArgs &a, hipStream_t s) {
  constexpr int BM = MT * 16;
  size_t lds = (size_t)2 * SPLIT * BM * 128 * sizeof(_Float16);
  dim3 grid((unsigned)ceil_div((size_t)a.nt, (size_t)(G_NTW * G_WAVES)), (unsigned)ceil_div((size_t)a.m, (size_t)BM));
  auto kern = int4_gemm_kernel<MT, SPLIT, GM, SF16>;
  if (lds > 64 * 1024)
    YSCV_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, a);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

template <int MT, int SPLIT>
static int32_t gemm_launch_gm(const GemmArgs &a, int gm, bool sf16, hipStream_t s) {
  if (gm == GM32) return sf16 ? gemm_launch_one<MT, SPLIT, GM32, true>(a, s) : gemm_launch_one<MT, SPLIT, GM32, false>(a, s);
  if (gm == GM64) return sf16 ? gemm_launch_one<MT, SPLIT, GM64, true>(a, s) : gemm_launch_one<MT, SPLIT, GM64, false>(a, s);
  return sf16 ? gemm_launch_one<MT, SPLIT, GM128, true>(a, s) : gemm_launch_one<MT, SPLIT, GM128, false>(a, s);
}

int32_t launch_int4_gemm(const yscv_hip_int4_weight *w, const _Float16 *xh, const _Float16 *xl,
                         const float *row_scale, size_t k_pad, int split, void *y, int y_dtype, size_t m,
                         hipStream_t s, int epi, float *partial, size_t partial_bytes) {
  if (!w->tiled) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "int4 GEMM kernel needs the tiled layout");
  // 16-bit activations: the LDS-ring kernel from the first row count the skinny kernel does not take (rows are
  // padded to its 128-row tile; with few rows the weights are still streamed exactly once)
  // 17 .. 32 rows: the register-resident kernel of int4_mid.hip where its partial sums (if any) have their scratch
  if (m > 16 && m <= 32 && int4_mid_eligible(w, xh, y, y_dtype, split, m, k_pad, kMidPartialCap)) {
    const size_t need = int4_mid_partial_bytes(w, m);
    if (need == 0 || (partial != nullptr && partial_bytes >= need))
      return launch_int4_mid(w, xh, row_scale, k_pad, y, y_dtype, m, s, epi, partial, partial_bytes);
  }
  if (m > 16 && int4_gemm_ring_eligible(w, xh, y, y_dtype, split, m, k_pad))
    return launch_int4_gemm_ring(w, xh, row_scale, k_pad, y, y_dtype, m, s, epi, partial, partial_bytes);
  if (epi != EPI_STORE) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "fused epilogues above 16 rows exist for the LDS-ring GEMM only");
  GemmArgs a;
  a.tiles = w->tiles;
  a.tscales = w->tscales;
  a.tzps = w->has_zp ? w->tzps : nullptr;
  a.xh = xh;
  a.xl = xl;
  a.row_scale = row_scale;
  a.y = y;
  a.m = (int)m;
  a.n = (int)w->n;
  a.nt = (int)w->nt;
  a.kt = (int)w->kt;
  a.ktp = (int)w->ktp;
  a.chunks = (int)w->chunks;
  a.chunk_div = w->gm == GM128 ? (int)(w->g / 128) : 1;
  a.k_pad = (int)k_pad;
  a.y_dtype = y_dtype;
  const bool sf16 = w->scale_dtype == YSCV_HIP_F16;
  if (split == 2) return gemm_launch_gm<4, 2>(a, w->gm, sf16, s);
  return gemm_launch_gm<4, 1>(a, w->gm, sf16, s);
}

}  // namespace yscv
