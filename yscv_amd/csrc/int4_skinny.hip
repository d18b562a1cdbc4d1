// Skinny-M packed-int4 matmul (decode GEMV, m <= 16): y[m][n] = sum_k x[m][k] * W[n][k].
// Replaces packed_int4_gemv_dispatch (crates/yscv-kernels/src/ops/int4_matmul.rs:310-377),
// which the reference calls once per activation row (crates/yscv-onnx/src/runner/linear.rs:255-267).
//
// Bandwidth-bound design for gfx950:
//   * weights stream from HBM exactly once, as 1 KiB coalesced tiles (one 128-bit load per
//     lane, see int4_common.hpp), and are decoded to fp16 in registers;
//   * the activation rows sit in registers for the whole kernel, pre-split into fp16
//     hi (+ lo for f32 input) and already in MFMA A-operand order, so the inner loop touches
//     neither LDS nor L2 for them;
//   * v_mfma_f32_16x16x32_f16 does the dot products: A = activations (rows = up to 16
//     batch rows, padded with zeros), B = decoded weights (16 output rows), one MFMA per
//     32-k block, i.e. per quantisation group when group_size is 32;
//   * group scales are applied in fp32 to the MFMA result (acc += scale * D), so the
//     fp16 operands are exact integers and exact activation halves;
//   * K is split across the wavefronts of a workgroup (each wave keeps its own K slice of
//     the activations); the per-wave partial sums meet in LDS once per 16-row tile.
//     When K is too long for one workgroup, a grid-level split writes fp32 partials that a
//     second small kernel adds up in a fixed order (no atomics: results are deterministic).
#include <type_traits>

#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

__device__ __forceinline__ float silu(float g) { return g / (1.0f + __expf(-g)); }

struct SkinnyArgs {
  const uint8_t *tiles;
  const void *tscales;
  const uint8_t *tzps;  // null: zero point 8 everywhere
  const _Float16 *xh;
  const _Float16 *xl;
  const float *row_scale;
  void *y;
  float *partial;  // [ksg][m][n] when ksg > 1
  int m, n;
  int nt, kt;      // tile counts
  int chunks;      // scale chunks per n-tile
  int chunk_div;   // GM128: tiles per scale chunk (group_size / 128)
  int k_pad;       // row stride of xh / xl
  int y_dtype;
  int ksg;
  int epi;  // EPI_STORE / EPI_ADD_F32 / EPI_SWIGLU
};

// Scales of one (tile, row) kept in their storage type until used: 1, 2 or 4 values.
template <int GM, bool SF16>
struct ScaleRaw {
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

template <int GM>
__device__ __forceinline__ void load_zps(const uint8_t *base, size_t chunk_idx, int r, uint32_t &packed) {
  constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  size_t off = (chunk_idx * 16 + r) * SPT;
  if constexpr (SPT == 4)
    packed = *reinterpret_cast<const uint32_t *>(base + off);
  else if constexpr (SPT == 2)
    packed = *reinterpret_cast<const uint16_t *>(base + off);
  else
    packed = base[off];
}

__device__ __forceinline__ void zp_consts(uint32_t zp, half2_t &c1, half2_t &c2) {
  _Float16 z = (_Float16)(float)zp;
  _Float16 a = (_Float16)(-1024.0f) - z;
  _Float16 b = (_Float16)(-64.0f) - z;
  c1 = half2_t{a, a};
  c2 = half2_t{b, b};
}

// One wave's registers for one 16-row tile: TPW weight tiles + their scales / zero points.
template <int TPW, int GM, bool SF16>
struct TileRegs {
  uint4_t w[TPW];
  ScaleRaw<GM, SF16> s[TPW];
  uint32_t z[TPW];
};

template <int TPW, int SPLIT, int NI, int GM, bool SF16, int P>
__global__ void __launch_bounds__(512, 1) int4_skinny_kernel(SkinnyArgs a) {
  extern __shared__ float red[];  // [2][waves][NI][64]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves = blockDim.x >> 6;
  const int r = lane & 15;
  const int c = lane >> 4;
  const int t0 = (blockIdx.y * waves + wave) * TPW;  // first 128-k tile of this wave's K slice

  // ---- activations -> registers, in A-operand order --------------------------------
  // A row `r` of the MFMA carries batch row m when r == 4*(m / NI) + (m % NI): the
  // useful results then sit in the first NI of the four accumulator registers.
  half8_t xa[TPW][4][SPLIT];
  {
    const int i = r & 3;
    const int mrow = (r >> 2) * NI + i;
    const bool valid = (i < NI) && (mrow < a.m);
#pragma unroll
    for (int t = 0; t < TPW; t++) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        half8_t h = {0, 0, 0, 0, 0, 0, 0, 0}, l = {0, 0, 0, 0, 0, 0, 0, 0};
        if (valid && (t0 + t) < a.kt) {
          size_t off = (size_t)mrow * a.k_pad + (size_t)(t0 + t) * 128 + j * 32 + c * 8;
          h = *reinterpret_cast<const half8_t *>(a.xh + off);
          if constexpr (SPLIT == 2) l = *reinterpret_cast<const half8_t *>(a.xl + off);
        }
        xa[t][j][0] = h;
        if constexpr (SPLIT == 2) xa[t][j][1] = l;
      }
    }
  }

  const half2_t c1_default = {(_Float16)(-1032.0f), (_Float16)(-1032.0f)};
  const half2_t c2_default = {(_Float16)(-72.0f), (_Float16)(-72.0f)};
  const bool has_zp = a.tzps != nullptr;

  auto issue = [&](int nt, TileRegs<TPW, GM, SF16> &tr) {
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      const int kt = t0 + t;
      if (kt < a.kt) {
        const uint4_t *src = reinterpret_cast<const uint4_t *>(a.tiles + ((size_t)nt * a.kt + kt) * kTileBytes) + lane;
        tr.w[t] = __builtin_nontemporal_load(src);
        size_t chunk = (size_t)nt * a.chunks + (GM == GM128 ? kt / a.chunk_div : kt);
        tr.s[t].load(a.tscales, chunk, r);
        if (has_zp) load_zps<GM>(a.tzps, chunk, r, tr.z[t]);
      }
    }
  };

  auto compute = [&](int nt, const TileRegs<TPW, GM, SF16> &tr, int it) {
    float acc[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) acc[i] = 0.0f;
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      if ((t0 + t) < a.kt) {
        const uint32_t wj[4] = {tr.w[t][0], tr.w[t][1], tr.w[t][2], tr.w[t][3]};
        float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
          half2_t c1 = c1_default, c2 = c2_default;
          if (has_zp) {
            uint32_t zp = GM == GM32 ? ((tr.z[t] >> (8 * j)) & 0xFF)
                                     : (GM == GM64 ? ((tr.z[t] >> (8 * (j >> 1))) & 0xFF) : tr.z[t]);
            zp_consts(zp, c1, c2);
          }
          half8_t b = decode8(wj[j], c1, c2);
          d = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][j][0], b, d, 0, 0, 0);
          if constexpr (SPLIT == 2) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][j][1], b, d, 0, 0, 0);
          const bool group_end = GM == GM32 || (GM == GM64 && (j & 1)) || (GM == GM128 && j == 3);
          if (group_end) {
            const float sc = tr.s[t].get(GM == GM32 ? j : (GM == GM64 ? (j >> 1) : 0));
#pragma unroll
            for (int i = 0; i < NI; i++) acc[i] = fmaf(sc, d[i], acc[i]);
            d = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
          }
        }
      }
    }
    // ---- meet the other K slices in LDS ---------------------------------------------
    float *buf = red + (size_t)(it & 1) * waves * NI * 64;
#pragma unroll
    for (int i = 0; i < NI; i++) buf[(wave * NI + i) * 64 + lane] = acc[i];
    __syncthreads();
    if (wave == (it % waves)) {
      const int col = nt * 16 + r;
#pragma unroll
      for (int i = 0; i < NI; i++) {
        float v = 0.0f;
        for (int w = 0; w < waves; w++) v += buf[(w * NI + i) * 64 + lane];
        const int mrow = c * NI + i;
        const bool live = mrow < a.m && col < a.n;
        if (a.ksg > 1) {
          if (live) a.partial[((size_t)blockIdx.y * a.m + mrow) * a.n + col] = v;
        } else {
          if (a.row_scale && mrow < a.m) v *= a.row_scale[mrow];
          if (a.epi == EPI_SWIGLU) {
            // rows 2i / 2i+1 of the weight are gate_i / up_i: neighbours in the wave
            const float up = __shfl_xor(v, 1, 64);
            if (live && !(r & 1))
              store_out(a.y, (size_t)mrow * (a.n >> 1) + (col >> 1), silu(v) * up, a.y_dtype);
          } else if (a.epi == EPI_ADD_F32) {
            if (live) {
              float *dst = reinterpret_cast<float *>(a.y) + (size_t)mrow * a.n + col;
              *dst = *dst + v;
            }
          } else if (live) {
            store_out(a.y, (size_t)mrow * a.n + col, v, a.y_dtype);
          }
        }
      }
    }
  };

  // Ring of P register slots: while one 16-row tile is being consumed, the loads of the next
  // P-1 are in flight, so the memory pipeline never drains at the per-tile barrier.
  TileRegs<TPW, GM, SF16> ring[P];
  const int stride = gridDim.x;
  int nt = blockIdx.x;
#pragma unroll
  for (int sl = 0; sl < P; sl++) {
    const int n = nt + sl * stride;
    if (n < a.nt) issue(n, ring[sl]);
  }
  int it = 0;
  while (nt < a.nt) {
#pragma unroll
    for (int sl = 0; sl < P; sl++) {
      if (nt < a.nt) {
        compute(nt, ring[sl], it);
        const int nn = nt + P * stride;
        if (nn < a.nt) issue(nn, ring[sl]);
        nt += stride;
        it++;
      }
    }
  }
}

// partial [ksg][m][n] -> y, fixed summation order, same epilogues as the fused path
__global__ void int4_skinny_finalize_kernel(const float *__restrict__ partial, int ksg, int m, int n,
                                            const float *__restrict__ row_scale, void *y, int y_dtype, int epi) {
  const size_t total = (size_t)m * n;
  if (epi == EPI_SWIGLU) {
    const size_t half_n = (size_t)(n >> 1);
    for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < (size_t)m * half_n;
         idx += (size_t)gridDim.x * blockDim.x) {
      const size_t row = idx / half_n, j = idx % half_n;
      float g = 0.0f, u = 0.0f;
      for (int s = 0; s < ksg; s++) {
        g += partial[(size_t)s * total + row * n + 2 * j];
        u += partial[(size_t)s * total + row * n + 2 * j + 1];
      }
      if (row_scale) {
        g *= row_scale[row];
        u *= row_scale[row];
      }
      store_out(y, idx, silu(g) * u, y_dtype);
    }
    return;
  }
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    float v = 0.0f;
    for (int s = 0; s < ksg; s++) v += partial[(size_t)s * total + idx];
    if (row_scale) v *= row_scale[idx / n];
    if (epi == EPI_ADD_F32) {
      float *dst = reinterpret_cast<float *>(y) + idx;
      *dst = *dst + v;
    } else {
      store_out(y, idx, v, y_dtype);
    }
  }
}

SkinnyPlan plan_int4_skinny(const yscv_hip_int4_weight *w, size_t m, int split, int num_cus) {
  (void)m;
  SkinnyPlan p;
  // x registers per wave: 16 * tpw * split <= 128
  (void)split;
  p.tpw = 4;
  const int max_waves = 8;
  int slices = (int)ceil_div(w->kt, (size_t)p.tpw);
  p.ksg = (int)ceil_div((size_t)slices, (size_t)max_waves);
  p.waves = (int)ceil_div((size_t)slices, (size_t)p.ksg);
  int gx = (int)w->nt;
  int cap = num_cus > 0 ? num_cus : 256;
  // one resident workgroup per CU and k-split slice; more tiles than that loop inside the kernel
  int per = cap / p.ksg;
  if (per < 1) per = 1;
  if (gx > per) {
    // spread the tiles evenly over the resident workgroups
    int rounds = (int)ceil_div((size_t)gx, (size_t)per);
    gx = (int)ceil_div((size_t)w->nt, (size_t)rounds);
  }
  p.grid_x = gx;
  p.partial_bytes = p.ksg > 1 ? (size_t)p.ksg * m * w->n * sizeof(float) : 0;
  return p;
}

template <int TPW, int SPLIT, int NI, int GM, bool SF16>
static int32_t launch_one(const SkinnyArgs &a, const SkinnyPlan &plan, hipStream_t s) {
  size_t lds = (size_t)2 * plan.waves * NI * 64 * sizeof(float);
  hipLaunchKernelGGL((int4_skinny_kernel<TPW, SPLIT, NI, GM, SF16, (SPLIT == 2 ? 2 : 4)>), dim3(plan.grid_x, plan.ksg),
                     dim3(plan.waves * 64), lds, s, a);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

template <int TPW, int SPLIT, int NI>
static int32_t launch_gm(const SkinnyArgs &a, const SkinnyPlan &plan, int gm, bool sf16, hipStream_t s) {
  if (gm == GM32) return sf16 ? launch_one<TPW, SPLIT, NI, GM32, true>(a, plan, s) : launch_one<TPW, SPLIT, NI, GM32, false>(a, plan, s);
  if (gm == GM64) return sf16 ? launch_one<TPW, SPLIT, NI, GM64, true>(a, plan, s) : launch_one<TPW, SPLIT, NI, GM64, false>(a, plan, s);
  return sf16 ? launch_one<TPW, SPLIT, NI, GM128, true>(a, plan, s) : launch_one<TPW, SPLIT, NI, GM128, false>(a, plan, s);
}

int32_t launch_int4_skinny(const yscv_hip_int4_weight *w, const SkinnyPlan &plan, const _Float16 *xh,
                           const _Float16 *xl, const float *row_scale, size_t k_pad, int split,
                           void *y, int y_dtype, size_t m, float *partial, int epi, hipStream_t s) {
  if (!w->tiled) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "skinny int4 kernel needs the tiled layout");
  if (m == 0 || m > 16) return set_error(YSCV_HIP_ERR_INVALID_ARG, "skinny int4 kernel handles 1 <= m <= 16, got %zu", m);
  if (plan.ksg > 1 && !partial) return set_error(YSCV_HIP_ERR_INVALID_ARG, "k-split needs a partial buffer");
  SkinnyArgs a;
  a.tiles = w->tiles;
  a.tscales = w->tscales;
  a.tzps = w->has_zp ? w->tzps : nullptr;
  a.xh = xh;
  a.xl = xl;
  a.row_scale = row_scale;
  a.y = y;
  a.partial = partial;
  a.m = (int)m;
  a.n = (int)w->n;
  a.nt = (int)w->nt;
  a.kt = (int)w->kt;
  a.chunks = (int)w->chunks;
  a.chunk_div = w->gm == GM128 ? (int)(w->g / 128) : 1;
  a.k_pad = (int)k_pad;
  a.y_dtype = y_dtype;
  a.ksg = plan.ksg;
  a.epi = epi;
  if (epi == EPI_ADD_F32 && y_dtype != YSCV_HIP_F32) return set_error(YSCV_HIP_ERR_INVALID_ARG, "residual accumulation needs an f32 output");
  if (epi == EPI_SWIGLU && (w->n & 1)) return set_error(YSCV_HIP_ERR_INVALID_ARG, "SwiGLU epilogue needs an even row count");
  const bool sf16 = w->scale_dtype == YSCV_HIP_F16;
  const bool small = m <= 4;
  int32_t st;
  if (split == 2) {
    st = small ? launch_gm<4, 2, 1>(a, plan, w->gm, sf16, s) : launch_gm<4, 2, 4>(a, plan, w->gm, sf16, s);
  } else {
    st = small ? launch_gm<4, 1, 1>(a, plan, w->gm, sf16, s) : launch_gm<4, 1, 4>(a, plan, w->gm, sf16, s);
  }
  YSCV_TRY(st);
  if (plan.ksg > 1) {
    size_t total = m * w->n;
    int blocks = (int)ceil_div(total, (size_t)256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(int4_skinny_finalize_kernel, dim3(blocks), dim3(256), 0, s, partial, plan.ksg,
                       (int)m, (int)w->n, row_scale, y, y_dtype, epi);
    YSCV_HIP_TRY(hipGetLastError());
  }
  return YSCV_HIP_OK;
}

}  // namespace yscv
