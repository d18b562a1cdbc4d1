// Packed-int4 matmul for 17 .. 32 activation rows (fp16-prepared activations): y[m][n] = sum_k x[m][k] * W[n][k].
// Replaces packed_int4_gemm_dispatch (crates/yscv-kernels/src/ops/int4_matmul.rs:548-605) where m is too large for
// the skinny kernel (one MFMA tile of rows) and too small for the LDS-ring GEMM, whose short tiles are bound by their
// per-stage hand-over between producer and MMA waves, not by the weight stream.
//
// Same plan as the skinny kernel, with more rows per wave: K is split across the eight waves of a workgroup, each
// wave keeps ITS k-slice of ALL activation rows in registers as MFMA operands (RT = 2 row tiles of 16 x TPWM = 4 128-k
// tiles x 4 k-steps = 32 fragments = 128 VGPRs: 32 rows x 512 k), streams its own weight tiles of one
// 16-column block after the other from HBM through a ring of register sets (one 128-bit load per lane and tile,
// every iteration issues the same loads), decodes each packed word once ((q - zp) * scale in fp16, as the LDS-ring
// GEMM folds it) and feeds it to RT MFMAs.  Nothing but the partial sums of the waves goes through LDS: RT x 1 KiB per
// wave and block, two buffers, one LDS-only barrier per block; the waves' sums are added in a fixed order.
// A workgroup covers 8 x TPWM x 128 = 4096 k; a longer K is cut into parts over blockIdx.y whose f32 products go to
// partial[part][m][n] (the caller's workspace) and are added, epilogue included, by mid_finalize_kernel.
// (The same kernel with four row tiles and 256 k per wave, for 33 .. 64 rows, was slower than the LDS-ring GEMM with
// its K split on the prompt-pass shapes -- 3.86 against 3.56 ms for 64 tokens -- and is not instantiated.)
// The MFMA is issued with the weights as the A operand (D = W_frag x X_frag): a lane holds four consecutive columns
// of one row of y.
#include <mutex>
#include <type_traits>

#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

namespace {

__device__ __forceinline__ float mid_silu(float g) { return g / (1.0f + __expf(-g)); }

struct MidArgs {
  const uint8_t *tiles;
  const void *tscales;
  const uint8_t *tzps;  // null: zero point 8 everywhere
  const _Float16 *xh;
  const float *row_scale;  // null: 1
  void *y;
  float *partial;  // [parts][m][n] when K is cut into parts, else null
  int m, n, nt, ktp, chunks, chunk_div, k_pad, y_dtype, epi, ldy;
};

template <int GM, bool SF16>
struct MidScale {
  static constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  static constexpr int BYTES = SPT * (SF16 ? 2 : 4);
  typedef typename std::conditional<SF16, _Float16, float>::type elem_t;
  typedef elem_t vec_t __attribute__((ext_vector_type(SPT)));
  vec_t v;
  __device__ __forceinline__ void load(const char *p) { v = *reinterpret_cast<const vec_t *>(p); }
  // scale of k-step ks (0..3) of the tile, as fp16
  __device__ __forceinline__ _Float16 get(int ks) const { return (_Float16)v[GM == GM32 ? ks : (GM == GM64 ? ks >> 1 : 0)]; }
};

template <int GM>
__device__ __forceinline__ uint32_t mid_load_zp(const uint8_t *p) {
  constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  if constexpr (SPT == 4) return *reinterpret_cast<const uint32_t *>(p);
  if constexpr (SPT == 2) return *reinterpret_cast<const uint16_t *>(p);
  return *p;
}

// one wave's registers for one 16-column block
template <int TPWM, int GM, bool SF16, bool HAS_ZP>
struct MidBlock {
  uint4_t w[TPWM];
  MidScale<GM, SF16> s[TPWM];
  uint32_t z[HAS_ZP ? TPWM : 1];
};

template <int RT, int TPWM, int GM, bool SF16, bool HAS_ZP, int P>
__global__ void __launch_bounds__(512, 1) int4_mid_kernel(MidArgs a) {
  constexpr int WAVES = 8;
  constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  typedef MidBlock<TPWM, GM, SF16, HAS_ZP> Block;
  extern __shared__ __attribute__((aligned(16))) float4_t mid_red[];  // [2][WAVES][RT][64]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int part = blockIdx.y;
  const int t0 = (part * WAVES + wave) * TPWM;  // first 128-k tile of this wave's slice
  NibbleConsts nc;
  nc.init();

  // ---- weight stream of this wave: block `it` of the workgroup is 16-column block blockIdx.x + it * gridDim.x.  Tiles
  // past the stored ones repeat the last one (their activations are zero), requests past the last block repeat it
  const int stride = gridDim.x;
  const int iters = (a.nt - (int)blockIdx.x + stride - 1) / stride;  // >= 1, uniform in the workgroup
  int tl[TPWM], ch[TPWM];
#pragma unroll
  for (int j = 0; j < TPWM; j++) {
    tl[j] = min(t0 + j, a.ktp - 1);
    ch[j] = GM == GM128 ? tl[j] / a.chunk_div : tl[j];
  }
  auto issue = [&](Block &b, int it) {
    const size_t nt = (size_t)blockIdx.x + (size_t)min(it, iters - 1) * stride;
#pragma unroll
    for (int j = 0; j < TPWM; j++) {
      b.w[j] = __builtin_nontemporal_load(
          reinterpret_cast<const uint4_t *>(a.tiles + (nt * a.ktp + tl[j]) * kTileBytes + lane * 16));
      b.s[j].load(reinterpret_cast<const char *>(a.tscales) + ((nt * a.chunks + ch[j]) * 16 + r) * MidScale<GM, SF16>::BYTES);
      if constexpr (HAS_ZP) b.z[j] = mid_load_zp<GM>(a.tzps + ((nt * a.chunks + ch[j]) * 16 + r) * SPT);
    }
  };
  Block ring[P];
#pragma unroll
  for (int p = 0; p < P; p++) issue(ring[p], p);

  // ---- activations -> registers: fragment (j, ks, rt) of lane (r, c) = row 16 rt + r, k = 128 (t0 + j) + 32 ks + 8 c .. + 7
  half8_t xa[TPWM][4][RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++) {
    const int row = min(rt * 16 + r, a.m - 1);  // rows past m repeat the last one and are not stored
#pragma unroll
    for (int j = 0; j < TPWM; j++) {
      const bool live = t0 + j < a.ktp;
      const _Float16 *src = a.xh + (size_t)row * a.k_pad + (size_t)tl[j] * 128 + c * 8;
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        half8_t v = *reinterpret_cast<const half8_t *>(src + ks * 32);
        if (!live) v = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        xa[j][ks][rt] = v;
      }
    }
  }

  // ---- epilogue constants of this thread's share of a block: float4 unit u = tid (rt = u / 64, lane' = u % 64)
  const bool reducer = tid < RT * 64;
  const int u_rt = tid >> 6, u_lane = tid & 63;
  const int out_row = u_rt * 16 + (u_lane & 15);
  const int out_c4 = (u_lane >> 4) * 4;
  float rs = 1.0f;
  if (reducer && a.row_scale != nullptr) rs = a.row_scale[min(out_row, a.m - 1)];

  auto compute = [&](const Block &b, int it) {
    float4_t acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) acc[rt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < TPWM; j++) {
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        const int e = GM == GM32 ? ks : (GM == GM64 ? ks >> 1 : 0);
        const uint32_t zq = HAS_ZP ? ((b.z[HAS_ZP ? j : 0] >> (8 * e)) & 0xFFu) : 8u;
        const _Float16 z = (_Float16)(float)zq;
        const _Float16 c1v = (_Float16)(-1024.0f) - z, c2v = (_Float16)(-64.0f) - z;
        const _Float16 s = b.s[j].get(ks);
        const half8_t sv = {s, s, s, s, s, s, s, s};
        const half8_t wf = decode8_exact(b.w[j][ks], nc, half2_t{c1v, c1v}, half2_t{c2v, c2v}) * sv;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, xa[j][ks][rt], acc[rt], 0, 0, 0);
      }
    }
    // the waves' partial sums meet in LDS; buffer it & 1 is free again once every wave has passed the barrier of block
    // it - 1, i.e. has finished adding block it - 2
    float4_t *buf = mid_red + (size_t)(it & 1) * WAVES * RT * 64;
#pragma unroll
    for (int rt = 0; rt < RT; rt++) buf[(wave * RT + rt) * 64 + lane] = acc[rt];
    lds_barrier();
    if (reducer) {
      float4_t v = buf[u_rt * 64 + u_lane];
#pragma unroll
      for (int w = 1; w < WAVES; w++) v += buf[(w * RT + u_rt) * 64 + u_lane];
      v = v * rs;
      const size_t nt = (size_t)blockIdx.x + (size_t)it * stride;
      const int col = (int)nt * 16 + out_c4;
      if (out_row < a.m && col < a.n) {
        const bool whole = col + 4 <= a.n && ((a.n | a.ldy) & 3) == 0;
        if (a.partial != nullptr) {
          float *dst = a.partial + ((size_t)part * a.m + out_row) * a.n + col;
          if (whole) {
            *reinterpret_cast<float4_t *>(dst) = v;
          } else {
            for (int e = 0; e < 4; e++)
              if (col + e < a.n) dst[e] = v[e];
          }
        } else if (a.epi == EPI_SWIGLU) {
          // columns col .. col + 3 are gate, up, gate, up of two channels (n is even, col a multiple of 4)
          const size_t oh = (size_t)out_row * (a.ldy >> 1) + (col >> 1);
          store_out(a.y, oh, mid_silu(v[0]) * v[1], a.y_dtype);
          if (col + 2 < a.n) store_out(a.y, oh + 1, mid_silu(v[2]) * v[3], a.y_dtype);
        } else if (a.epi == EPI_ADD_F32) {
          float *dst = reinterpret_cast<float *>(a.y) + (size_t)out_row * a.ldy + col;
          if (whole) {
            *reinterpret_cast<float4_t *>(dst) = *reinterpret_cast<const float4_t *>(dst) + v;
          } else {
            for (int e = 0; e < 4; e++)
              if (col + e < a.n) dst[e] += v[e];
          }
        } else {
          const size_t o = (size_t)out_row * a.ldy + col;
          if (whole && a.y_dtype == YSCV_HIP_F32) {
            *reinterpret_cast<float4_t *>(reinterpret_cast<float *>(a.y) + o) = v;
          } else if (whole && a.y_dtype == YSCV_HIP_F16) {
            *reinterpret_cast<half4_t *>(reinterpret_cast<_Float16 *>(a.y) + o) =
                half4_t{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
          } else {
            for (int e = 0; e < 4; e++)
              if (col + e < a.n) store_out(a.y, o + e, v[e], a.y_dtype);
          }
        }
      }
    }
  };

  for (int it0 = 0; it0 < iters; it0 += P) {
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int it = it0 + p;
      if (it < iters) {  // uniform in the workgroup
        compute(ring[p], it);
        issue(ring[p], it + P);
      }
    }
  }
}

// Adds the K parts in a fixed order and applies the epilogue: four columns per thread.
__global__ void __launch_bounds__(256) mid_finalize_kernel(const float *__restrict__ partial, int parts, int m, int n, void *y,
                                                           int y_dtype, int epi, int ldy) {
  const int chunks = (n + 3) / 4;
  const size_t total = (size_t)m * chunks;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const int row = (int)(idx / chunks), col = (int)(idx % chunks) * 4;
    const bool whole = col + 4 <= n && (n & 3) == 0;
    float4_t v = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j = 0; j < parts; j++) {
      const float *src = partial + ((size_t)j * m + row) * n + col;
      if (whole) {
        v += *reinterpret_cast<const float4_t *>(src);
      } else {
        for (int e = 0; e < 4; e++)
          if (col + e < n) v[e] += src[e];
      }
    }
    const size_t o = (size_t)row * ldy + col;
    if (epi == EPI_SWIGLU) {
      const size_t oh = (size_t)row * (ldy >> 1) + (col >> 1);
      store_out(y, oh, mid_silu(v[0]) * v[1], y_dtype);
      if (col + 2 < n) store_out(y, oh + 1, mid_silu(v[2]) * v[3], y_dtype);
    } else if (epi == EPI_ADD_F32) {
      float *dst = reinterpret_cast<float *>(y) + o;
      for (int e = 0; e < 4; e++)
        if (col + e < n) dst[e] += v[e];
    } else {
      for (int e = 0; e < 4; e++)
        if (col + e < n) store_out(y, o + e, v[e], y_dtype);
    }
  }
}

template <int RT, int TPWM, int GM, bool SF16, bool HAS_ZP, int P>
int32_t mid_launch_one(const MidArgs &a, int parts, int cus, hipStream_t s) {
  constexpr int LDS = 2 * 8 * RT * 64 * 16;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kern = int4_mid_kernel<RT, TPWM, GM, SF16, HAS_ZP, P>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
  });
  if (attr_err != hipSuccess)
    return set_error(YSCV_HIP_ERR_DEVICE, "cannot reserve %d bytes of LDS: %s", LDS, hipGetErrorString(attr_err));
  int nparts = cus / parts;
  nparts = nparts < 1 ? 1 : (nparts > a.nt ? a.nt : nparts);
  hipLaunchKernelGGL(kern, dim3((unsigned)nparts, (unsigned)parts), dim3(512), LDS, s, a);
  YSCV_HIP_TRY(hipGetLastError());
  if (a.partial != nullptr) {
    const size_t work = (size_t)a.m * ((a.n + 3) / 4);
    const unsigned fb = (unsigned)std::min<size_t>((work + 255) / 256, 4096);
    hipLaunchKernelGGL(mid_finalize_kernel, dim3(fb), dim3(256), 0, s, a.partial, parts, a.m, a.n, a.y, a.y_dtype, a.epi, a.ldy);
    YSCV_HIP_TRY(hipGetLastError());
  }
  return YSCV_HIP_OK;
}

template <int RT, int TPWM, int P, int GM, bool SF16>
int32_t mid_launch_zp(const MidArgs &a, int parts, int cus, hipStream_t s) {
  return a.tzps ? mid_launch_one<RT, TPWM, GM, SF16, true, P>(a, parts, cus, s) : mid_launch_one<RT, TPWM, GM, SF16, false, P>(a, parts, cus, s);
}

template <int RT, int TPWM, int P>
int32_t mid_launch_gm(const MidArgs &a, int gm, bool sf16, int parts, int cus, hipStream_t s) {
  if (gm == GM32) return sf16 ? mid_launch_zp<RT, TPWM, P, GM32, true>(a, parts, cus, s) : mid_launch_zp<RT, TPWM, P, GM32, false>(a, parts, cus, s);
  if (gm == GM64) return sf16 ? mid_launch_zp<RT, TPWM, P, GM64, true>(a, parts, cus, s) : mid_launch_zp<RT, TPWM, P, GM64, false>(a, parts, cus, s);
  return sf16 ? mid_launch_zp<RT, TPWM, P, GM128, true>(a, parts, cus, s) : mid_launch_zp<RT, TPWM, P, GM128, false>(a, parts, cus, s);
}

// k tiles a workgroup covers: eight waves x four tiles
inline size_t mid_tiles_per_wg(size_t) { return 8 * 4; }

}  // namespace

// K parts of the launch for m rows (1: the workgroup covers all of K, no partial sums)
size_t int4_mid_parts(const yscv_hip_int4_weight *w, size_t m) { return ceil_div(w->ktp, mid_tiles_per_wg(m)); }

size_t int4_mid_partial_bytes(const yscv_hip_int4_weight *w, size_t m) {
  const size_t parts = int4_mid_parts(w, m);
  return parts > 1 ? parts * m * w->n * sizeof(float) : 0;
}

// 17 .. 32 rows of fp16-prepared activations against a tiled weight.  A workgroup covers 4096 k; a longer K needs the
// partial-sum scratch: the kernel is taken where that scratch stays within `max_partial_bytes`.
bool int4_mid_eligible(const yscv_hip_int4_weight *w, const _Float16 *xh, const void *y, int y_dtype, int split, size_t m,
                       size_t k_pad, size_t max_partial_bytes) {
  if (!w->tiled || split != 1 || m <= 16 || m > 32) return false;
  if ((reinterpret_cast<uintptr_t>(xh) & 15) != 0 || (k_pad & 7) != 0) return false;
  const size_t align = y_dtype == YSCV_HIP_F32 ? 16 : 8;
  if ((reinterpret_cast<uintptr_t>(y) & (align - 1)) != 0) return false;
  return int4_mid_partial_bytes(w, m) <= max_partial_bytes;
}

int32_t launch_int4_mid(const yscv_hip_int4_weight *w, const _Float16 *xh, const float *row_scale, size_t k_pad, void *y,
                        int y_dtype, size_t m, hipStream_t s, int epi, float *partial, size_t partial_bytes) {
  if (epi == EPI_ADD_F32 && y_dtype != YSCV_HIP_F32) return set_error(YSCV_HIP_ERR_INVALID_ARG, "the add epilogue updates an f32 tensor");
  if (epi == EPI_SWIGLU && (w->n & 1)) return set_error(YSCV_HIP_ERR_INVALID_ARG, "SwiGLU epilogue needs an even row count");
  const Context *ctx = nullptr;
  YSCV_TRY(ensure_context(&ctx));
  const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  const size_t parts = int4_mid_parts(w, m);
  const size_t need = int4_mid_partial_bytes(w, m);
  if (need > 0 && (partial == nullptr || partial_bytes < need || (reinterpret_cast<uintptr_t>(partial) & 15) != 0))
    return set_error(YSCV_HIP_ERR_INVALID_ARG, "this shape needs %zu bytes of partial-sum scratch", need);
  MidArgs a;
  a.tiles = w->tiles;
  a.tscales = w->tscales;
  a.tzps = w->has_zp ? w->tzps : nullptr;
  a.xh = xh;
  a.row_scale = row_scale;
  a.y = y;
  a.partial = need > 0 ? partial : nullptr;
  a.m = (int)m;
  a.n = (int)w->n;
  a.nt = (int)w->nt;
  a.ktp = (int)w->ktp;
  a.chunks = (int)w->chunks;
  a.chunk_div = w->gm == GM128 ? (int)(w->g / 128) : 1;
  a.k_pad = (int)k_pad;
  a.y_dtype = y_dtype;
  a.epi = epi;
  a.ldy = (int)w->n;
  const bool sf16 = w->scale_dtype == YSCV_HIP_F16;
  return mid_launch_gm<2, 4, 2>(a, w->gm, sf16, (int)parts, cus, s);
}

}  // namespace yscv
