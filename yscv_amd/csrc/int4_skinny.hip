// Skinny-M packed-int4 matmul (decode GEMV, m <= 16): y[m][n] = sum_k x[m][k] * W[n][k].
// Replaces packed_int4_gemv_dispatch (crates/yscv-kernels/src/ops/int4_matmul.rs:310-377),
// which the reference calls once per activation row (crates/yscv-onnx/src/runner/linear.rs:255-267).
//
// Bandwidth-bound design for gfx950.  The kernel is limited by how many instructions a SIMD can
// issue per byte streamed (about 80 VALU slots per KiB of weights at 8 TB/s), so everything in the
// inner loop is there to keep that count low:
//   * weights stream from HBM exactly once, as 1 KiB coalesced tiles (one 128-bit load per lane,
//     layout in int4_common.hpp); a ring of P register slots keeps P-1 blocks in flight per wave.
//     Every iteration issues the same loads (requests past the last block repeat it, served by the
//     caches), so the compiler's s_waitcnt counts are exact; the first P blocks are requested
//     before the activations are fetched, and no load in the kernel sits behind a per-load branch
//     (a guarded load costs one memory round trip each, under load more than a microsecond);
//   * the activation rows sit in registers for the whole kernel, as fp16 hi (+ lo for f32 input),
//     already in MFMA A-operand order: the inner loop reads neither LDS nor L2 for them;
//   * v_mfma_f32_16x16x32_f16 does the dot products (A = up to 16 activation rows, B = 16 weight
//     rows), one MFMA per 32-k block = one quantisation group when group_size is 32;
//   * nibbles become fp16 with one v_and_or_b32 per pair: 0x6400 | q = 1024 + q and
//     0x6400 | (q << 4) = 1024 + 16 q.  For symmetric weights (zero point 8) and fp16/bf16
//     activations the offsets are not subtracted per weight: the activation slots that meet the
//     16 q form are pre-divided by 16, and the offset term sum_k x_k * (1024 + 8 or 1024 + 128)
//     -- which does not depend on the weight row -- is computed once per kernel by the same MFMA
//     against a constant operand.  With m <= 4 it is subtracted from each group's result; with
//     m > 4 (four useful accumulators per lane) the products -offset[row][block] * scale[n][block]
//     of a whole 16-row block are added by four v_mfma_f32_16x16x4_f32 at the end of the block.
//     With explicit zero points or f32 activations the offsets are subtracted exactly in fp16
//     before the MFMA;
//   * group scales are applied in fp32 to the MFMA result (acc += scale * D);
//   * K is split across the wavefronts of a workgroup (each wave owns 512 k of the activations);
//     the per-wave partial sums meet in LDS behind an LDS-only barrier, once per four 16-row blocks
//     where the ring depth allows (fewer barriers, and every wave has a share of the sums to add).
//     When K is too long for one workgroup, a grid-level split writes fp32 partials that a second
//     small kernel adds in a fixed order (no atomics on shared outputs: results are deterministic).
#include <mutex>
#include <type_traits>

#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

__device__ __forceinline__ float silu(float g) { return g / (1.0f + __expf(-g)); }

constexpr int TPW = 4;  // 128-k tiles per wave: 512 k of activations live in 64 VGPRs (hi)

struct SkinnyArgs {
  const uint8_t *tiles;
  const void *tscales;
  const uint8_t *tzps;  // null: zero point 8 everywhere
  const _Float16 *xh;
  const _Float16 *xl;
  const float *xf;     // raw f32 activations (row stride k_pad) for the kernels that split them themselves, else null
  const uint16_t *xb;  // raw bf16 activations (row stride k_pad), else null
  const float *row_scale;
  void *y;
  float *partial;  // [ksg][m][n] when ksg > 1
  int m, n;
  int nt, ktp;     // tile counts; ktp = 128-k tiles per 16-row block as stored (multiple of TPW)
  int chunks;      // scale chunks per 16-row block
  int chunk_div;   // GM128: tiles per scale chunk (group_size / 128)
  int k_pad;       // row stride of xh / xl, = ktp * 128
  int y_dtype;
  int ksg;
  int epi;         // EPI_STORE / EPI_ADD_F32 / EPI_SWIGLU
  int slices;      // ktp / TPW: number of wave-sized k slices that exist
  // RMSNorm folded into the projections around it (NormFold in kernels.hpp); all null / 0 when unused
  const float *gamma_next;  // producer: scale vector of the norm that follows the residual update
  const float *pre;         // producer: power of two per row, [m]
  _Float16 *xg;             // producer: fp16(h_new * gamma_next * pre[row]), [m][n]
  float *ss_out;            // producer: sums of h_new^2 per row and 16-column block, [m][ss_out_stride]
  int ss_out_stride;
  const float *ss_in;       // consumer: partial sums of squares of the rows it multiplies, [m][ss_in_stride]
  const float *pre_in;      // consumer: what the rows of its activations were multiplied by, [m]
  float *pre_next;          // consumer, may be null: power of two per row for the residual update behind this norm
  int ss_in_count, ss_in_stride;
  float ss_inv_d, ss_eps;
};

// Scales of one (tile, row) kept in their storage type until used: 1, 2 or 4 values.
template <int GM, bool SF16>
struct ScaleRaw {
  static constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  typedef typename std::conditional<SF16, _Float16, float>::type elem_t;
  typedef elem_t vec_t __attribute__((ext_vector_type(SPT)));
  vec_t v;
  __device__ __forceinline__ void load(const char *p) { v = *reinterpret_cast<const vec_t *>(p); }
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
};

template <int GM>
__device__ __forceinline__ uint32_t load_zp_raw(const uint8_t *p) {
  constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  if constexpr (SPT == 4) return *reinterpret_cast<const uint32_t *>(p);
  if constexpr (SPT == 2) return *reinterpret_cast<const uint16_t *>(p);
  return *p;
}

// One wave's registers for one 16-row block: TPW weight tiles + their scales / zero points.
template <int GM, bool SF16, bool HAS_ZP>
struct TileRegs {
  uint4_t w[TPW];
  ScaleRaw<GM, SF16> s[TPW];
  uint32_t z[HAS_ZP ? TPW : 1];
};


__device__ __forceinline__ void zp_consts(uint32_t zp, half2_t &c1, half2_t &c2) {
  const _Float16 z = (_Float16)(float)zp;
  const _Float16 a = (_Float16)(-1024.0f) - z;
  const _Float16 b = (_Float16)(-64.0f) - z;
  c1 = half2_t{a, a};
  c2 = half2_t{b, b};
}

// 16-row blocks whose partial sums cross the waves together (must divide the ring depth).  Four at a time measured
// best for every m; two at a time is slower than one for m <= 4, where only two waves would have a piece to add.
// LDS staging of the raw-f32 path for at most four rows: per wave, fp16 hi then lo parts of 4 rows x 512 k; rows are
// 64 bytes apart modulo the bank cycle so the sixteen lanes that carry a row read conflict-free
constexpr int kStageRow = 512 * 2 + 64, kStageWave = 2 * 4 * kStageRow;
constexpr int skinny_ub(int ni, int p) { return p % 4 == 0 ? 4 : (p % 2 == 0 && ni > 1 ? 2 : 1); }

// XM: where the activations come from -- 0 prepared fp16 (hi [+ lo]), 1 raw f32 (split into hi + lo here), 2 raw bf16
template <int SPLIT, int NI, int GM, bool SF16, bool HAS_ZP, int P, int XM>
__global__ void __launch_bounds__(512, 1) int4_skinny_kernel(SkinnyArgs a) {
  constexpr bool RAWX = XM != 0;
  static_assert(XM != 1 || SPLIT == 2, "raw f32 activations are split into hi + lo");
  static_assert(XM != 2 || SPLIT == 1, "bf16 activations fit one fp16 operand exactly");
  // OFFSET mode: leave the 1024-offsets in the weights and cancel them per group (see file header)
  constexpr bool OFFSET = (SPLIT == 1) && !HAS_ZP;
  constexpr int UB = skinny_ub(NI, P);  // 16-row blocks per cross-wave reduction
  constexpr bool OFFSET1 = OFFSET && NI == 1;  // one useful accumulator: offset subtracted after the MFMA
  constexpr bool OFFSETC = OFFSET && NI > 1;   // all four useful: minus-offset enters as the MFMA's C operand
  constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  constexpr int SC_BYTES = SPT * (SF16 ? 2 : 4);
  extern __shared__ float red[];  // [2][waves][UB][NI][64]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves = blockDim.x >> 6;
  const int r = lane & 15;
  const int c = lane >> 4;
  const int slice = blockIdx.y * waves + wave;     // this wave's 512-k slice
  const bool wave_active = slice < a.slices;       // trailing waves of the last k-split may be idle
  const int t0 = (wave_active ? slice : 0) * TPW;  // first 128-k tile of the slice
  NibbleConsts nc;
  nc.init();

  // ---- per-wave stream pointers (advance by one grid stride of 16-row blocks per iteration) ----
  const int stride = gridDim.x;
  const size_t w_step = (size_t)stride * a.ktp * kTileBytes;
  const size_t s_step = (size_t)stride * a.chunks * 16 * SC_BYTES;
  const size_t z_step = (size_t)stride * a.chunks * 16 * SPT;
  const char *wp = reinterpret_cast<const char *>(a.tiles) + ((size_t)blockIdx.x * a.ktp + t0) * kTileBytes + lane * 16;
  const int chunk0 = GM == GM128 ? t0 / a.chunk_div : t0;
  const char *sp = reinterpret_cast<const char *>(a.tscales) + (((size_t)blockIdx.x * a.chunks + chunk0) * 16 + r) * SC_BYTES;
  const uint8_t *zp = HAS_ZP ? a.tzps + (((size_t)blockIdx.x * a.chunks + chunk0) * 16 + r) * SPT : nullptr;

  using Regs = TileRegs<GM, SF16, HAS_ZP>;

  // issue the loads of the block `ahead` grid strides after the current one
  auto issue = [&](Regs &tr, int ahead) {
    const char *wq = wp + (size_t)ahead * w_step;
    const char *sq = sp + (size_t)ahead * s_step;
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      tr.w[t] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(wq + t * kTileBytes));
      const int ch = GM == GM128 ? ((t0 + t) / a.chunk_div - chunk0) : t;
      tr.s[t].load(sq + (size_t)ch * 16 * SC_BYTES);
      if constexpr (HAS_ZP) tr.z[t] = load_zp_raw<GM>(zp + (size_t)ahead * z_step + (size_t)ch * 16 * SPT);
    }
  };

  auto advance = [&]() {
    wp += w_step;
    sp += s_step;
    if constexpr (HAS_ZP) zp += z_step;
  };

  // ---- the first P blocks are requested before the activation set-up (EARLY, where the registers allow it: their
  // HBM latency then overlaps the set-up) or right after it ----
  // Block `it` of this workgroup is 16-row block blockIdx.x + it * stride.  Requests past the last block are clamped
  // to it (a repeat served by the caches) so that every iteration issues the same number of loads and the
  // compiler's s_waitcnt counts stay exact.
  constexpr bool EARLY = (SPLIT == 1 || (XM == 1 && NI == 1)) && !HAS_ZP;
  const int iters = (a.nt - (int)blockIdx.x + stride - 1) / stride;  // >= 1, uniform in the workgroup
  Regs ring[P];
  auto fill_ring = [&]() {
    if (wave_active) {
#pragma unroll
      for (int sl = 0; sl < P; sl++) issue(ring[sl], sl < iters ? sl : iters - 1);
    }
  };
  if constexpr (EARLY) fill_ring();
  // folded norm, consumer side: this wave's share of the partial sums of squares (see further down), requested
  // here so that their round trip overlaps the activations'
  constexpr int kSsRowsPerWave = 4;  // rows wave, wave + waves, ...: the launcher checks that four per wave cover m
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  float ss_pre[kSsRowsPerWave][4], ss_scale[kSsRowsPerWave];
  if (a.ss_in) {
#pragma unroll
    for (int u = 0; u < kSsRowsPerWave; u++) {
      const int row = wave_u + u * waves;
      ss_scale[u] = a.pre_in[min(row, a.m - 1)];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int j = 4 * lane + e;
        ss_pre[u][e] = (row < a.m && j < a.ss_in_count) ? a.ss_in[(size_t)row * a.ss_in_stride + j] : 0.0f;
      }
    }
  }

  // folded norm, producer side: the residual values and the gammas this wave's first two pieces of the first
  // reduction will need, requested now (their round trip would otherwise sit at the end of a one-block kernel)
  // (only in the instantiations with a ring of one or two blocks, where a residual update of a decode step lands and
  // registers are to spare)
  constexpr bool PREFETCH_H = P <= 2;
  float h_pre[2] = {0.0f, 0.0f}, g_pre[2] = {0.0f, 0.0f}, p_pre[2] = {0.0f, 0.0f};
  if (PREFETCH_H && a.xg) {
#pragma unroll
    for (int sl = 0; sl < 2; sl++) {
      const int q = wave_u + sl * waves;
      if (q < UB * NI) {  // uniform in the wave
        const int u = q / NI, i = q % NI;
        const int col = ((int)blockIdx.x + u * stride) * 16 + r;
        const int mrow = c * NI + i;
        if (col < a.n) g_pre[sl] = a.gamma_next[col];
        if (mrow < a.m && col < a.n) {
          h_pre[sl] = reinterpret_cast<const float *>(a.y)[(size_t)mrow * a.n + col];
          p_pre[sl] = a.pre[mrow];
        }
      }
    }
  }

  // ---- activations -> registers, in A-operand order ------------------------------------------
  // MFMA row `r` carries batch row m when r == 4*(m / NI) + (m % NI): the useful results then sit
  // in the first NI of the four accumulator registers of each lane.
  half8_t xa[TPW][4][SPLIT];
  float slice_scale = 1.0f;  // RAWX: what this wave's products of the row it loads must be multiplied by
  {
    const int i = r & 3;
    const int mrow = (r >> 2) * NI + i;
    const bool valid = wave_active && (i < NI) && (mrow < a.m);
    const half8_t pre = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)0.0625f, (_Float16)0.0625f,
                         (_Float16)1.0f, (_Float16)1.0f, (_Float16)0.0625f, (_Float16)0.0625f};
    if constexpr (XM == 2) {
      // bf16 activations straight from the caller: the wave scales its own 512-k slice of every row by a power of
      // two (abs-max to [2^14, 2^15)), which makes every bf16 value an exact fp16 one (8 significant bits; only
      // values below 2^-29 of the slice maximum are lost); the power of two is undone on the wave's partial sums.
      const uint16_t *src = a.xb + (size_t)(valid ? mrow : 0) * a.k_pad + (size_t)t0 * 128 + c * 8;
      uint4_t raw[TPW][4];
#pragma unroll
      for (int t = 0; t < TPW; t++)
#pragma unroll
        for (int j = 0; j < 4; j++) raw[t][j] = *reinterpret_cast<const uint4_t *>(src + t * 128 + j * 32);
      uint32_t amax_bits = 0;  // |bf16| orders like its bit pattern
#pragma unroll
      for (int t = 0; t < TPW; t++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const uint32_t wd = raw[t][j][e];
            const uint32_t lo = wd & 0x7FFFu, hi = (wd >> 16) & 0x7FFFu;
            amax_bits = max(amax_bits, max(lo, hi));
          }
      float amax = valid ? __uint_as_float(amax_bits << 16) : 0.0f;
      amax = max_xor16_xor32(amax);
      int e2 = 14;
      if (amax > 0.0f && amax < 3.0e38f) {
        (void)frexpf(amax, &e2);
        e2 -= 1;
      }
      int shift = 14 - e2;
      shift = shift > 100 ? 100 : (shift < -100 ? -100 : shift);
      const float up = valid ? ldexpf(1.0f, shift) : 0.0f;
      slice_scale = ldexpf(1.0f, -shift);
#pragma unroll
      for (int t = 0; t < TPW; t++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          half8_t h;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const uint32_t wd = raw[t][j][e];
            h[2 * e] = (_Float16)(__uint_as_float(wd << 16) * up);
            h[2 * e + 1] = (_Float16)(__uint_as_float(wd & 0xFFFF0000u) * up);
          }
          if (!valid) h = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
          if constexpr (OFFSET) h = h * pre;
          xa[t][j][0] = h;
        }
      }
    } else if constexpr (XM == 1 && NI == 1) {
      // f32 activations straight from the caller, at most four rows: converting them in the operand layout would
      // have every lane convert 128 values although only a quarter of the lanes carry a row.  Instead lane L converts
      // 32 values (row L / 16, 32-k block L % 16) and the fp16 hi + lo parts change places through this wave's own
      // piece of LDS.  As below, the wave normalises its 512-k slice of every row by a power of two, undone on its
      // partial sums.  Lanes without a row read row 0 and discard it (unconditional loads: one round trip for all).
      const int srow = lane >> 4, q = lane & 15;
      const bool svalid = wave_active && srow < a.m;
      const float *src = a.xf + (size_t)(svalid ? srow : 0) * a.k_pad + (size_t)t0 * 128 + q * 32;
      float4_t raw[8];
#pragma unroll
      for (int e = 0; e < 8; e++) raw[e] = *reinterpret_cast<const float4_t *>(src + 4 * e);
      float amax = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; e++)
#pragma unroll
        for (int u = 0; u < 4; u++) amax = fmaxf(amax, fabsf(raw[e][u]));
      if (!svalid) amax = 0.0f;
      amax = row_max16(amax);
      int e2 = 14;
      if (amax > 0.0f && amax < 3.0e38f) {
        (void)frexpf(amax, &e2);
        e2 -= 1;
      }
      int shift = 14 - e2;
      shift = shift > 100 ? 100 : (shift < -100 ? -100 : shift);
      const float up = svalid ? ldexpf(1.0f, shift) : 0.0f;
      slice_scale = ldexpf(1.0f, -shift);
      unsigned char *stage = reinterpret_cast<unsigned char *>(red) + (size_t)2 * waves * UB * NI * 64 * sizeof(float) +
                             (size_t)wave * kStageWave;
#pragma unroll
      for (int cc = 0; cc < 4; cc++) {
        half8_t h, l;
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float sv = (e < 4 ? raw[2 * cc][e] : raw[2 * cc + 1][e - 4]) * up;
          h[e] = (_Float16)sv;
          l[e] = (_Float16)(sv - (float)h[e]);
        }
        *reinterpret_cast<half8_t *>(stage + srow * kStageRow + (q * 32 + cc * 8) * 2) = h;
        *reinterpret_cast<half8_t *>(stage + 4 * kStageRow + srow * kStageRow + (q * 32 + cc * 8) * 2) = l;
      }
      // the wave reads what its own lanes wrote: LDS serves a wave's accesses in order, the compiler must not reorder
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      const half8_t hz = {0, 0, 0, 0, 0, 0, 0, 0};
      const unsigned char *rd = stage + (r >> 2) * kStageRow + c * 16;  // lanes without a row share a neighbour's address
#pragma unroll
      for (int t = 0; t < TPW; t++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const half8_t h = *reinterpret_cast<const half8_t *>(rd + (t * 4 + j) * 64);
          const half8_t l = *reinterpret_cast<const half8_t *>(rd + 4 * kStageRow + (t * 4 + j) * 64);
          xa[t][j][0] = valid ? h : hz;
          xa[t][j][1] = valid ? l : hz;
        }
      }
    } else if constexpr (XM == 1) {
      // f32 activations straight from the caller: the wave normalises its own 512-k slice of every row by a power
      // of two (abs-max to [2^14, 2^15), as the separate activation pass does per row) and splits it into fp16
      // hi + lo; the power of two is undone on the wave's partial sums before they meet the other slices.
      // Idle lanes read row 0 and discard it: every load is unconditional, so all of them are in flight together
      // instead of one round trip per guarded load.
      const float *src = a.xf + (size_t)(valid ? mrow : 0) * a.k_pad + (size_t)t0 * 128 + c * 8;
      float amax = 0.0f;
#pragma unroll
      for (int t = 0; t < TPW; t++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float4_t v0 = *reinterpret_cast<const float4_t *>(src + t * 128 + j * 32);
          const float4_t v1 = *reinterpret_cast<const float4_t *>(src + t * 128 + j * 32 + 4);
#pragma unroll
          for (int e = 0; e < 4; e++) amax = fmaxf(amax, fmaxf(fabsf(v0[e]), fabsf(v1[e])));
        }
      if (!valid) amax = 0.0f;
      amax = max_xor16_xor32(amax);
      int e2 = 14;
      if (amax > 0.0f && amax < 3.0e38f) {
        (void)frexpf(amax, &e2);
        e2 -= 1;
      }
      int shift = 14 - e2;
      shift = shift > 100 ? 100 : (shift < -100 ? -100 : shift);
      const float up = valid ? ldexpf(1.0f, shift) : 0.0f;
      slice_scale = ldexpf(1.0f, -shift);
#pragma unroll
      for (int t = 0; t < TPW; t++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          // second read of the slice: served by the caches
          const float4_t v0 = *reinterpret_cast<const float4_t *>(src + t * 128 + j * 32);
          const float4_t v1 = *reinterpret_cast<const float4_t *>(src + t * 128 + j * 32 + 4);
          half8_t h, l;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float sv = (e < 4 ? v0[e] : v1[e - 4]) * up;
            h[e] = (_Float16)sv;
            l[e] = (_Float16)(sv - (float)h[e]);
          }
          if (!valid) {
            h = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            l = h;
          }
          xa[t][j][0] = h;
          xa[t][j][1] = l;
        }
      }
    } else {
      const size_t row_off = (size_t)(valid ? mrow : 0) * a.k_pad;
      const half8_t hz = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int t = 0; t < TPW; t++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const size_t off = row_off + (size_t)(t0 + t) * 128 + j * 32 + c * 8;
          half8_t h = *reinterpret_cast<const half8_t *>(a.xh + off);
          if (!valid) h = hz;
          if constexpr (OFFSET) h = h * pre;  // slots that meet 1024 + 16 q carry x / 16 (a power of two)
          xa[t][j][0] = h;
          if constexpr (SPLIT == 2) {
            half8_t l = *reinterpret_cast<const half8_t *>(a.xl + off);
            xa[t][j][1] = valid ? l : hz;
          }
        }
      }
    }
  }
  // Folded RMSNorm, consumer side: the row factors 1 / (pre * sqrt(sum(h^2) / d + eps)) come from the partial sums
  // the kernel that wrote the residual left behind and from the power of two it scaled the row with.  Row q is added
  // up by wave q % waves (four consecutive partials per lane, requested further up together with the activations,
  // then a fixed tree of DPP moves and lane swaps: the same order in every run); the sixteen factors meet in LDS
  // behind the barrier of the first reduction, which every use of them follows.
  float *rs_lds = red + (size_t)2 * waves * (UB * NI) * 64;
  if (a.ss_in) {
#pragma unroll
    for (int u = 0; u < kSsRowsPerWave; u++) {
      const int row = wave_u + u * waves;
      if (row < a.m) {  // uniform in the wave
        const float t = wave_sum((ss_pre[u][0] + ss_pre[u][1]) + (ss_pre[u][2] + ss_pre[u][3]));
        const float inv_rms = 1.0f / sqrtf(t * a.ss_inv_d + a.ss_eps);
        if (lane == 0) {
          rs_lds[row] = inv_rms / ss_scale[u];
          // one workgroup leaves the scale of the next residual update behind (every workgroup holds the same bits)
          if (a.pre_next && blockIdx.x == 0 && blockIdx.y == 0) a.pre_next[row] = norm_fold_prescale(inv_rms);
        }
      }
    }
  }

  // RAWX: accumulator i of lane (c, .) belongs to row c * NI + i, which lanes 4 c + i (+16, +32, +48) loaded
  float acc_scale[NI];
#pragma unroll
  for (int i = 0; i < NI; i++)
    acc_scale[i] = RAWX ? __shfl(slice_scale, (XM == 1 && NI == 1) ? 16 * c : 4 * c + i, 64) : 1.0f;
  // offset term of every 32-k block: sum_k x'_k * (1024 + 8 | 1024 + 128), same register layout as D
  float corr1[OFFSET1 ? TPW : 1][4];
  // OFFSETC: minus the offset term of MFMA row r and 32-k block (t, j = c), i.e. in the A-operand layout of
  // v_mfma_f32_16x16x4_f32: at the end of a 16-row block, four of those MFMAs (one per tile, B = the scale that
  // applies to weight row r in 32-k block c) add sum_blocks -offset * scale to all four accumulators at once.
  float ncorr_a[OFFSETC ? TPW : 1];
  if constexpr (OFFSET) {
    const half8_t bc = {(_Float16)1032.0f, (_Float16)1032.0f, (_Float16)1152.0f, (_Float16)1152.0f,
                        (_Float16)1032.0f, (_Float16)1032.0f, (_Float16)1152.0f, (_Float16)1152.0f};
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      float sel = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float4_t z = {0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (OFFSET1) {
          z = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][j][0], bc, z, 0, 0, 0);
          corr1[t][j] = z[0];
        } else {
          // operands swapped: the activations are the B matrix, so column r of the result (every register of lanes
          // (r, .)) is the offset term of MFMA row r
          z = __builtin_amdgcn_mfma_f32_16x16x32_f16(bc, xa[t][j][0], z, 0, 0, 0);
          if (c == j) sel = z[0];
        }
      }
      if constexpr (OFFSETC) ncorr_a[t] = -sel;
    }
  }

  if constexpr (!EARLY) fill_ring();

  // dot products of one 16-row block against this wave's k slice
  auto dots = [&](const Regs &tr, float acc[NI]) {
#pragma unroll
    for (int i = 0; i < NI; i++) acc[i] = 0.0f;
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      if constexpr (GM == GM32 && SPLIT == 1) {
        // one group per 32-k block: the four MFMAs of a tile are issued before the first result is consumed, so the
        // scale FMAs of one block never wait for its own MFMA
        float4_t dd[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          half8_t b;
          if constexpr (OFFSET) {
            b = extract8(tr.w[t][j], nc);
          } else {
            half2_t c1 = {(_Float16)(-1032.0f), (_Float16)(-1032.0f)};
            half2_t c2 = {(_Float16)(-72.0f), (_Float16)(-72.0f)};
            if constexpr (HAS_ZP) zp_consts((tr.z[t] >> (8 * j)) & 0xFF, c1, c2);
            b = decode8_exact(tr.w[t][j], nc, c1, c2);
          }
          dd[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][j][0], b, float4_t{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float sc = tr.s[t].get(j);
          if constexpr (OFFSET1) {
            acc[0] = fmaf(sc, dd[j][0] - corr1[t][j], acc[0]);
          } else {
#pragma unroll
            for (int i = 0; i < NI; i++) acc[i] = fmaf(sc, dd[j][i], acc[i]);
          }
        }
        continue;
      }
      float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
      float csum = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const bool group_start = GM == GM32 || (GM == GM64 && !(j & 1)) || (GM == GM128 && j == 0);
        const bool group_end = GM == GM32 || (GM == GM64 && (j & 1)) || (GM == GM128 && j == 3);
        half8_t b;
        if constexpr (OFFSET) {
          b = extract8(tr.w[t][j], nc);
          if constexpr (OFFSET1) csum = group_start ? corr1[t][j] : csum + corr1[t][j];
        } else {
          half2_t c1 = {(_Float16)(-1032.0f), (_Float16)(-1032.0f)};
          half2_t c2 = {(_Float16)(-72.0f), (_Float16)(-72.0f)};
          if constexpr (HAS_ZP) {
            const uint32_t z = GM == GM32 ? ((tr.z[t] >> (8 * j)) & 0xFF)
                                          : (GM == GM64 ? ((tr.z[t] >> (8 * (j >> 1))) & 0xFF) : (tr.z[t] & 0xFF));
            zp_consts(z, c1, c2);
          }
          b = decode8_exact(tr.w[t][j], nc, c1, c2);
        }
        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][j][0], b, d, 0, 0, 0);
        if constexpr (SPLIT == 2) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][j][1], b, d, 0, 0, 0);
        if (group_end) {
          const float sc = tr.s[t].get(GM == GM32 ? j : (GM == GM64 ? (j >> 1) : 0));
          if constexpr (OFFSET1) {
            acc[0] = fmaf(sc, d[0] - csum, acc[0]);
          } else {
#pragma unroll
            for (int i = 0; i < NI; i++) acc[i] = fmaf(sc, d[i], acc[i]);
          }
          d = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
      }
    }
    if constexpr (OFFSETC) {
      float4_t av = {acc[0], NI > 1 ? acc[1 % NI] : 0.0f, NI > 2 ? acc[2 % NI] : 0.0f, NI > 3 ? acc[3 % NI] : 0.0f};
#pragma unroll
      for (int t = 0; t < TPW; t++) {
        const float sb = tr.s[t].get(GM == GM32 ? c : (GM == GM64 ? (c >> 1) : 0));
        av = __builtin_amdgcn_mfma_f32_16x16x4f32(ncorr_a[t], sb, av, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < NI; i++) acc[i] = av[i];
    }
    if constexpr (RAWX) {
#pragma unroll
      for (int i = 0; i < NI; i++) acc[i] *= acc_scale[i];
    }
  };

  // row scales of the activation pass, one per accumulator of this lane (loaded once: a load inside the loop
  // would make the compiler wait for every weight block in flight)
  float4_t rs = {1.0f, 1.0f, 1.0f, 1.0f};  // (a vector: an array here ended up in scratch memory once the epilogues grew)
  if (a.row_scale) {  // one branch around all of them: rows past m read the last row's scale and are never stored
#pragma unroll
    for (int i = 0; i < NI; i++) rs[i] = a.row_scale[min(c * NI + i, a.m - 1)];
  }

  // Meet the other k slices in LDS, once per UB blocks: every wave leaves its UB x NI x 64 partial sums, and after
  // one barrier the sums are shared out over the waves in 64-lane pieces (piece q = block q / NI of the group,
  // accumulator q % NI), rotating so that no wave is always the late one.
  // the wave index as the scalar it is (the compiler takes anything derived from threadIdx for a per-lane value, and
  // the piece loop below would then run under exec masks with its indices in vector registers)
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  int exm = 0;  // reductions done so far, modulo the number of waves: rotates the piece-to-wave assignment

  auto reduce_store = [&](const float (&accs)[UB][NI], int nt0, int ex) {
    float *buf = red + (size_t)(ex & 1) * waves * (UB * NI) * 64;
    {
      float *wb = buf + wave * (UB * NI) * 64 + lane;
#pragma unroll
      for (int u = 0; u < UB; u++)
#pragma unroll
        for (int i = 0; i < NI; i++) wb[(u * NI + i) * 64] = accs[u][i];
    }
    lds_barrier();
    // epilogue of one finished 64-lane piece q = u * NI + i: block u of the group, accumulator i
    auto finish = [&](float v, int q, int slot) {
      const int u = q / NI, i = q % NI;
      const int col = (nt0 + u * stride) * 16 + r;
      const int mrow = c * NI + i;
      const bool live = mrow < a.m && col < a.n;
      if (a.ksg > 1) {
        if (live) a.partial[((size_t)blockIdx.y * a.m + mrow) * a.n + col] = v;
      } else {
        float rsv = rs[0];
#pragma unroll
        for (int ii = 1; ii < NI; ii++) rsv = (i == ii) ? rs[ii] : rsv;
        if (a.ss_in) rsv = rs_lds[min(mrow, a.m - 1)];
        v *= rsv;
        if (a.epi == EPI_ADD_F32 && a.xg) {
          // residual update that also feeds the next norm: h_new, its fp16 image times gamma and the row's power of
          // two, and the sum of h_new^2 over the sixteen columns of this block (the lanes r = 0..15 of a lane group),
          // one per row
          float hn = 0.0f;
          if (live) {
            float *hp = reinterpret_cast<float *>(a.y) + (size_t)mrow * a.n + col;
            const bool pre = PREFETCH_H && ex == 0 && slot >= 0 && slot < 2;  // requested at the start of the kernel
            const float hold = pre ? (slot == 0 ? h_pre[0] : h_pre[1]) : *hp;
            const float gam = pre ? (slot == 0 ? g_pre[0] : g_pre[1]) : a.gamma_next[col];
            const float pw = pre ? (slot == 0 ? p_pre[0] : p_pre[1]) : a.pre[mrow];
            hn = hold + v;
            *hp = hn;
            const float gx = fminf(fmaxf(hn * gam * pw, -65504.0f), 65504.0f);
            a.xg[(size_t)mrow * a.n + col] = (_Float16)gx;
          }
          const float sq = row_sum16(hn * hn);
          if (r == 0 && mrow < a.m && (nt0 + u * stride) < a.nt) a.ss_out[(size_t)mrow * a.ss_out_stride + (nt0 + u * stride)] = sq;
          return;
        }
        if (a.epi == EPI_SWIGLU) {
          // rows 2i / 2i+1 of the weight are gate_i / up_i: neighbours in the wave
          const float up = dpp_move<DPP_XOR1>(v);
          if (live && !(r & 1))
            store_out(a.y, (size_t)mrow * (a.n >> 1) + (col >> 1), silu(v) * up, a.y_dtype);
        } else if (a.epi == EPI_ADD_F32) {
          // single writer per element: a returnless add keeps the residual update off the load queue
          if (live) unsafeAtomicAdd(reinterpret_cast<float *>(a.y) + (size_t)mrow * a.n + col, v);
        } else if (live) {
          store_out(a.y, (size_t)mrow * a.n + col, v, a.y_dtype);
        }
      }
    };
    int q = wave_s + exm;
    if (q >= waves) q -= waves;
    exm = exm + 1 == waves ? 0 : exm + 1;
    // slice w of piece q sits at buf[(w * UB * NI + q) * 64 + lane]: one base per piece, constant offsets per slice
    if (waves == 8 && UB * NI == 16) {
      // the usual shape, two pieces per wave (q and q + 8): all sixteen slices are requested in one go (one LDS round
      // trip per reduction instead of four), then added in slice order
      const float *rb = buf + q * 64 + lane;
      float p0[8], p1[8];
#pragma unroll
      for (int w = 0; w < 8; w++) {
        p0[w] = rb[w * (UB * NI) * 64];
        p1[w] = rb[w * (UB * NI) * 64 + 8 * 64];
      }
      float v0 = 0.0f, v1 = 0.0f;
#pragma unroll
      for (int w = 0; w < 8; w++) {
        v0 += p0[w];
        v1 += p1[w];
      }
      finish(v0, q, 0);
      finish(v1, q + 8, 1);
      return;
    }
    for (int slot = 0; q < UB * NI; q += waves, slot++) {
      const float *rb = buf + q * 64 + lane;
      float v = 0.0f;
      if (waves == 8) {  // all eight slices in one LDS round trip
        float part[8];
#pragma unroll
        for (int w = 0; w < 8; w++) part[w] = rb[w * (UB * NI) * 64];
#pragma unroll
        for (int w = 0; w < 8; w++) v += part[w];
      } else {
#pragma unroll
        for (int w0 = 0; w0 < 8; w0 += 4) {  // four slices at a time: two LDS round trips, few registers
          float part[4];
#pragma unroll
          for (int w = 0; w < 4; w++) part[w] = w0 + w < waves ? rb[(w0 + w) * (UB * NI) * 64] : 0.0f;
#pragma unroll
          for (int w = 0; w < 4; w++) v += part[w];
        }
      }
      finish(v, q, slot);
    }
  };

  // ---- main loop: slot it % P holds block it; after its dot products the slot is refilled with block it + P ----
  int nt = blockIdx.x;  // first block of the current group of UB
  int it = 0, ex = 0;
  float accs[UB][NI];

  if (!wave_active) {
    // an idle wave only takes part in the reductions
#pragma unroll
    for (int u = 0; u < UB; u++)
#pragma unroll
      for (int i = 0; i < NI; i++) accs[u][i] = 0.0f;
    for (; it < iters; it += UB, nt += UB * stride, ex++) reduce_store(accs, nt, ex);
    return;
  }

  const int steady = (iters + P - 1) / P - 1;  // groups of P iterations that refill; the last group only drains
  for (int g = 0; g < steady; g++) {
#pragma unroll
    for (int sl = 0; sl < P; sl++) {
      dots(ring[sl], accs[sl % UB]);
      const int left = iters - 1 - it;  // blocks after this one (>= P - sl, as one more group follows)
      issue(ring[sl], left < P ? left : P);
      if (sl % UB == UB - 1) {
        reduce_store(accs, nt, ex);
        nt += UB * stride;
        ex++;
      }
      advance();
      it++;
    }
  }
#pragma unroll
  for (int sl = 0; sl < P; sl++) {
    if (it < iters) {
      dots(ring[sl], accs[sl % UB]);
    } else {
#pragma unroll
      for (int i = 0; i < NI; i++) accs[sl % UB][i] = 0.0f;
    }
    if (sl % UB == UB - 1) {
      if (it - (UB - 1) < iters) reduce_store(accs, nt, ex);  // the group's first block exists
      nt += UB * stride;
      ex++;
    }
    it++;
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
    // issue the loads of this element together (one memory round trip), the residual it is added to included, then
    // add in slice order
    float p[8];
#pragma unroll
    for (int s = 0; s < 8; s++) p[s] = s < ksg ? partial[(size_t)s * total + idx] : 0.0f;
    const float before = epi == EPI_ADD_F32 ? reinterpret_cast<const float *>(y)[idx] : 0.0f;
    float v = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; s++) v += p[s];
    for (int s = 8; s < ksg; s++) v += partial[(size_t)s * total + idx];
    if (row_scale) v *= row_scale[idx / n];
    if (epi == EPI_ADD_F32) {
      reinterpret_cast<float *>(y)[idx] = before + v;
    } else {
      store_out(y, idx, v, y_dtype);
    }
  }
}

// The second pass of a K-split residual update that also feeds the next norm (NormFold): one workgroup per (row, 256
// columns); h += sum of the partials in slice order, xg = fp16(h * gamma * pre[row]), and the sum of h^2 over the 256 columns
// (fixed order: shuffle tree per wave, then the four waves in turn) as one partial of the row.  n % 256 == 0.
__global__ void __launch_bounds__(256) int4_skinny_finalize_norm_kernel(const float *__restrict__ partial, int ksg, int m, int n,
                                                                        float *__restrict__ h, const float *__restrict__ gamma,
                                                                        const float *__restrict__ pre, _Float16 *__restrict__ xg, float *__restrict__ ss_out,
                                                                        int ss_stride) {
  __shared__ float red4[4];
  const int chunks = n >> 8;
  const int row = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
  const size_t total = (size_t)m * n;
  const size_t idx = (size_t)row * n + (size_t)chunk * 256 + threadIdx.x;
  float p[8];
#pragma unroll
  for (int s = 0; s < 8; s++) p[s] = s < ksg ? partial[(size_t)s * total + idx] : 0.0f;
  const float before = h[idx];
  const float g = gamma[chunk * 256 + threadIdx.x] * pre[row];
  float v = 0.0f;
#pragma unroll
  for (int s = 0; s < 8; s++) v += p[s];
  for (int s = 8; s < ksg; s++) v += partial[(size_t)s * total + idx];
  const float hn = before + v;
  h[idx] = hn;
  xg[idx] = (_Float16)fminf(fmaxf(hn * g, -65504.0f), 65504.0f);
  const float sq = wave_sum(hn * hn);
  if ((threadIdx.x & 63) == 0) red4[threadIdx.x >> 6] = sq;
  __syncthreads();
  if (threadIdx.x == 0) ss_out[(size_t)row * ss_stride + chunk] = ((red4[0] + red4[1]) + red4[2]) + red4[3];
}

SkinnyPlan plan_int4_skinny(const yscv_hip_int4_weight *w, size_t m, int split, int num_cus) {
  (void)split;
  SkinnyPlan p;
  p.tpw = TPW;
  const int max_waves = 8;  // 8 waves x <= 256 VGPRs: one workgroup per CU
  const int slices = (int)(w->ktp / TPW);
  p.ksg = (int)ceil_div((size_t)slices, (size_t)max_waves);
  p.waves = (int)ceil_div((size_t)slices, (size_t)p.ksg);
  int gx = (int)w->nt;
  const int cap = num_cus > 0 ? num_cus : 256;
  // one resident workgroup per CU and k-split slice; more blocks than that loop inside the kernel
  int per = cap / p.ksg;
  if (per < 1) per = 1;
  if (gx > per) {
    const int rounds = (int)ceil_div((size_t)gx, (size_t)per);
    gx = (int)ceil_div((size_t)w->nt, (size_t)rounds);  // spread the blocks evenly
  }
  p.grid_x = gx;
  p.partial_bytes = p.ksg > 1 ? (size_t)p.ksg * m * w->n * sizeof(float) : 0;
  return p;
}

template <int SPLIT, int NI, int GM, bool SF16, bool HAS_ZP, int P>
static int32_t launch_p(const SkinnyArgs &a, const SkinnyPlan &plan, hipStream_t s) {
  constexpr int UB = skinny_ub(NI, P);
  const size_t lds = (size_t)2 * plan.waves * UB * NI * 64 * sizeof(float) + 64;  // + the sixteen row factors of a folded norm
  if constexpr (SPLIT == 2) {
    if (a.xf != nullptr) {
      const size_t stage = NI == 1 ? (size_t)plan.waves * kStageWave : 0;
      if (stage > 0) {  // 8 waves: 68 KB, above the default dynamic-LDS limit
        static std::once_flag once;
        static hipError_t attr_err = hipSuccess;
        std::call_once(once, [] {
          attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(int4_skinny_kernel<SPLIT, NI, GM, SF16, HAS_ZP, P, 1>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 8 * (2 * UB * NI * 64 * 4 + kStageWave) + 64);
        });
        if (attr_err != hipSuccess)
          return set_error(YSCV_HIP_ERR_DEVICE, "cannot reserve LDS for the activation staging: %s", hipGetErrorString(attr_err));
      }
      hipLaunchKernelGGL((int4_skinny_kernel<SPLIT, NI, GM, SF16, HAS_ZP, P, 1>), dim3(plan.grid_x, plan.ksg),
                         dim3(plan.waves * 64), lds + stage, s, a);
      YSCV_HIP_TRY(hipGetLastError());
      return YSCV_HIP_OK;
    }
  } else {
    if (a.xb != nullptr) {
      hipLaunchKernelGGL((int4_skinny_kernel<SPLIT, NI, GM, SF16, HAS_ZP, P, 2>), dim3(plan.grid_x, plan.ksg),
                         dim3(plan.waves * 64), lds, s, a);
      YSCV_HIP_TRY(hipGetLastError());
      return YSCV_HIP_OK;
    }
  }
  hipLaunchKernelGGL((int4_skinny_kernel<SPLIT, NI, GM, SF16, HAS_ZP, P, 0>), dim3(plan.grid_x, plan.ksg),
                     dim3(plan.waves * 64), lds, s, a);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

template <int SPLIT, int NI, int GM, bool SF16, bool HAS_ZP>
static int32_t launch_one(const SkinnyArgs &a, const SkinnyPlan &plan, hipStream_t s) {
  // ring depth: bounded by the VGPR budget (activations: 64 per split, ring: ~26 per slot)
  if constexpr (SPLIT == 2 && NI == 1) {
    // two slots fit only with a few spilled registers, whose cost a workgroup recovers over sixteen or more blocks
    const int blocks_per_wg = (a.nt + plan.grid_x - 1) / plan.grid_x;
    if (blocks_per_wg < 16) return launch_p<SPLIT, NI, GM, SF16, HAS_ZP, 1>(a, plan, s);
    return launch_p<SPLIT, NI, GM, SF16, HAS_ZP, 2>(a, plan, s);
  } else {
    constexpr int P = SPLIT == 2 ? 1 : (SF16 && !HAS_ZP ? 4 : 3);
    if constexpr (SPLIT == 1) {
      // A workgroup with one or two blocks (the short projections of a decode step) gets a ring of that depth: the
      // requests past the last block that keep a deeper ring's load count fixed are real instructions, each holds the
      // CU's memory pipeline for sixteen cycles whatever it asks for, and with one block three quarters of the ring
      // fill would be such fillers (2 of the 8 us of an output projection at m = 16).
      const int blocks_per_wg = (a.nt + plan.grid_x - 1) / plan.grid_x;
      if (blocks_per_wg == 1) return launch_p<SPLIT, NI, GM, SF16, HAS_ZP, 1>(a, plan, s);
      if (blocks_per_wg == 2) return launch_p<SPLIT, NI, GM, SF16, HAS_ZP, 2>(a, plan, s);
    }
    return launch_p<SPLIT, NI, GM, SF16, HAS_ZP, P>(a, plan, s);
  }
}

template <int SPLIT, int NI, int GM>
static int32_t launch_sz(const SkinnyArgs &a, const SkinnyPlan &plan, bool sf16, bool has_zp, hipStream_t s) {
  if (sf16)
    return has_zp ? launch_one<SPLIT, NI, GM, true, true>(a, plan, s) : launch_one<SPLIT, NI, GM, true, false>(a, plan, s);
  return has_zp ? launch_one<SPLIT, NI, GM, false, true>(a, plan, s) : launch_one<SPLIT, NI, GM, false, false>(a, plan, s);
}

template <int SPLIT, int NI>
static int32_t launch_gm(const SkinnyArgs &a, const SkinnyPlan &plan, int gm, bool sf16, bool has_zp, hipStream_t s) {
  if (gm == GM32) return launch_sz<SPLIT, NI, GM32>(a, plan, sf16, has_zp, s);
  if (gm == GM64) return launch_sz<SPLIT, NI, GM64>(a, plan, sf16, has_zp, s);
  return launch_sz<SPLIT, NI, GM128>(a, plan, sf16, has_zp, s);
}

int32_t launch_int4_skinny(const yscv_hip_int4_weight *w, const SkinnyPlan &plan, const _Float16 *xh,
                           const _Float16 *xl, const void *xraw, const float *row_scale, size_t k_pad, int split,
                           void *y, int y_dtype, size_t m, float *partial, int epi, hipStream_t s, const NormFold *nf) {
  if (!w->tiled) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "skinny int4 kernel needs the tiled layout");
  if (m == 0 || m > 16) return set_error(YSCV_HIP_ERR_INVALID_ARG, "skinny int4 kernel handles 1 <= m <= 16, got %zu", m);
  if (plan.ksg > 1 && !partial) return set_error(YSCV_HIP_ERR_INVALID_ARG, "k-split needs a partial buffer");
  if (k_pad != w->ktp * 128)
    return set_error(YSCV_HIP_ERR_INVALID_ARG, "activation row stride %zu != padded K %zu", k_pad, w->ktp * 128);
  SkinnyArgs a;
  a.tiles = w->tiles;
  a.tscales = w->tscales;
  a.tzps = w->has_zp ? w->tzps : nullptr;
  a.xh = xh;
  a.xl = xl;
  a.xf = split == 2 ? static_cast<const float *>(xraw) : nullptr;
  a.xb = split == 1 ? static_cast<const uint16_t *>(xraw) : nullptr;
  a.row_scale = row_scale;
  a.y = y;
  a.partial = partial;
  a.m = (int)m;
  a.n = (int)w->n;
  a.nt = (int)w->nt;
  a.ktp = (int)w->ktp;
  a.chunks = (int)w->chunks;
  a.chunk_div = w->gm == GM128 ? (int)(w->g / 128) : 1;
  a.k_pad = (int)k_pad;
  a.y_dtype = y_dtype;
  a.ksg = plan.ksg;
  a.epi = epi;
  a.slices = (int)(w->ktp / TPW);
  a.gamma_next = nullptr;
  a.xg = nullptr;
  a.pre = a.pre_in = nullptr;
  a.pre_next = nullptr;
  a.ss_out = nullptr;
  a.ss_out_stride = 0;
  a.ss_in = nullptr;
  a.ss_in_count = a.ss_in_stride = 0;
  a.ss_inv_d = a.ss_eps = 0.0f;
  const bool produce = nf && nf->xg != nullptr;
  if (produce && row_scale) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "folded norm: the producing call takes activations as they are");
  if (nf) {
    if (nf->ss_in) {
      if (plan.ksg > 1) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "folded norm: the consuming projection must not be K-split");
      if (m > (size_t)4 * plan.waves || nf->ss_in_count > 256)
        return set_error(YSCV_HIP_ERR_UNSUPPORTED, "folded norm: %zu rows on %d waves, %d partial sums per row", m, plan.waves, nf->ss_in_count);
      if (split != 1 || xraw) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "folded norm: fp16 activations only");
      if (!nf->pre_in) return set_error(YSCV_HIP_ERR_INVALID_ARG, "folded norm: the row scales of the activations are missing");
      a.ss_in = nf->ss_in;
      a.pre_in = nf->pre_in;
      a.pre_next = nf->pre_next;
      a.ss_in_count = nf->ss_in_count;
      a.ss_in_stride = nf->ss_in_stride;
      a.ss_inv_d = nf->inv_d;
      a.ss_eps = nf->eps;
    }
    if (produce) {
      if (epi != EPI_ADD_F32 || !nf->gamma_next || !nf->ss_out || !nf->ss_out_count || !nf->pre)
        return set_error(YSCV_HIP_ERR_INVALID_ARG, "folded norm: the producing call is a residual update with gamma and a place for the sums");
      if (plan.ksg > 1) {
        if (w->n % 256 != 0 || plan.ksg > 64 || nf->ss_out_stride < (int)(w->n / 256))
          return set_error(YSCV_HIP_ERR_UNSUPPORTED, "folded norm: K-split update needs n a multiple of 256");
        *nf->ss_out_count = (int)(w->n / 256);
      } else {
        if (nf->ss_out_stride < (int)w->nt) return set_error(YSCV_HIP_ERR_INVALID_ARG, "folded norm: room for %zu partial sums per row", w->nt);
        a.gamma_next = nf->gamma_next;
        a.pre = nf->pre;
        a.xg = nf->xg;
        a.ss_out = nf->ss_out;
        a.ss_out_stride = nf->ss_out_stride;
        *nf->ss_out_count = (int)w->nt;
      }
    }
  }
  if (epi == EPI_ADD_F32 && y_dtype != YSCV_HIP_F32)
    return set_error(YSCV_HIP_ERR_INVALID_ARG, "residual accumulation needs an f32 output");
  if (epi == EPI_SWIGLU && (w->n & 1)) return set_error(YSCV_HIP_ERR_INVALID_ARG, "SwiGLU epilogue needs an even row count");
  const bool sf16 = w->scale_dtype == YSCV_HIP_F16;
  const bool small = m <= 4;
  int32_t st;
  if (split == 2)
    st = small ? launch_gm<2, 1>(a, plan, w->gm, sf16, w->has_zp, s) : launch_gm<2, 4>(a, plan, w->gm, sf16, w->has_zp, s);
  else if (m > 4 && m <= 8)  // two accumulators per lane: half the scale FMAs and half the exchange of the 16-row form
    st = launch_gm<1, 2>(a, plan, w->gm, sf16, w->has_zp, s);
  else
    st = small ? launch_gm<1, 1>(a, plan, w->gm, sf16, w->has_zp, s) : launch_gm<1, 4>(a, plan, w->gm, sf16, w->has_zp, s);
  YSCV_TRY(st);
  if (plan.ksg > 1 && produce) {
    hipLaunchKernelGGL(int4_skinny_finalize_norm_kernel, dim3((unsigned)(m * (w->n / 256))), dim3(256), 0, s, partial, plan.ksg,
                       (int)m, (int)w->n, static_cast<float *>(y), nf->gamma_next, nf->pre, nf->xg, nf->ss_out, nf->ss_out_stride);
    YSCV_HIP_TRY(hipGetLastError());
    return YSCV_HIP_OK;
  }
  if (plan.ksg > 1) {
    const size_t total = epi == EPI_SWIGLU ? m * (w->n / 2) : m * w->n;
    int blocks = (int)ceil_div(total, (size_t)256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(int4_skinny_finalize_kernel, dim3(blocks), dim3(256), 0, s, partial, plan.ksg,
                       (int)m, (int)w->n, row_scale, y, y_dtype, epi);
    YSCV_HIP_TRY(hipGetLastError());
  }
  return YSCV_HIP_OK;
}

}  // namespace yscv
