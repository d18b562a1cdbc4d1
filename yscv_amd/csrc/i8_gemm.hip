// int8 x int8 -> int32 GEMM on the gfx950 integer matrix cores, with the zero-point
// correction and the requantize epilogue fused.
// Replaces int8_matmul_dispatch / int8_matmul_prepacked_dispatch
// (crates/yscv-kernels/src/ops/int8_matmul.rs:2407-2425) and the epilogues of
// exec_qlinear_matmul (crates/yscv-onnx/src/runner/linear.rs:481-485) and
// requant_i8_per_channel (crates/yscv-kernels/src/ops/int8_requant.rs:537-555).
//
// Layout: B is packed once (pack_i8_b_for_matmul, int8_matmul.rs:163) into MFMA fragments
//   frag[nt][ks][lane][16 B],  lane = 16*c + r  <-  b[k = 64*ks + 16*c + 0..15][n = 16*nt + r]
// so each wave fetches its B operand of v_mfma_i32_16x16x64_i8 with one coalesced 128-bit load
// per lane straight from global memory -- B never goes through LDS.  A (activations, [m][k]
// row-major) is staged through LDS in the same fragment order, which makes every
// ds_read_b128 of an A operand a contiguous, conflict-free 1 KiB read.
// A workgroup owns a 64 x 128 tile of C with 4 waves side by side along N (each wave
// 64 x 32: 4 x 2 MFMA tiles), so no two waves load the same B fragment.
// uint8 activations are fed to the signed MFMA as (a ^ 0x80) = a - 128, the same bias shift
// the reference uses for VNNI (int8_matmul.rs:1866-1868); the epilogue adds
// (128 - a_zp) * colsum(b), the algebra of runner/conv/quantized.rs:119-147.
#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

constexpr int I8_BM = 64;    // rows of C per workgroup
constexpr int I8_BN = 128;   // columns of C per workgroup
constexpr int I8_KC = 256;   // k per LDS stage (4 MFMA k-steps)
constexpr int I8_THREADS = 256;

// ---- B packing + column sums ---------------------------------------------------------
__global__ void i8_pack_b_kernel(const int8_t *__restrict__ b, size_t k, size_t n, size_t kp, size_t np,
                                 int8_t *__restrict__ frag) {
  const size_t ksteps = kp / 64;
  const size_t total = (np / 16) * ksteps * 64 * 16;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    size_t e = idx & 15;
    size_t lane = (idx >> 4) & 63;
    size_t blk = idx >> 10;
    size_t ks = blk % ksteps, nt = blk / ksteps;
    size_t r = lane & 15, c = lane >> 4;
    size_t kk = ks * 64 + c * 16 + e, col = nt * 16 + r;
    frag[idx] = (kk < k && col < n) ? b[kk * n + col] : (int8_t)0;
  }
}

__global__ void i8_col_sum_kernel(const int8_t *__restrict__ b, size_t k, size_t n, size_t np,
                                  int32_t *__restrict__ col_sum) {
  size_t j = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  if (j >= np) return;
  int32_t s = 0;
  if (j < n)
    for (size_t kk = 0; kk < k; kk++) s += (int32_t)b[kk * n + j];
  col_sum[j] = s;
}

int32_t launch_i8_pack_b(const int8_t *b_kn, size_t k, size_t n, size_t kp, size_t np, int8_t *frag,
                         int32_t *col_sum, hipStream_t s) {
  size_t total = np * kp;
  size_t blocks = ceil_div(total, (size_t)256);
  if (blocks > 262140) blocks = 262140;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(i8_pack_b_kernel, dim3((unsigned)blocks), dim3(256), 0, s, b_kn, k, n, kp, np, frag);
  YSCV_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(i8_col_sum_kernel, dim3((unsigned)ceil_div(np, (size_t)256)), dim3(256), 0, s, b_kn,
                     k, n, np, col_sum);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// ---- rounding helpers (bit-exact with the reference's two rules) -----------------------
// f32::round: half away from zero.  v - trunc(v) is exact, so the comparison is too.
__device__ __forceinline__ float round_half_away(float v) {
  float t = truncf(v);
  float d = fabsf(__fsub_rn(v, t));
  return (d >= 0.5f) ? __fadd_rn(t, copysignf(1.0f, v)) : t;
}

__device__ __forceinline__ int requant_one(int32_t acc, int32_t corr, float comp, float y_zp, int round_mode,
                                           float lo, float hi) {
  int32_t a = (int32_t)((uint32_t)acc + (uint32_t)corr);         // wrapping_add
  float v = __fadd_rn(__fmul_rn((float)a, comp), y_zp);          // two roundings, never an FMA
  float r = round_mode == YSCV_HIP_ROUND_HALF_AWAY ? round_half_away(v) : rintf(v);
  if (r != r) return 0;                                          // clamp keeps NaN, `as i8` -> 0
  r = fminf(fmaxf(r, lo), hi);
  return (int)r;
}

struct I8Args {
  const uint8_t *a;   // [m][k]
  const int8_t *frag; // packed B
  const int32_t *col_sum;
  void *out;
  const int32_t *corr;
  const float *composite_v;
  float composite, y_zp;
  int round_mode, lo, hi, mode;
  int m, n, k;
  int ksteps;       // kp / 64
  int a_xor;        // 0x80808080 for uint8 activations, 0 for int8
  int zp_mul;       // multiplies col_sum in the epilogue
};

template <bool VEC>
__global__ void __launch_bounds__(I8_THREADS) i8_gemm_kernel(I8Args p) {
  // A stage in fragment order: [mt 4][kstep 4][lane 64][16 B] = 16 KiB, double buffered
  __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][I8_BM * I8_KC];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int m0 = blockIdx.y * I8_BM;
  const int n0 = blockIdx.x * I8_BN + wave * 32;
  const int nt0 = n0 / 16;
  const int nt_total = (p.n + 15) / 16;

  int4_t acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) acc[i][j] = int4_t{0, 0, 0, 0};

  const int kc_count = (p.ksteps * 64 + I8_KC - 1) / I8_KC;

  // global -> LDS: thread handles 16-byte chunk `chunk` of row `row`, 4 passes of 16 rows
  auto stage_load = [&](int kc, uint4_t regs[4]) {
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
      const int row = pass * 16 + (tid >> 4);
      const int chunk = tid & 15;
      const int gm = m0 + row;
      const int gk = kc * I8_KC + chunk * 16;
      uint4_t v = {0, 0, 0, 0};
      if (gm < p.m) {
        if constexpr (VEC) {
          if (gk + 16 <= p.k) {
            v = *reinterpret_cast<const uint4_t *>(p.a + (size_t)gm * p.k + gk);
          } else if (gk < p.k) {
            uint8_t tmp[16];
            for (int e = 0; e < 16; e++) tmp[e] = (gk + e < p.k) ? p.a[(size_t)gm * p.k + gk + e] : 0;
            v = *reinterpret_cast<uint4_t *>(tmp);
          }
        } else {
          uint32_t wv[4] = {0, 0, 0, 0};
          for (int e = 0; e < 16; e++)
            if (gk + e < p.k) wv[e >> 2] |= (uint32_t)p.a[(size_t)gm * p.k + gk + e] << (8 * (e & 3));
          v = uint4_t{wv[0], wv[1], wv[2], wv[3]};
        }
        // bytes beyond k must stay 0 *after* the xor: they meet zero-padded B, so any value is fine
        v ^= uint4_t{(uint32_t)p.a_xor, (uint32_t)p.a_xor, (uint32_t)p.a_xor, (uint32_t)p.a_xor};
      }
      regs[pass] = v;
    }
  };
  auto stage_store = [&](int buf, const uint4_t regs[4]) {
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
      const int row = pass * 16 + (tid >> 4);
      const int chunk = tid & 15;
      const int mt = row >> 4, rr = row & 15;
      const int kstep = chunk >> 2, cc = chunk & 3;
      const int off = (((mt * 4 + kstep) * 64) + cc * 16 + rr) * 16;
      *reinterpret_cast<uint4_t *>(&lds_a[buf][off]) = regs[pass];
    }
  };

  uint4_t stage[4];
  stage_load(0, stage);
  stage_store(0, stage);
  __syncthreads();

  for (int kc = 0; kc < kc_count; kc++) {
    const int buf = kc & 1;
    if (kc + 1 < kc_count) stage_load(kc + 1, stage);
    // B fragments of this stage: 4 k-steps x 2 n-tiles
    int4_t bfrag[4][2];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      const int gks = kc * 4 + ks;
#pragma unroll
      for (int j = 0; j < 2; j++) {
        int4_t v = {0, 0, 0, 0};
        if (gks < p.ksteps && (nt0 + j) < nt_total)
          v = *(reinterpret_cast<const int4_t *>(p.frag + ((size_t)(nt0 + j) * p.ksteps + gks) * 1024) + lane);
        bfrag[ks][j] = v;
      }
    }
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int4_t afrag = *reinterpret_cast<const int4_t *>(&lds_a[buf][(((i * 4 + ks) * 64) + lane) * 16]);
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag, bfrag[ks][j], acc[i][j], 0, 0, 0);
      }
    }
    if (kc + 1 < kc_count) {
      stage_store(buf ^ 1, stage);
    }
    __syncthreads();
  }

  // ---- epilogue ---------------------------------------------------------------------------
  const float lo = (float)p.lo, hi = (float)p.hi;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int col = n0 + j * 16 + r;
    if (col >= p.n) continue;
    const int32_t zc = p.zp_mul * p.col_sum[col];
    const int32_t corr = p.corr ? p.corr[col] : 0;
    const float comp = p.composite_v ? p.composite_v[col] : p.composite;
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int row = m0 + i * 16 + c * 4 + e;
        if (row >= p.m) continue;
        const int32_t v = (int32_t)((uint32_t)acc[i][j][e] + (uint32_t)zc);
        const size_t o = (size_t)row * p.n + col;
        if (p.mode == 0) {
          reinterpret_cast<int32_t *>(p.out)[o] = v;
        } else {
          int q = requant_one(v, corr, comp, p.y_zp, p.round_mode, lo, hi);
          reinterpret_cast<uint8_t *>(p.out)[o] = (uint8_t)q;
        }
      }
    }
  }
}

int32_t launch_i8_gemm(const void *a, int a_is_u8, int a_zp, const yscv_hip_i8_weight *b, size_t m,
                       void *out, const I8Epilogue &ep, hipStream_t s) {
  I8Args p;
  p.a = static_cast<const uint8_t *>(a);
  p.frag = b->frag;
  p.col_sum = b->col_sum;
  p.out = out;
  p.corr = ep.corr;
  p.composite_v = ep.composite_v;
  p.composite = ep.composite;
  p.y_zp = ep.y_zp;
  p.round_mode = ep.round_mode;
  p.lo = ep.lo;
  p.hi = ep.hi;
  p.mode = ep.mode;
  p.m = (int)m;
  p.n = (int)b->n;
  p.k = (int)b->k;
  p.ksteps = (int)(b->kp / 64);
  p.a_xor = a_is_u8 ? (int)0x80808080u : 0;
  p.zp_mul = a_is_u8 ? (128 - a_zp) : -a_zp;
  dim3 grid((unsigned)ceil_div(b->n, (size_t)I8_BN), (unsigned)ceil_div(m, (size_t)I8_BM));
  const bool vec = (b->k % 16 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0);
  if (vec)
    hipLaunchKernelGGL(i8_gemm_kernel<true>, grid, dim3(I8_THREADS), 0, s, p);
  else
    hipLaunchKernelGGL(i8_gemm_kernel<false>, grid, dim3(I8_THREADS), 0, s, p);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

}  // namespace yscv
