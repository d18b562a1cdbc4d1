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
#include <mutex>
#include <utility>

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

// requantise, then DequantizeLinear of the quantised value: (q - y_zp) * dq_scale (crates/yscv-onnx/src/runner/misc.rs:124-128)
__device__ __forceinline__ int32_t requant_dequant_bits(int32_t acc, int32_t corr, float comp, float y_zp, int round_mode,
                                                        float lo, float hi, float dq_scale) {
  const int q = requant_one(acc, corr, comp, y_zp, round_mode, lo, hi);
  return __float_as_int(__fmul_rn(__fsub_rn((float)q, y_zp), dq_scale));
}

// requantise and keep the value as an f32 carrier, the form exec_qlinear_matmul returns (crates/yscv-onnx/src/runner/
// linear.rs:481-485): clamp keeps a NaN
__device__ __forceinline__ int32_t requant_f32_bits(int32_t acc, int32_t corr, float comp, float y_zp, int round_mode,
                                                    float lo, float hi) {
  int32_t a = (int32_t)((uint32_t)acc + (uint32_t)corr);
  float v = __fadd_rn(__fmul_rn((float)a, comp), y_zp);
  float r = round_mode == YSCV_HIP_ROUND_HALF_AWAY ? round_half_away(v) : rintf(v);
  if (r == r) r = fminf(fmaxf(r, lo), hi);
  return __float_as_int(r);
}

struct I8Args {
  const uint8_t *a;   // [m][k]
  const int8_t *frag; // packed B
  const int32_t *col_sum;
  void *out;
  const int32_t *corr;
  const float *composite_v;
  float composite, y_zp, dq_scale;
  int round_mode, lo, hi, mode;  // as I8Epilogue::mode
  int m, n, k;
  int ksteps;       // kp / 64
  int a_xor;        // 0x80808080 for uint8 activations, 0 for int8
  int zp_mul;       // multiplies col_sum in the epilogue
  const float *a_zp_dev;  // null, or the uint8 zero point of A as an f32 in device memory (then zp_mul = 128 - that)
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
    const int32_t zc = (p.a_zp_dev ? 128 - (int)p.a_zp_dev[0] : p.zp_mul) * p.col_sum[col];
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
        } else if (p.mode == 3) {
          reinterpret_cast<float *>(p.out)[o] = (float)v;
        } else if (p.mode == 2) {
          reinterpret_cast<int32_t *>(p.out)[o] = requant_dequant_bits(v, corr, comp, p.y_zp, p.round_mode, lo, hi, p.dq_scale);
        } else if (p.mode == 4) {
          reinterpret_cast<int32_t *>(p.out)[o] = requant_f32_bits(v, corr, comp, p.y_zp, p.round_mode, lo, hi);
        } else {
          int q = requant_one(v, corr, comp, p.y_zp, p.round_mode, lo, hi);
          reinterpret_cast<uint8_t *>(p.out)[o] = (uint8_t)q;
        }
      }
    }
  }
}

// ---- ring kernel: both operands stream through an LDS ring filled by LDS-direct loads -----------------
// Used when k is a multiple of 64 and A is 16-byte aligned.  A workgroup has four compute waves (2 x 2) and four
// producer waves.  It owns a (32 MT) x (32 NT) tile of C, a compute wave MT x NT MFMA tiles of it.  A stage holds
// KS k-steps of 64: the A part in fragment order [m-tile][ks][lane][16 B] (each lane fetches its own 16 bytes of a
// row, so the row-major -> fragment transposition costs nothing), the B part [n-tile][ks][lane][16 B] copied as
// it lies in memory.  S stages form a ring: while the MFMAs of stage i run, the producers have the loads of
// stages i+1 .. i+S-1 in flight, track them with their own vmcnt and publish a landed stage with one s_barrier
// per stage; the compute waves never issue a global load, so their MFMAs do not queue behind the address
// processing of the loads.  The MFMA is issued with the operands swapped, D = Bfrag x Afrag, which yields the
// transposed tile: a lane holds four consecutive columns of one row of C.  The finished tile goes through LDS so
// that all eight waves store whole rows of it (512 contiguous bytes of int32, 128 of requantised bytes).
// Workgroups are numbered so that the ones sharing an XCD (id mod 8) cover a contiguous range of n-tiles over
// all m-tiles: an XCD's L2 holds its slice of B once.
typedef __attribute__((address_space(3))) void lds_void;
#define I8_AS1(ptr) ((const void __attribute__((address_space(1))) *)(ptr))
constexpr int I8R_THREADS = 512;

template <int N>
__device__ __forceinline__ void i8_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// one fragment read; the value is valid only after i8_frags_wait
template <int OFF>
__device__ __forceinline__ void i8_ds_read(int4_t &v, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int MT, int NT>
struct I8Frags {
  int4_t a[MT], b[NT];
};
template <int KS, int MT, int NT, int... I, int... J>
__device__ __forceinline__ void i8_frags_issue_impl(I8Frags<MT, NT> &f, uint32_t a_addr, uint32_t b_addr,
                                                    std::integer_sequence<int, I...>, std::integer_sequence<int, J...>) {
  (i8_ds_read<I * KS * 1024>(f.a[I], a_addr), ...);
  (i8_ds_read<J * KS * 1024>(f.b[J], b_addr), ...);
}
template <int KS, int MT, int NT>
__device__ __forceinline__ void i8_frags_issue(I8Frags<MT, NT> &f, uint32_t a_addr, uint32_t b_addr) {
  i8_frags_issue_impl<KS>(f, a_addr, b_addr, std::make_integer_sequence<int, MT>{}, std::make_integer_sequence<int, NT>{});
}
template <int MT, int NT>
__device__ __forceinline__ void i8_frags_wait(I8Frags<MT, NT> &f) {
  if constexpr (MT == 2 && NT == 4) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.b[3])::"memory");
  } else {
    static_assert(MT == 4 && NT == 4, "add a wait for this fragment count");
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]),
                   "+v"(f.b[3])::"memory");
  }
}

// WIDE_A (k-steps come in pairs, i.e. k % 128 == 0): an A load instruction takes eight whole 128-byte lines (eight
// rows x two k-steps, eight neighbouring lanes per line) instead of sixteen half lines; lane i fetches 16-byte chunk
// (i & 7) ^ g of row i / 8 with g = 4 h + (i / 8) / 2 (h = which eight rows of the 16-row group), so that the sixteen
// lanes which later read one k-chunk of sixteen rows in one ds_read_b128 pass hit sixteen different 16-byte slots.
template <int MT, int NT, int KS, int S, bool WIDE_A>
__global__ void __launch_bounds__(I8R_THREADS) i8_gemm_ring_kernel(I8Args p, int tiles_m, int tiles_n, int sbm_log2) {
  constexpr int BM = 32 * MT, BN = 32 * NT;
  constexpr int A_BYTES = 2 * MT * KS * 1024, STAGE = 2 * (MT + NT) * KS * 1024;
  constexpr int PER_WAVE = (MT + NT) * KS / 2;  // 1 KiB chunks a producer wave fetches per stage
  static_assert(((MT + NT) * KS) % 2 == 0 && S >= 2 && S <= 7 && (S - 1) * PER_WAVE < 64, "vmcnt budget");
  constexpr int RS32 = BN * 4 + 16, RS8 = BN + 16;  // row strides of the C tile in LDS (odd multiples of 16 B)
  static_assert(BM * RS32 <= S * STAGE, "the C tile reuses the ring");
  // Registers of a compute lane: accumulators, two fragment sets, the epilogue's per-column terms, addresses.  With
  // eight waves per workgroup a wave has 256; a tile that needs more spills, and this pipeline (literal wait counts,
  // registers of pending LDS reads named in asm statements) is not written for spill code: a 256 x 128 tile
  // (MT 8, NT 4) comes to 128 + 96 + 48 + ~16 = 288 and was measured by the compiler at 256 + 29 spilled.
  static_assert(MT * NT * 4 + 2 * (MT + NT) * 4 + 3 * NT * 4 + 16 <= 256, "tile too large for the register file");
  extern __shared__ __attribute__((aligned(1024))) uint8_t i8_ring[];
  const uint32_t lds0 = (uint32_t)(size_t)i8_ring;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;

  // XCD-aware tile numbering: the grid of tiles is cut into super-blocks of 32 tiles, 2^sbm_log2 (at most 8) along
  // m; workgroup ids that share an XCD (id mod 8) walk through one super-block at a time, so the 32 workgroups an
  // XCD runs together share row panels of A and column panels of B in its L2.
  const int sbm = 1 << sbm_log2, sbn = 32 >> sbm_log2;
  const int sb_m = (tiles_m + sbm - 1) >> sbm_log2;
  const int j_in_xcd = (int)(blockIdx.x >> 3);
  const int sb = (j_in_xcd >> 5) * 8 + (int)(blockIdx.x & 7);
  const int tm = (sb % sb_m) * sbm + (j_in_xcd & (sbm - 1)), tn = (sb / sb_m) * sbn + ((j_in_xcd & 31) >> sbm_log2);
  if (tm >= tiles_m || tn >= tiles_n) return;
  const int m0 = tm * BM, n0 = tn * BN;
  const int nt_total = (p.n + 15) / 16;
  const int nstages = (p.ksteps + KS - 1) / KS;

  int4_t acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++) acc[i][j] = int4_t{0, 0, 0, 0};
  const int wm = (wave >> 1) & 1, wn = wave & 1;

  // The per-column terms of the epilogue are requested before the main loop (compute waves issue no other global
  // load, so nothing in the loop waits for them): their round trip is over long before the tile is finished.
  int32_t zc_all[NT][4], corr_all[NT][4];
  float comp_all[NT][4];
  if (wave < 4) {
    // absent tables are read from the column sums instead and ignored later: the loads stay unconditional and no
    // instruction consumes them before the epilogue
    const int32_t *corr_src = p.corr ? p.corr : p.col_sum;
    const float *comp_src = p.composite_v ? p.composite_v : reinterpret_cast<const float *>(p.col_sum);
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int cc = min(n0 + wn * NT * 16 + j * 16 + c * 4 + e, p.n - 1);
        zc_all[j][e] = p.col_sum[cc];
        corr_all[j][e] = corr_src[cc];
        comp_all[j][e] = comp_src[cc];
      }
  }

  if (wave >= 4) {
    // ---- producer: per-lane source addresses of this wave's chunks at k = 0 (chunk q < 2 MT KS: A, else B)
    const int pw = wave - 4;
    const uint8_t *src[PER_WAVE];
#pragma unroll
    for (int j = 0; j < PER_WAVE; j++) {
      const int q = pw * PER_WAVE + j;
      if (q < 2 * MT * KS) {
        if constexpr (WIDE_A) {
          // piece (q % KS) of 16-row group q / KS: k-step pair (q % KS) / 2, rows 8 h .. 8 h + 7 with h = q % 2
          const int h = q & 1, row8 = lane >> 3;
          const int chunk = (lane & 7) ^ (4 * h + (row8 >> 1));
          const int row = min(m0 + (q / KS) * 16 + 8 * h + row8, p.m - 1);
          src[j] = p.a + (size_t)row * p.k + chunk * 16;
        } else {
          const int row = min(m0 + (q / KS) * 16 + r, p.m - 1);
          src[j] = p.a + (size_t)row * p.k + c * 16;
        }
      } else {
        const int gnt = min(n0 / 16 + (q - 2 * MT * KS) / KS, nt_total - 1);
        src[j] = reinterpret_cast<const uint8_t *>(p.frag) + (size_t)gnt * p.ksteps * 1024 + lane * 16;
      }
    }
    uint32_t fill_slot = 0;  // ring slot the next issued stage goes to
    auto issue_stage = [&](int st) {
      const uint32_t dst = lds0 + fill_slot + (uint32_t)(pw * PER_WAVE * 1024);
      fill_slot = fill_slot + STAGE == S * STAGE ? 0 : fill_slot + STAGE;
#pragma unroll
      for (int j = 0; j < PER_WAVE; j++) {
        const int q = pw * PER_WAVE + j;                      // wave-uniform
        const bool is_a = q < 2 * MT * KS;
        const int ks = (is_a ? q : q - 2 * MT * KS) % KS;
        // k-steps past the end re-read the last one (WIDE_A pieces: the last pair)
        const int gks = (WIDE_A && is_a) ? min(st * KS + (ks & ~1), p.ksteps - 2) : min(st * KS + ks, p.ksteps - 1);
        const uint8_t *g = src[j] + (size_t)gks * (is_a ? 64 : 1024);
        __builtin_amdgcn_global_load_lds(I8_AS1(g), (lds_void *)(uintptr_t)(dst + j * 1024), 16, 0, 0);
      }
    };
    // wait until this wave's part of a stage has landed, given how many later stages it has in flight
    auto wait_landed = [&](int later) {
      switch (later) {
        case 0: i8_wait_vm<0>(); break;
        case 1: i8_wait_vm<PER_WAVE>(); break;
        case 2: i8_wait_vm<(S > 2 ? 2 : 0) * PER_WAVE>(); break;
        case 3: i8_wait_vm<(S > 3 ? 3 : 0) * PER_WAVE>(); break;
        case 4: i8_wait_vm<(S > 4 ? 4 : 0) * PER_WAVE>(); break;
        case 5: i8_wait_vm<(S > 5 ? 5 : 0) * PER_WAVE>(); break;
        default: i8_wait_vm<(S > 6 ? 6 : 0) * PER_WAVE>(); break;
      }
    };
    for (int st = 0; st < S; st++)
      if (st < nstages) issue_stage(st);
    wait_landed(min(S - 1, nstages - 1));
    __builtin_amdgcn_s_barrier();
    for (int st = 0; st + 1 < nstages; st++) {
      // stages st+1 .. st+S-1 are in flight; after the barrier every compute wave is done with stage st
      wait_landed(min(S - 2, nstages - 2 - st));
      __builtin_amdgcn_s_barrier();
      if (st + S < nstages) issue_stage(st + S);
    }
  } else {
    // ---- compute -------------------------------------------------------------------------------------
    // A fragment of k-step ks: lane (r, c) wants chunk 4 (ks % 2) + c of row r.  WIDE_A stores it at slot
    // (r % 8) * 8 + (chunk ^ g) of piece 2 (ks / 2) + r / 8 of its 16-row group (see the producer's swizzle).
    uint32_t a_lane_ks[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if constexpr (WIDE_A) {
        const int g = 4 * (r >> 3) + ((r & 7) >> 1);
        a_lane_ks[ks] = lds0 + (uint32_t)(wm * MT * KS * 1024 + (2 * (ks >> 1) + (r >> 3)) * 1024 +
                                          ((r & 7) * 8 + ((4 * (ks & 1) + c) ^ g)) * 16);
      } else {
        a_lane_ks[ks] = lds0 + (uint32_t)(wm * MT * KS * 1024 + ks * 1024 + lane * 16);
      }
    }
    const uint32_t b_lane = lds0 + (uint32_t)(A_BYTES + wn * NT * KS * 1024 + lane * 16);
    const int4_t xr = {p.a_xor, p.a_xor, p.a_xor, p.a_xor};
    I8Frags<MT, NT> f[2];
    __builtin_amdgcn_s_barrier();
    i8_frags_issue<KS>(f[0], a_lane_ks[0], b_lane);
    auto mfmas = [&](I8Frags<MT, NT> &cur, int i0, int i1) {
#pragma unroll
      for (int i = i0; i < i1; i++) {
        const int4_t av = cur.a[i] ^ xr;
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.b[j], av, acc[i][j], 0, 0, 0);
      }
    };
    uint32_t slot = 0;
    for (int st = 0; st < nstages; st++) {
      const uint32_t nslot = slot + STAGE == S * STAGE ? 0 : slot + STAGE;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        I8Frags<MT, NT> &cur = f[ks & 1], &nxt = f[(ks + 1) & 1];
        const bool live = st * KS + ks < p.ksteps;  // false only in the padding of the last stage
        i8_frags_wait(cur);
        if (ks + 1 < KS) {
          i8_frags_issue<KS>(nxt, a_lane_ks[(ks + 1) % KS] + slot, b_lane + slot + (ks + 1) * 1024);
          if (live) mfmas(cur, 0, MT);
        } else {
          // the first half of the MFMAs runs while this wave waits at the barrier, the second half while the
          // first fragments of the next stage arrive
          if (live) mfmas(cur, 0, MT / 2);
          if (st + 1 < nstages) {
            // every read of stage st by this wave has returned: tell the producers, pick up stage st+1
            __builtin_amdgcn_s_barrier();
            i8_frags_issue<KS>(nxt, a_lane_ks[0] + nslot, b_lane + nslot);
          }
          if (live) mfmas(cur, MT / 2, MT);
        }
      }
      slot = nslot;
    }
  }
  static_assert(KS % 2 == 0, "the two fragment sets alternate per k-step");

  // ---- epilogue: the tile goes to LDS (lane (c, r) holds C[16 i + r][16 j + 4 c + 0..3] of its wave's part),
  // then all waves store whole rows ---------------------------------------------------------------------
  __syncthreads();  // every wave is done with the ring
  const float lo = (float)p.lo, hi = (float)p.hi;
  const int zp_mul = p.a_zp_dev ? 128 - (int)p.a_zp_dev[0] : p.zp_mul;
  if (wave < 4) {
#pragma unroll
    for (int j = 0; j < NT; j++) {
      const int lcol = wn * NT * 16 + j * 16 + c * 4;
      int32_t zc[4], corr[4];
      float comp[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        zc[e] = zp_mul * zc_all[j][e];
        corr[e] = p.corr ? corr_all[j][e] : 0;
        comp[e] = p.composite_v ? comp_all[j][e] : p.composite;
      }
#pragma unroll
      for (int i = 0; i < MT; i++) {
        const int lrow = wm * MT * 16 + i * 16 + r;
        int32_t v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = (int32_t)((uint32_t)acc[i][j][e] + (uint32_t)zc[e]);
        if (p.mode == 0) {
          *reinterpret_cast<int4_t *>(i8_ring + lrow * RS32 + lcol * 4) = int4_t{v[0], v[1], v[2], v[3]};
        } else if (p.mode == 3) {
          *reinterpret_cast<int4_t *>(i8_ring + lrow * RS32 + lcol * 4) =
              int4_t{__float_as_int((float)v[0]), __float_as_int((float)v[1]), __float_as_int((float)v[2]), __float_as_int((float)v[3])};
        } else if (p.mode == 2) {
          int4_t f;
#pragma unroll
          for (int e = 0; e < 4; e++)
            f[e] = requant_dequant_bits(v[e], corr[e], comp[e], p.y_zp, p.round_mode, lo, hi, p.dq_scale);
          *reinterpret_cast<int4_t *>(i8_ring + lrow * RS32 + lcol * 4) = f;
        } else if (p.mode == 4) {
          int4_t f;
#pragma unroll
          for (int e = 0; e < 4; e++) f[e] = requant_f32_bits(v[e], corr[e], comp[e], p.y_zp, p.round_mode, lo, hi);
          *reinterpret_cast<int4_t *>(i8_ring + lrow * RS32 + lcol * 4) = f;
        } else {
          uint32_t packed = 0;
#pragma unroll
          for (int e = 0; e < 4; e++)
            packed |= (uint32_t)(uint8_t)requant_one(v[e], corr[e], comp[e], p.y_zp, p.round_mode, lo, hi) << (8 * e);
          *reinterpret_cast<uint32_t *>(i8_ring + lrow * RS8 + lcol) = packed;
        }
      }
    }
  }
  __syncthreads();
  if (p.mode != 1) {  // four-byte results: int32 sums or dequantised f32
    constexpr int CPR = BN / 4;  // 16-byte chunks per row
    const bool vec = (p.n & 3) == 0;
    for (int q = tid; q < BM * CPR; q += I8R_THREADS) {
      const int lrow = q / CPR, ch = q % CPR;
      const int row = m0 + lrow, col = n0 + ch * 4;
      if (row >= p.m || col >= p.n) continue;
      const int4_t v = *reinterpret_cast<const int4_t *>(i8_ring + lrow * RS32 + ch * 16);
      int32_t *out = reinterpret_cast<int32_t *>(p.out) + (size_t)row * p.n + col;
      if (vec) {
        *reinterpret_cast<int4_t *>(out) = v;
      } else {
        for (int e = 0; e < 4; e++)
          if (col + e < p.n) out[e] = v[e];
      }
    }
  } else {
    constexpr int CPR = BN / 16;
    const bool vec = (p.n & 15) == 0;
    for (int q = tid; q < BM * CPR; q += I8R_THREADS) {
      const int lrow = q / CPR, ch = q % CPR;
      const int row = m0 + lrow, col = n0 + ch * 16;
      if (row >= p.m || col >= p.n) continue;
      const uint4_t v = *reinterpret_cast<const uint4_t *>(i8_ring + lrow * RS8 + ch * 16);
      uint8_t *out = reinterpret_cast<uint8_t *>(p.out) + (size_t)row * p.n + col;
      if (vec) {
        *reinterpret_cast<uint4_t *>(out) = v;
      } else {
        for (int e = 0; e < 16; e++)
          if (col + e < p.n) out[e] = (uint8_t)(v[e >> 2] >> (8 * (e & 3)));
      }
    }
  }
}

template <int MT, int NT, int KS, int S, bool WIDE_A>
int32_t launch_ring(const I8Args &p, size_t m, size_t n, hipStream_t s) {
  constexpr int LDS = 2 * (MT + NT) * KS * 1024 * S;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(i8_gemm_ring_kernel<MT, NT, KS, S, WIDE_A>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
  });
  if (attr_err != hipSuccess)
    return set_error(YSCV_HIP_ERR_DEVICE, "cannot reserve %d bytes of LDS: %s", LDS, hipGetErrorString(attr_err));
  const int tiles_m = (int)ceil_div(m, (size_t)(32 * MT)), tiles_n = (int)ceil_div(n, (size_t)(32 * NT));
  int sbm_log2 = 3;
  while (sbm_log2 > 0 && (1 << sbm_log2) > tiles_m) sbm_log2--;
  const int sbm = 1 << sbm_log2, sbn = 32 >> sbm_log2;
  const int super_blocks = ((tiles_m + sbm - 1) / sbm) * ((tiles_n + sbn - 1) / sbn);
  const unsigned grid = (unsigned)((super_blocks + 7) / 8) * 8 * 32;
  hipLaunchKernelGGL((i8_gemm_ring_kernel<MT, NT, KS, S, WIDE_A>), dim3(grid), dim3(I8R_THREADS), LDS, s, p, tiles_m, tiles_n, sbm_log2);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
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
  p.dq_scale = ep.dq_scale;
  p.m = (int)m;
  p.n = (int)b->n;
  p.k = (int)b->k;
  p.ksteps = (int)(b->kp / 64);
  p.a_xor = a_is_u8 ? (int)0x80808080u : 0;
  p.zp_mul = a_is_u8 ? (128 - a_zp) : -a_zp;
  p.a_zp_dev = ep.a_zp_dev;
  const bool aligned = (reinterpret_cast<uintptr_t>(a) & 15) == 0;
  const bool out_ok = (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  if (b->k % 64 == 0 && aligned && out_ok && m * b->k < ((size_t)1 << 31)) {
    // 128 x 128 tiles halve the LDS fill per MFMA; 64 x 128 tiles are for shapes that would not fill the CUs otherwise
    const Context *ctx = nullptr;
    YSCV_TRY(ensure_context(&ctx));
    const size_t big_tiles = ceil_div(m, (size_t)128) * ceil_div(b->n, (size_t)128);
    const bool wide_a = b->k % 128 == 0;  // k-steps come in pairs: A is fetched as whole 128-byte lines
    if (big_tiles >= (size_t)ctx->num_cus)
      return wide_a ? launch_ring<4, 4, 2, 4, true>(p, m, b->n, s) : launch_ring<4, 4, 2, 4, false>(p, m, b->n, s);
    return wide_a ? launch_ring<2, 4, 4, 3, true>(p, m, b->n, s) : launch_ring<2, 4, 4, 3, false>(p, m, b->n, s);
  }
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
