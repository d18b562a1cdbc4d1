// Wide-M packed-int4 matmul for fp16 / bf16 activations: y[m][n] = sum_k x[m][k] * W[n][k], MFMA-bound design.
// Replaces packed_int4_gemm_dispatch (crates/yscv-kernels/src/ops/int4_matmul.rs:548-605) for prefill-sized m.
//
// A workgroup owns a (32 MT) x (32 NT) tile of y: 32, 64 or 128 rows by 128 columns by m, or 128 x 256 / 256 x 128
// where such tiles still fill the CUs in whole rounds.  It has four MMA waves (2 x 2, MT x NT MFMA tiles each) and NP producer waves.  Per stage of KS k-steps (32 k each) the producers
//   * fetch the activation rows (fp16, prepared by x_prep) with LDS-direct loads, one 16-byte piece per lane: an
//     instruction takes eight whole 128-byte lines (eight rows x both k-steps of the stage), and a per-row XOR of
//     the chunk index makes the later fragment reads conflict-free, so the row-major -> MFMA-fragment
//     transposition costs nothing, and
//   * load the packed weight words of the stage into registers, decode them to fp16 (q - zp) * scale ONCE per
//     workgroup and write them to LDS in fragment order.
// The MMA waves only read fragments (ds_read_b128) and issue v_mfma_f32_16x16x32_f16; a decoded weight is used by
// 2 MT MFMAs and its decode never competes with them for issue slots.  The activation pieces of SA stages form a
// ring (SA - 1 stages in flight hide the memory latency); decoded weights need two slots only because they are
// written just before the stage is published, with one s_barrier per stage.
// The scale is folded into the fp16 weight (relative rounding 2^-11 per weight, exact when the scales are stored
// as fp16), so any group size costs the same; results stay inside the int4 tolerance (max-abs <= 1e-3 sqrt(K)
// max|x|) by more than an order of magnitude.  f32 activations keep the exact-scale kernel of int4_gemm.hip.
// The MFMA is issued with the operands swapped (D = Wfrag x Xfrag): a lane holds four consecutive columns of one
// row of y; the finished tile goes through LDS so that whole rows are stored.
#include <mutex>
#include <type_traits>
#include <utility>

#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

namespace {

__device__ const float kOne = 1.0f;  // stands in for an absent row-scale vector
__device__ __forceinline__ float ring_silu(float g) { return g / (1.0f + __expf(-g)); }

typedef __attribute__((address_space(3))) void lds_void;
#define G4_AS1(ptr) ((const void __attribute__((address_space(1))) *)(ptr))

struct RingArgs {
  const uint8_t *tiles;
  const void *tscales;
  const uint8_t *tzps;
  const _Float16 *xh;
  const float *row_scale;
  void *y;
  int m, n;        // rows; end of the column range of this launch
  int col0, ldy;   // first column of this launch (a multiple of the tile width); row stride of y
  int nt, kt, ktp;
  int chunks, chunk_div;
  int k_pad;
  int y_dtype;
  int epi;         // EPI_STORE, EPI_ADD_F32 (y f32, y += product) or EPI_SWIGLU (y [m][n / 2] = silu(gate) * up, columns 2i / 2i+1)
  // K split (shapes with fewer tiles than CUs): the workgroups of split j multiply 128-k tiles j * kt_per .. and
  // stores its f32 products to partial[j][m][n]; ring_finalize_kernel adds the splits in order and applies `epi`
  float *partial;  // null: no split
  int kt_per, splits;  // splits == 1 and kt_per == kt without a split
};

template <int N>
__device__ __forceinline__ void g4_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
template <int OFF>
__device__ __forceinline__ void g4_ds_read(half8_t &v, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int MT, int NT>
struct G4Frags {
  half8_t a[MT], b[NT];
};
template <int KS, int MT, int NT, int... I, int... J>
__device__ __forceinline__ void g4_issue_impl(G4Frags<MT, NT> &f, uint32_t a_addr, uint32_t b_addr,
                                              std::integer_sequence<int, I...>, std::integer_sequence<int, J...>) {
  (g4_ds_read<I * KS * 1024>(f.a[I], a_addr), ...);
  (g4_ds_read<J * KS * 1024>(f.b[J], b_addr), ...);
}
template <int KS, int MT, int NT>
__device__ __forceinline__ void g4_issue(G4Frags<MT, NT> &f, uint32_t a_addr, uint32_t b_addr) {
  g4_issue_impl<KS>(f, a_addr, b_addr, std::make_integer_sequence<int, MT>{}, std::make_integer_sequence<int, NT>{});
}
template <int MT, int NT>
__device__ __forceinline__ void g4_wait(G4Frags<MT, NT> &f) {
  if constexpr (MT == 4 && NT == 4) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]),
                   "+v"(f.b[3])::"memory");
  } else if constexpr (MT == 4 && NT == 8) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]),
                   "+v"(f.b[3]), "+v"(f.b[4]), "+v"(f.b[5]), "+v"(f.b[6]), "+v"(f.b[7])::"memory");
  } else if constexpr (MT == 8 && NT == 4) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.a[4]), "+v"(f.a[5]), "+v"(f.a[6]),
                   "+v"(f.a[7]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.b[3])::"memory");
  } else if constexpr (MT == 2 && NT == 4) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.b[3])::"memory");
  } else {
    static_assert(MT == 1 && NT == 4, "add a wait for this fragment count");
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.a[0]), "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.b[3])::"memory");
  }
}

typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));

template <int B, int E, class F>
__device__ __forceinline__ void g4_static_for(F &&f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    g4_static_for<B + 1, E>(f);
  }
}

// Loads the producers keep in flight across stages are issued and awaited with opaque instructions: the compiler
// cannot follow registers that rotate through a ring of stages and would wait for every load in flight.  All of
// them use a uniform base pointer plus a 32-bit per-lane offset that never changes, so a stage costs a producer
// a handful of scalar additions and no vector address arithmetic.
template <int GM, bool SF16>
struct G4Scale {
  static constexpr int SPT = GM == GM32 ? 4 : (GM == GM64 ? 2 : 1);
  static constexpr int SC_BYTES = SPT * (SF16 ? 2 : 4);
  static constexpr int ZP_BYTES = SPT;
  static constexpr int SC_REGS = (SC_BYTES + 3) / 4;
};

// One weight tile's share of two stages (128 k): four packed words, the scale chunk and the zero-point chunk of lane
// row r.
// Every member is the destination of exactly one load instruction, and nothing may copy a register between the
// load and the wait (the data is not there yet): the loads name their destination as a read-write operand, which
// ties every reload of a ring position to the same physical register, and the producer code below has no branch
// between the issue of a load and its wait.
template <int SC_REGS>
struct G4ScaleRegs {
  typedef uint32_t type __attribute__((ext_vector_type(SC_REGS)));
};
template <>
struct G4ScaleRegs<1> {
  typedef uint32_t type;
};
template <int SC_REGS>
struct G4Tile {
  uint4_t raw;
  typename G4ScaleRegs<SC_REGS>::type sc;
  uint32_t zp;
  __device__ __forceinline__ uint32_t sc_reg(int i) const {
    if constexpr (SC_REGS == 1) return sc;
    else return sc[i];
  }
};
template <int BYTES, int SC_REGS>
__device__ __forceinline__ void g4_load_scale(G4Tile<SC_REGS> &t, uint32_t voff, const void *base) {
  static_assert((BYTES + 3) / 4 == SC_REGS, "one load fills the scale registers");
  if constexpr (BYTES == 2) asm volatile("global_load_ushort %0, %1, %2" : "+v"(t.sc) : "v"(voff), "s"(base) : "memory");
  if constexpr (BYTES == 4) asm volatile("global_load_dword %0, %1, %2" : "+v"(t.sc) : "v"(voff), "s"(base) : "memory");
  if constexpr (BYTES == 8) asm volatile("global_load_dwordx2 %0, %1, %2" : "+v"(t.sc) : "v"(voff), "s"(base) : "memory");
  if constexpr (BYTES == 16) asm volatile("global_load_dwordx4 %0, %1, %2" : "+v"(t.sc) : "v"(voff), "s"(base) : "memory");
}
template <int BYTES, int SC_REGS>
__device__ __forceinline__ void g4_load_zp(G4Tile<SC_REGS> &t, uint32_t voff, const void *base) {
  if constexpr (BYTES == 1) asm volatile("global_load_ubyte %0, %1, %2" : "+v"(t.zp) : "v"(voff), "s"(base) : "memory");
  if constexpr (BYTES == 2) asm volatile("global_load_ushort %0, %1, %2" : "+v"(t.zp) : "v"(voff), "s"(base) : "memory");
  if constexpr (BYTES == 4) asm volatile("global_load_dword %0, %1, %2" : "+v"(t.zp) : "v"(voff), "s"(base) : "memory");
}
template <int SC_REGS>
__device__ __forceinline__ void g4_load_raw(G4Tile<SC_REGS> &t, uint32_t voff, const void *base) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "+v"(t.raw) : "v"(voff), "s"(base) : "memory");
}
// wait until at most N loads are in flight; the tile registers count as written by the wait
template <int N, int SC_REGS>
__device__ __forceinline__ void g4_wait_tiles(G4Tile<SC_REGS> (&t)[1]) {
  asm volatile("s_waitcnt vmcnt(%3)" : "+v"(t[0].raw), "+v"(t[0].sc), "+v"(t[0].zp) : "n"(N) : "memory");
}
template <int N, int SC_REGS>
__device__ __forceinline__ void g4_wait_tiles(G4Tile<SC_REGS> (&t)[2]) {
  asm volatile("s_waitcnt vmcnt(%6)"
               : "+v"(t[0].raw), "+v"(t[0].sc), "+v"(t[0].zp), "+v"(t[1].raw), "+v"(t[1].sc), "+v"(t[1].zp)
               : "n"(N)
               : "memory");
}
template <int N, int SC_REGS>
__device__ __forceinline__ void g4_wait_tiles(G4Tile<SC_REGS> (&t)[4]) {
  asm volatile("s_waitcnt vmcnt(%12)"
               : "+v"(t[0].raw), "+v"(t[0].sc), "+v"(t[0].zp), "+v"(t[1].raw), "+v"(t[1].sc), "+v"(t[1].zp), "+v"(t[2].raw),
                 "+v"(t[2].sc), "+v"(t[2].zp), "+v"(t[3].raw), "+v"(t[3].sc), "+v"(t[3].zp)
               : "n"(N)
               : "memory");
}
template <int N>
__device__ __forceinline__ void g4_wait_vm_n() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int MT, int NT, int KS, int SA, int NP, int GM, bool SF16>
__global__ void __launch_bounds__(256 + 64 * NP) int4_gemm_ring_kernel(RingArgs p, int tiles_m, int tiles_n, int sbm_log2) {
  constexpr int THREADS = 256 + 64 * NP;
  constexpr int BM = 32 * MT, BN = 32 * NT;
  constexpr int A_BYTES = 2 * MT * KS * 1024, B_BYTES = 2 * NT * KS * 1024;  // one stage of each operand
  constexpr int B_BASE = SA * A_BYTES, LDS_BYTES = SA * A_BYTES + 2 * B_BYTES;
  constexpr int APW = 2 * MT * KS / NP;  // activation chunks (1 KiB) a producer wave fetches per stage
  constexpr int WT = 2 * NT / NP;        // weight tiles (16 columns) a producer wave decodes per stage
  static_assert(KS == 2, "a stage is half a 128-k weight tile");
  static_assert((2 * MT * KS) % NP == 0 && (2 * NT) % NP == 0 && (WT == 1 || WT == 2 || WT == 4), "work split over the producer waves");
  static_assert(SA >= 2 && SA <= 6 && SA % 2 == 0, "stage parity must follow the ring position");
  constexpr int RS = BN * 4 + 16;  // row stride of the f32 result tile in LDS (odd multiple of 16 B)
  // the result tile reuses the ring: whole when it fits, else the rows of the upper and the lower MMA waves in turn
  constexpr int EPI_PASSES = BM * RS <= LDS_BYTES ? 1 : 2;
  constexpr int EPI_ROWS = BM / EPI_PASSES;
  static_assert(EPI_ROWS * RS <= LDS_BYTES && (EPI_PASSES == 1 || EPI_ROWS == MT * 16), "the result tile reuses the ring");
  extern __shared__ __attribute__((aligned(1024))) uint8_t g4_ring[];
  const uint32_t lds0 = (uint32_t)(size_t)g4_ring;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;

  // XCD-aware tile numbering: the grid of tiles is cut into super-blocks of 32 tiles, 2^sbm_log2 (at most 8) along
  // m; workgroup ids that share an XCD (id mod 8) walk through one super-block at a time, so the 32 workgroups an
  // XCD runs together share row panels of A and column panels of B in its L2.
  // With a K split the (super-block, split) pairs are numbered the same way: the splits of one super-block land on
  // different XCDs (a shape with a single super-block would otherwise keep all its workgroups on one).
  const int sbm = 1 << sbm_log2, sbn = 32 >> sbm_log2;
  const int sb_m = (tiles_m + sbm - 1) >> sbm_log2;
  const int sb_count = sb_m * ((tiles_n + sbn - 1) / sbn);
  const int j_in_xcd = (int)(blockIdx.x >> 3);
  const int pair = (j_in_xcd >> 5) * 8 + (int)(blockIdx.x & 7);
  const int sb = pair % sb_count, ksplit = pair / sb_count;
  const int tm = (sb % sb_m) * sbm + (j_in_xcd & (sbm - 1)), tn = (sb / sb_m) * sbn + ((j_in_xcd & 31) >> sbm_log2);
  if (tm >= tiles_m || tn >= tiles_n || ksplit >= p.splits) return;
  const int m0 = tm * BM, n0 = p.col0 + tn * BN;
  const int kt_lo = ksplit * p.kt_per;
  const int kt_n = min(p.kt - kt_lo, p.kt_per);
  const int nstages = kt_n * (4 / KS), st_base = kt_lo * (4 / KS);  // this workgroup's stages are st_base + 0 .. nstages - 1

  float4_t acc[MT][NT];  // MMA waves only; the producers never touch it
  const int wm = (wave >> 1) & 1, wn = wave & 1;

  if (wave >= 4) {
    // ---- producer ------------------------------------------------------------------------------------
    typedef G4Scale<GM, SF16> SC;
    typedef G4Tile<SC::SC_REGS> Tile;
    // loads of this wave per stage: an even stage fetches the weight side of its 128-k tile (both stages of it)
    // before its activation pieces, an odd stage only activation pieces
    constexpr int PE = 3 * WT + APW, PO = APW;
    static_assert((SA / 2) * PE + (SA / 2) * PO + APW < 64, "vmcnt budget");
    const int pw = wave - 4;
    const bool has_zp = p.tzps != nullptr;
    NibbleConsts nc;  // one v_and_or_b32 per pair of nibbles: the decode shares the SIMD's issue port with the MFMAs
    nc.init();
    // per-lane byte offsets (fixed) and uniform base pointers (advanced per stage)
    uint32_t aoff[APW];
#pragma unroll
    // Piece q of a stage = rows 8 h .. 8 h + 7 (h = q & 1) of 16-row group q / 2, both k-steps: eight whole 128-byte
    // lines per load instruction, eight neighbouring lanes per line.  Lane i fetches 16-byte chunk (i & 7) ^ g of
    // row i / 8, g = 4 h + (i / 8) / 2: with this swizzle the 16 lanes that later read one k-chunk of 16 rows in
    // one ds_read_b128 pass hit 16 different 16-byte slots (no bank conflict).
    for (int j = 0; j < APW; j++) {
      const int q = pw * APW + j;
      const int h = q & 1, row8 = lane >> 3;
      const int chunk = (lane & 7) ^ (4 * h + (row8 >> 1));
      const int row = min(m0 + (q >> 1) * 16 + 8 * h + row8, p.m - 1);
      aoff[j] = (uint32_t)(((size_t)row * p.k_pad + chunk * 8) * sizeof(_Float16));
    }
    const uint32_t woff = lane * 16, soff = r * SC::SC_BYTES, zoff = r * SC::ZP_BYTES;
    const uint8_t *wbase[WT], *sbase[WT], *zbase[WT];
#pragma unroll
    for (int u = 0; u < WT; u++) {
      const int nt = min(n0 / 16 + pw * WT + u, p.nt - 1);
      wbase[u] = p.tiles + (size_t)nt * p.ktp * kTileBytes;
      sbase[u] = reinterpret_cast<const uint8_t *>(p.tscales) + (size_t)nt * p.chunks * 16 * SC::SC_BYTES;
      zbase[u] = has_zp ? p.tzps + (size_t)nt * p.chunks * 16 * SC::ZP_BYTES : sbase[u];  // keeps the load count uniform
    }
    const int zstride = has_zp ? 16 * SC::ZP_BYTES : 16 * SC::SC_BYTES;

    Tile wr[SA / 2][WT];  // weight registers of the even stages in flight
    // stage st goes to activation slot / register set ri = st mod SA; par = st & 1 picks the words of the tile
    auto issue_stage = [&](int st_local, auto ric, auto parc) {
      constexpr int ri = decltype(ric)::value, par = decltype(parc)::value;
      const int st = st_base + st_local;
      if constexpr (par == 0) {
        const int kt = st >> 1;
        const int chunk = GM == GM128 ? kt / p.chunk_div : kt;
#pragma unroll
        for (int u = 0; u < WT; u++) {
          g4_load_raw(wr[ri / 2][u], woff, wbase[u] + (size_t)kt * kTileBytes);
          g4_load_scale<SC::SC_BYTES>(wr[ri / 2][u], soff, sbase[u] + (size_t)chunk * 16 * SC::SC_BYTES);
          g4_load_zp<SC::ZP_BYTES>(wr[ri / 2][u], zoff, zbase[u] + (size_t)chunk * zstride);
        }
      }
      const char *abase = reinterpret_cast<const char *>(p.xh) + (size_t)st * KS * 32 * sizeof(_Float16);
#pragma unroll
      for (int j = 0; j < APW; j++) {
        // uniform base + per-lane 32-bit offset, written out: left to the compiler, the loads inside the loop take
        // 64-bit per-lane addresses, one more vector instruction each next to the MFMAs
        const uint32_t dst = lds0 + (uint32_t)(ri * A_BYTES + (pw * APW + j) * 1024);
        const uint32_t off = aoff[j];
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(abase)
                     : "memory");  // m0: reserved, never allocated by the compiler; nothing else in this kernel reads it
      }
    };
    // decode the weights of a stage (register set ri, parity par) into weight slot par
    auto decode_stage = [&](auto ric, auto parc) {
      constexpr int ri = decltype(ric)::value, par = decltype(parc)::value;
      const uint32_t dst = lds0 + (uint32_t)(B_BASE + par * B_BYTES + pw * WT * KS * 1024 + lane * 16);
#pragma unroll
      for (int u = 0; u < WT; u++) {
        half2_t c1[KS], c2[KS];
        half8_t sv[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          constexpr int dummy = 0;
          (void)dummy;
          const int e = GM == GM32 ? (par * KS + ks) : (GM == GM64 ? par : 0);  // group inside the chunk
          if (ks > 0 && GM != GM32) {
            c1[ks] = c1[0];
            c2[ks] = c2[0];
            sv[ks] = sv[0];
            continue;
          }
          const uint32_t zq = has_zp ? ((wr[ri / 2][u].zp >> (8 * e)) & 0xFF) : 8u;
          const _Float16 z = (_Float16)(float)zq;
          const _Float16 c1v = (_Float16)(-1024.0f) - z, c2v = (_Float16)(-64.0f) - z;
          c1[ks] = half2_t{c1v, c1v};
          c2[ks] = half2_t{c2v, c2v};
          _Float16 s;
          if constexpr (SF16) {
            U32H2 t;
            t.u = wr[ri / 2][u].sc_reg(e >> 1);
            s = t.h[e & 1];
          } else {
            s = (_Float16)__uint_as_float(wr[ri / 2][u].sc_reg(e));
          }
          sv[ks] = half8_t{s, s, s, s, s, s, s, s};
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          const half8_t h = decode8_exact(wr[ri / 2][u].raw[par * KS + ks], nc, c1[ks], c2[ks]) * sv[ks];
          // written with an opaque instruction: a compiler-visible LDS store would first wait for every LDS-direct
          // load in flight
          asm volatile("ds_write_b128 %0, %1" ::"v"(dst + (uint32_t)((u * KS + ks) * 1024)), "v"(h) : "memory");
        }
      }
    };
    // Loads complete in order and an even stage issues its weight loads before its activation pieces: the weights
    // are decoded while the latter still fly.  NE / NO = even / odd stages issued after the published one.
    auto publish = [&](auto ric, auto parc, auto nec, auto noc) {
      constexpr int ri = decltype(ric)::value, par = decltype(parc)::value;
      constexpr int L = decltype(nec)::value * PE + decltype(noc)::value * PO;
      if constexpr (par == 0) g4_wait_tiles<L + APW>(wr[ri / 2]);
      decode_stage(ric, parc);
      g4_wait_vm_n<L>();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
    };
    // Exactly SA stages are in flight at any time: past the last stage the producers keep fetching it again (into
    // slots and registers nobody reads any more), so no wait count and no branch depends on how far the end is.
    const int last = nstages - 1;
    // one step while the MMA waves work on stage s: publish stage s+1, then refill the slot and registers of stage s
    auto step = [&](int s, auto uc) {
      constexpr int u = decltype(uc)::value;
      publish(std::integral_constant<int, (u + 1) % SA>{}, std::integral_constant<int, ((u + 1) & 1)>{},
              std::integral_constant<int, (SA - 2) / 2>{}, std::integral_constant<int, (SA - 2) / 2>{});
      issue_stage(min(s + SA, last), uc, std::integral_constant<int, (u & 1)>{});
    };

#pragma unroll
    for (int i = 0; i < SA / 2; i++)
#pragma unroll
      for (int u = 0; u < WT; u++) {
        wr[i][u].raw = uint4_t{0, 0, 0, 0};
        wr[i][u].sc = typename G4ScaleRegs<SC::SC_REGS>::type(0);
        wr[i][u].zp = 0;
      }
    g4_static_for<0, SA>([&](auto uc) {
      constexpr int u = decltype(uc)::value;
      issue_stage(min(u, last), uc, std::integral_constant<int, (u & 1)>{});
    });
    publish(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, SA / 2 - 1>{},
            std::integral_constant<int, SA / 2>{});
    // The steps run in whole groups of SA, one loop and nothing after it: `last` steps are needed, the group is
    // completed with steps past the end (they publish the last stage again into a slot nobody reads; the MMA waves
    // answer their barriers, see below).  Straight-line code for the 1 .. SA-1 left-over steps behind the loop gave the
    // compiler a place to move the tile registers of loads still in flight (copies at the entry of each left-over
    // path, executed before the data had landed): wrong weights in the last stages, now and then.
    for (int s0 = 0; s0 < last; s0 += SA) g4_static_for<0, SA>([&](auto uc) { step(s0 + decltype(uc)::value, uc); });
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // the registers of the loads issued past the end stay reserved until those loads have landed
#pragma unroll
    for (int i = 0; i < SA / 2; i++)
#pragma unroll
      for (int u = 0; u < WT; u++) asm volatile("" ::"v"(wr[i][u].raw), "v"(wr[i][u].sc), "v"(wr[i][u].zp));
  } else {
    // ---- MMA waves -----------------------------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) acc[i][j] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    // k-step ks of 16-row group: lane (r, c) wants chunk 4 ks + c of row r, stored at slot (r % 8) * 8 + (chunk ^ g)
    // of the half r / 8 (see the producer's swizzle)
    uint32_t a_lane_ks[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const int g = 4 * (r >> 3) + ((r & 7) >> 1);
      a_lane_ks[ks] = lds0 + (uint32_t)(wm * MT * KS * 1024 + (r >> 3) * 1024 + (((r & 7) * 8 + ((4 * ks + c) ^ g)) * 16));
    }
    const uint32_t b_lane = lds0 + B_BASE + (uint32_t)(wn * NT * KS * 1024 + lane * 16);
    G4Frags<MT, NT> f[2];
    auto mfmas = [&](const G4Frags<MT, NT> &cur, int i0, int i1) {
#pragma unroll
      for (int i = i0; i < i1; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cur.b[j], cur.a[i], acc[i][j], 0, 0, 0);
    };
    __builtin_amdgcn_s_barrier();
    g4_issue<KS>(f[0], a_lane_ks[0], b_lane);
    uint32_t aslot = 0, bslot = 0;
    for (int st = 0; st < nstages; st++) {
      const uint32_t naslot = aslot + A_BYTES == SA * A_BYTES ? 0 : aslot + A_BYTES;
      const uint32_t nbslot = bslot ^ B_BYTES;
      // k-step 0: the fragments of k-step 1 are on their way while its MFMAs run
      g4_wait(f[0]);
      g4_issue<KS>(f[1], a_lane_ks[1] + aslot, b_lane + bslot + 1024);
      mfmas(f[0], 0, MT);
      // k-step 1: the first MFMAs cover the barrier, the others the fragment reads of the next stage
      g4_wait(f[1]);
      mfmas(f[1], 0, MT / 2);
      if (st + 1 < nstages) {
        __builtin_amdgcn_s_barrier();
        g4_issue<KS>(f[0], a_lane_ks[0] + naslot, b_lane + nbslot);
      }
      mfmas(f[1], MT / 2, MT);
      aslot = naslot;
      bslot = nbslot;
    }
    // the producers run their steps in whole groups of SA: answer the barriers of the steps past the last stage
    const int steps = nstages - 1;
    for (int e = steps; e < (steps + SA - 1) / SA * SA; e++) __builtin_amdgcn_s_barrier();
  }

  // ---- epilogue: lane (c, r) of an MMA wave holds y[16 i + r][16 j + 4 c + 0..3] of its part; through LDS so that
  // all waves store whole rows ------------------------------------------------------------------------------
  __syncthreads();
  // all row scales are requested together (a load behind a branch of its own is waited for on its own)
  float rs[MT];
  if (wave < 4) {
#pragma unroll
    for (int i = 0; i < MT; i++) {
      const int row = min(m0 + wm * MT * 16 + i * 16 + r, p.m - 1);
      const float *src = p.row_scale ? p.row_scale + row : &kOne;
      rs[i] = *src;
    }
  }
  constexpr int CPR = BN / 4;  // four-column chunks per row
  const bool vec = ((p.n | p.ldy) & 3) == 0;
#pragma unroll
  for (int hp = 0; hp < EPI_PASSES; hp++) {
    if (hp > 0) __syncthreads();  // the stores of the previous pass have read their rows
    if (wave < 4 && (EPI_PASSES == 1 || wm == hp)) {
#pragma unroll
      for (int i = 0; i < MT; i++) {
        const int lrow = wm * MT * 16 + i * 16 + r - hp * EPI_ROWS;
#pragma unroll
        for (int j = 0; j < NT; j++) {
          const int lcol = wn * NT * 16 + j * 16 + c * 4;
          *reinterpret_cast<float4_t *>(g4_ring + lrow * RS + lcol * 4) = acc[i][j] * rs[i];
        }
      }
    }
    __syncthreads();
    for (int q = tid; q < EPI_ROWS * CPR; q += THREADS) {
      const int lrow = q / CPR, ch = q % CPR;
      const int row = m0 + hp * EPI_ROWS + lrow, col = n0 + ch * 4;
      if (row >= p.m || col >= p.n) continue;
      const float4_t v = *reinterpret_cast<const float4_t *>(g4_ring + lrow * RS + ch * 16);
      const size_t o = (size_t)row * p.ldy + col;
      if (p.partial) {
        float *dst = p.partial + ((size_t)ksplit * p.m + row) * p.n + col;
        if (vec) {
          *reinterpret_cast<float4_t *>(dst) = v;
        } else {
          for (int e = 0; e < 4; e++)
            if (col + e < p.n) dst[e] = v[e];
        }
      } else if (p.epi == EPI_SWIGLU) {
        // columns col .. col + 3 are gate, up, gate, up of two channels (n is even, col a multiple of 4)
        const size_t oh = (size_t)row * (p.ldy >> 1) + (col >> 1);
        store_out(p.y, oh, ring_silu(v[0]) * v[1], p.y_dtype);
        if (col + 2 < p.n) store_out(p.y, oh + 1, ring_silu(v[2]) * v[3], p.y_dtype);
      } else if (p.epi == EPI_ADD_F32) {
        float *dst = reinterpret_cast<float *>(p.y) + o;  // every element has one writer in a launch
        if (vec) {
          *reinterpret_cast<float4_t *>(dst) = *reinterpret_cast<const float4_t *>(dst) + v;
        } else {
          for (int e = 0; e < 4; e++)
            if (col + e < p.n) dst[e] += v[e];
        }
      } else if (vec) {
        if (p.y_dtype == YSCV_HIP_F32) {
          *reinterpret_cast<float4_t *>(reinterpret_cast<float *>(p.y) + o) = v;
        } else if (p.y_dtype == YSCV_HIP_F16) {
          *reinterpret_cast<half4_t *>(reinterpret_cast<_Float16 *>(p.y) + o) =
              half4_t{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        } else {
          uint2 b;
          b.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
          b.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
          *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.y) + o) = b;
        }
      } else {
        for (int e = 0; e < 4; e++)
          if (col + e < p.n) store_out(p.y, o + e, v[e], p.y_dtype);
      }
    }
  }
}

// Adds the K splits of a launch in a fixed order and applies the epilogue: four columns per thread.
__global__ void __launch_bounds__(256) ring_finalize_kernel(const float *__restrict__ partial, int splits, int m, int n, void *y,
                                                            int y_dtype, int epi, int ldy) {
  const int chunks = (n + 3) / 4;
  const size_t total = (size_t)m * chunks;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const int row = (int)(idx / chunks), col = (int)(idx % chunks) * 4;
    const bool whole = col + 4 <= n && (n & 3) == 0;
    float4_t v = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j = 0; j < splits; j++) {
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
      store_out(y, oh, ring_silu(v[0]) * v[1], y_dtype);
      if (col + 2 < n) store_out(y, oh + 1, ring_silu(v[2]) * v[3], y_dtype);
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

template <int MT, int NT, int KS, int SA, int NP, int GM, bool SF16>
int32_t ring_launch_one(const RingArgs &a, hipStream_t s) {
  constexpr int LDS = 2 * MT * KS * 1024 * SA + 2 * 2 * NT * KS * 1024;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  auto kern = int4_gemm_ring_kernel<MT, NT, KS, SA, NP, GM, SF16>;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
  });
  if (attr_err != hipSuccess)
    return set_error(YSCV_HIP_ERR_DEVICE, "cannot reserve %d bytes of LDS: %s", LDS, hipGetErrorString(attr_err));
  const int tiles_m = (int)ceil_div((size_t)a.m, (size_t)(32 * MT)), tiles_n = (int)ceil_div((size_t)(a.n - a.col0), (size_t)(32 * NT));
  int sbm_log2 = 3;
  while (sbm_log2 > 0 && (1 << sbm_log2) > tiles_m) sbm_log2--;
  const int sbm = 1 << sbm_log2, sbn = 32 >> sbm_log2;
  const int super_blocks = ((tiles_m + sbm - 1) / sbm) * ((tiles_n + sbn - 1) / sbn);
  const unsigned splits = (unsigned)a.splits;
  const unsigned grid = (unsigned)((super_blocks * splits + 7) / 8) * 8 * 32;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256 + 64 * NP), LDS, s, a, tiles_m, tiles_n, sbm_log2);
  YSCV_HIP_TRY(hipGetLastError());
  if (a.partial) {
    const size_t work = (size_t)a.m * ((a.n + 3) / 4);
    const unsigned fb = (unsigned)std::min<size_t>((work + 255) / 256, 4096);
    hipLaunchKernelGGL(ring_finalize_kernel, dim3(fb), dim3(256), 0, s, a.partial, (int)splits, a.m, a.n, a.y, a.y_dtype, a.epi, a.ldy);
    YSCV_HIP_TRY(hipGetLastError());
  }
  return YSCV_HIP_OK;
}

template <int MT, int NT, int KS, int SA, int NP>
int32_t ring_launch_gm(const RingArgs &a, int gm, bool sf16, hipStream_t s) {
  if (gm == GM32)
    return sf16 ? ring_launch_one<MT, NT, KS, SA, NP, GM32, true>(a, s) : ring_launch_one<MT, NT, KS, SA, NP, GM32, false>(a, s);
  if (gm == GM64)
    return sf16 ? ring_launch_one<MT, NT, KS, SA, NP, GM64, true>(a, s) : ring_launch_one<MT, NT, KS, SA, NP, GM64, false>(a, s);
  return sf16 ? ring_launch_one<MT, NT, KS, SA, NP, GM128, true>(a, s) : ring_launch_one<MT, NT, KS, SA, NP, GM128, false>(a, s);
}

}  // namespace

bool int4_gemm_ring_eligible(const yscv_hip_int4_weight *w, const _Float16 *xh, const void *y, int y_dtype, int split, size_t m,
                             size_t k_pad) {
  if (!w->tiled || split != 1) return false;
  if ((reinterpret_cast<uintptr_t>(xh) & 15) != 0) return false;
  if (m * k_pad * sizeof(_Float16) >= ((size_t)1 << 32)) return false;  // per-lane offsets are 32 bits wide
  const size_t align = y_dtype == YSCV_HIP_F32 ? 16 : 8;
  return (reinterpret_cast<uintptr_t>(y) & (align - 1)) == 0;
}

namespace {

// Tile shapes: 0 = 128 x 128, 1 = 128 x 256, 2 = 256 x 128 (m > 128), 3 = 32 x 128 (m <= 32), 4 = 64 x 128 (m <= 64)
struct RingPlan {
  int one;           // shape of the launch, or of the first of two launches
  int second;        // < 0: one launch; else the shape of the launch that takes the columns from split_col on
  size_t split_col;
  int splits, kt_per;  // K split of a single launch (splits == 1: none)
};

RingPlan ring_plan(size_t m, size_t n, size_t kt, size_t cus) {
  RingPlan pl{0, -1, 0, 1, (int)kt};
  size_t tiles;
  if (m <= 32) {
    // The tile height follows m: the MFMA work of a workgroup, and with it the time a weight tile stays in LDS, is
    // proportional to the tile's rows whether they exist or not, so a short m streams the weights faster on a
    // 32- or 64-row tile.
    pl.one = 3;
    tiles = ceil_div(n, (size_t)128);
  } else if (m <= 64) {
    pl.one = 4;
    tiles = ceil_div(n, (size_t)128);
  } else {
    // Larger tiles: 128 x 256 (a third fewer fragment reads per MFMA) and 256 x 128 (the same, and every decoded
    // weight feeds twice as many MFMAs).  A workgroup needs about 1.72 / 1.63 times as long for them as for a
    // 128 x 128 tile; they pay when the tiles come in rounds over the CUs and the larger ones need sufficiently fewer
    // rounds.  When the last round of the best shape would leave most CUs idle, the columns of its whole rounds go to
    // one launch and the rest to a second one with the shape that suits the rest (config 3: three rounds of
    // 256 x 128 tiles, then one round of 128 x 128 tiles, instead of three and a half rounds).
    struct Shape {
      size_t bm, bn, cost;
      int code;
    };
    // cost: time of one tile in hundredths of a 128 x 128 tile's (measured on K 4096: 40 us; the 64-row tile 30 us).
    // The 64-row tile decodes every weight twice as often per MFMA; it pays where it fills CUs that the taller tiles
    // would leave idle (512 rows against N 4096: 256 tiles instead of 128).
    const Shape shapes[4] = {{128, 128, 100, 0}, {128, 256, 172, 1}, {256, 128, 163, 2}, {64, 128, 75, 4}};
    // best single shape for columns [c0, n): cost of its rounds over the CUs
    auto best_single = [&](size_t c0, int *which, size_t *tiles_out) {
      size_t best = (size_t)-1;
      for (int i = 0; i < 4; i++) {
        if (i == 2 && m <= 128) continue;
        const size_t t = ceil_div(m, shapes[i].bm) * ceil_div(n - c0, shapes[i].bn);
        const size_t cost = ceil_div(t, cus) * shapes[i].cost;
        if (cost < best) {
          best = cost;
          *which = shapes[i].code;
          *tiles_out = t;
        }
      }
      return best;
    };
    size_t best = best_single(0, &pl.one, &tiles);
    const size_t launch_cost = 10;  // a second launch: about a tenth of a tile time
    for (int i = 0; i < 3; i++) {
      if (i == 2 && m <= 128) continue;
      const size_t tm = ceil_div(m, shapes[i].bm), tn = ceil_div(n, shapes[i].bn);
      const size_t rounds = tm * tn / cus;    // whole rounds
      const size_t cols = rounds * cus / tm;  // whole tile columns inside them
      if (rounds == 0 || cols == 0 || cols >= tn) continue;
      int rest = 0;
      size_t rest_tiles = 0;
      const size_t cost =
          ceil_div(tm * cols, cus) * shapes[i].cost + best_single(cols * shapes[i].bn, &rest, &rest_tiles) + launch_cost;
      if (cost < best) {
        best = cost;
        pl.one = shapes[i].code;
        pl.second = rest;
        pl.split_col = cols * shapes[i].bn;
      }
    }
    if (pl.second >= 0) return pl;
  }
  // K split: a shape whose tiles cover at most half the CUs is cut along k, each part with at least four 128-k tiles
  // (eight stages), as long as the f32 partial sums stay within 16 MB and, together with a prepared fp16 copy of the
  // activations, within 31 MB (they travel in the caller's workspace; yscv_hip_int4_matmul_static has 32 MB for
  // both).  The workgroups of one
  // (super-block, split) pair share an XCD, eight pairs run side by side: the number of splits is the one with the
  // shortest estimated time, rounds of eight pairs x (a part's k-tiles at 0.9 us each + 5 us to start and end a
  // workgroup), + 5 us for the kernel that adds the parts.
  if (tiles * 2 <= cus && kt >= 8) {
    const size_t bm = pl.one == 3 ? 32 : (pl.one == 4 ? 64 : (pl.one == 2 ? 256 : 128)), bn = pl.one == 1 ? 256 : 128;
    const size_t tiles_m = ceil_div(m, bm), tiles_n = ceil_div(n, bn);
    size_t sbm = 8;
    while (sbm > 1 && sbm > tiles_m) sbm >>= 1;
    const size_t sb = ceil_div(tiles_m, sbm) * ceil_div(tiles_n, 32 / sbm);
    size_t best_ks = 1, best_t = ceil_div(sb, (size_t)8) * (kt * 18 + 100);  // units of 0.05 us
    const size_t x_bytes = m * kt * 128 * sizeof(_Float16);
    const size_t room = x_bytes >= ((size_t)31 << 20) ? 0 : ((size_t)31 << 20) - x_bytes;
    const size_t cap = room < ((size_t)16 << 20) ? room : ((size_t)16 << 20);
    for (size_t ks = 2; ks <= 16 && ks <= kt / 4; ks++) {
      if (ks * m * n * sizeof(float) > cap) break;
      const size_t t = ceil_div(sb * ks, (size_t)8) * (ceil_div(kt, ks) * 18 + 100) + 100;
      if (t < best_t) {
        best_t = t;
        best_ks = ks;
      }
    }
    if (best_ks >= 2) {
      pl.kt_per = (int)ceil_div(kt, best_ks);
      pl.splits = (int)ceil_div(kt, (size_t)pl.kt_per);
    }
  }
  return pl;
}

}  // namespace

size_t int4_gemm_ring_partial_bytes(const yscv_hip_int4_weight *w, size_t m, int num_cus) {
  if (!w->tiled || m <= 16) return 0;
  const RingPlan pl = ring_plan(m, w->n, w->kt, (size_t)(num_cus > 0 ? num_cus : 256));
  return pl.splits > 1 ? (size_t)pl.splits * m * w->n * sizeof(float) : 0;
}

int32_t launch_int4_gemm_ring(const yscv_hip_int4_weight *w, const _Float16 *xh, const float *row_scale, size_t k_pad,
                              void *y, int y_dtype, size_t m, hipStream_t s, int epi, float *partial, size_t partial_bytes) {
  if (epi == EPI_ADD_F32 && y_dtype != YSCV_HIP_F32) return set_error(YSCV_HIP_ERR_INVALID_ARG, "the add epilogue updates an f32 tensor");
  if (epi == EPI_SWIGLU && (w->n & 1)) return set_error(YSCV_HIP_ERR_INVALID_ARG, "SwiGLU epilogue needs an even row count");
  RingArgs a;
  a.epi = epi;
  a.tiles = w->tiles;
  a.tscales = w->tscales;
  a.tzps = w->has_zp ? w->tzps : nullptr;
  a.xh = xh;
  a.row_scale = row_scale;
  a.y = y;
  a.m = (int)m;
  a.n = (int)w->n;
  a.col0 = 0;
  a.ldy = (int)w->n;
  a.nt = (int)w->nt;
  a.kt = (int)w->kt;
  a.ktp = (int)w->ktp;
  a.chunks = (int)w->chunks;
  a.chunk_div = w->gm == GM128 ? (int)(w->g / 128) : 1;
  a.k_pad = (int)k_pad;
  a.y_dtype = y_dtype;
  a.partial = nullptr;
  a.kt_per = (int)w->kt;
  a.splits = 1;
  const bool sf16 = w->scale_dtype == YSCV_HIP_F16;
  const Context *ctx = nullptr;
  YSCV_TRY(ensure_context(&ctx));
  const RingPlan pl = ring_plan(m, w->n, w->kt, (size_t)(ctx->num_cus > 0 ? ctx->num_cus : 256));
  if (pl.splits > 1 && partial != nullptr && partial_bytes >= (size_t)pl.splits * m * w->n * sizeof(float) &&
      (reinterpret_cast<uintptr_t>(partial) & 15) == 0) {
    a.partial = partial;
    a.kt_per = pl.kt_per;
    a.splits = pl.splits;
  }
  auto launch_shape = [&](int which, const RingArgs &r) {
    switch (which) {
      case 4: return ring_launch_gm<2, 4, 2, 6, 8>(r, w->gm, sf16, s);
      case 3: return ring_launch_gm<1, 4, 2, 6, 4>(r, w->gm, sf16, s);
      case 2: return ring_launch_gm<8, 4, 2, 4, 4>(r, w->gm, sf16, s);
      case 1: return ring_launch_gm<4, 8, 2, 4, 4>(r, w->gm, sf16, s);
      default: return ring_launch_gm<4, 4, 2, 6, 8>(r, w->gm, sf16, s);
    }
  };
  if (pl.second < 0) return launch_shape(pl.one, a);
  RingArgs a1 = a, a2 = a;
  a1.n = (int)pl.split_col;
  a2.col0 = (int)pl.split_col;
  YSCV_TRY(launch_shape(pl.one, a1));
  return launch_shape(pl.second, a2);
}

}  // namespace yscv
