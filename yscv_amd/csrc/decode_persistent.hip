// Persistent batch-1 decode: one cooperative launch runs whole decode steps of the Llama-style
// decoder (the loop of apps/llm-bench/src/main.rs:525-548: feed the last token and the KV cache,
// take the greedy pick, repeat) with the int4 weights streamed exactly once per step.
//
// Why one launch: at batch 1 a decode step is ~4.3 GB of HBM traffic cut into ~160 dependent
// stages; as separate kernels every stage pays a launch and a cold start.  Here G workgroups (one per
// CU, 8 waves each) stay resident and
//   * every wave streams its own pre-ordered weight records (layout in persist.hpp) through a ring
//     in LDS filled by direct global->LDS loads; the ring keeps running across stage boundaries, so
//     the weights of the next stages are already in flight while a stage waits for its input;
//   * stages exchange their small activation vectors through "tagged entries" in global memory:
//     an 8-byte {payload, tag} word written with one agent-scope store and polled with coherent
//     128-bit loads.  A consumer wave waits for exactly the entries it needs, so there is no grid
//     barrier and no cache flush; the tag (step epoch, layer) makes stale data recognisable;
//   * the residual stream lives in registers of the threads that own its rows.
// Every wait is bounded: a wave that gives up sets abort_flag, every later wait returns at once and
// the host reports the failure.
//
// Arithmetic per 32-k block: one v_mfma_f32_16x16x32_f16.  With a single activation row the 16 rows
// of the A operand carry 16 different k-blocks of the activation (row i = k-block i of the wave's
// 512-k fragment), and the 16 columns of B carry 8 weight rows x 2 k-blocks, so each MFMA produces
// the dot products of 8 rows over two k-blocks in rows {j, j+4, ...} of D; the lanes that hold a
// useful element apply the group scale in fp32.  Weights stay exact integers (0x6400 | q = 1024 + q);
// the offset term sum_k x_k * (1024 + 8) is computed once per fragment by the same MFMA against a
// constant operand and subtracted per group.
//
// Semantics of the glue (tolerance-checked against the numpy restatement, like the multi-kernel path):
// RMSNorm crates/yscv-kernels/src/ops/norm.rs:1497-1518, RoPE ops/rope.rs:24-117, grouped-query
// attention crates/yscv-onnx/src/runner/linear.rs:552-646 over the fp16 cache, greedy pick = last
// maximal logit (apps/llm-bench/src/main.rs:538-543).
#include <hip/hip_runtime.h>

#include "int4_common.hpp"
#include "persist.hpp"

namespace yscv {

typedef unsigned long long u64;
// Stage timestamps (wall clock, per workgroup and layer) for performance work: build with
// -DYSCV_PERSIST_TRACE=1 (the decoder then allocates the [G][n_layers][PERSIST_TRACE_SLOTS] buffer).
#ifndef YSCV_PERSIST_TRACE
#define YSCV_PERSIST_TRACE 0
#endif
// records a producer may issue per served wave between two looks at its outstanding-load counter (measured with the
// scalar state machine: 1 -> 626, 2 -> 638, 3 -> 643, 4 -> 645, 5 -> 647, 7 -> 647, 10 -> 637 tokens/s: more amortises
// the bookkeeping, too many delay the publication of landed records)
#ifndef ISSUE_PER_ITER
#define ISSUE_PER_ITER 5
#endif
#ifndef INFLIGHT_CAP
#define INFLIGHT_CAP 20
#endif
#ifndef GEMV_INL
#define GEMV_INL __noinline__
#endif
// (the attention stages are inlined: as functions their argument structure travels through scratch memory, a memory
// round trip in front of each of them -- 668 -> 693 tokens/s; the projection stage stays a function: inlined at its
// five call sites, or with its arguments passed one by one in registers, the kernel is slower, 688 and 663)
#ifndef ATTN_INL
#define ATTN_INL __forceinline__
#endif

constexpr int CW = PS_WAVES;                   // compute waves per workgroup (waves 0 .. CW-1)
constexpr int PW = 4;                          // producer waves (waves CW .. CW+PW-1), each feeds CW/PW compute waves
constexpr int THREADS = 64 * (CW + PW);
constexpr int RING = 14;                       // ring slots (records) per compute wave
constexpr int SLOT = PS_REC_FULL;              // LDS bytes per ring slot
constexpr int RING_BYTES = CW * RING * SLOT;
constexpr int PART_ROWS = 256;                 // rows a workgroup may own in one projection
constexpr int PART_BYTES = 2 * CW * PART_ROWS * 4;
constexpr int ATT_BYTES = 10240;
constexpr int SYNC_BYTES = 256;                // landed[CW], consumed[CW], barrier counter
constexpr int PERSIST_LDS = RING_BYTES + PART_BYTES + ATT_BYTES + SYNC_BYTES;
constexpr int MAXF = 8;                        // 512-k fragments per compute wave: k <= 4 * 8 * 512
constexpr unsigned SPIN_LIMIT = 300000u;
constexpr int ACHUNK = 128;                    // positions per attention work item (4 waves x 32)
constexpr int PART_REC = 132;                  // entries per (head, chunk) partial: max, sum, o[128], pad

#define AS1(p) ((const void __attribute__((address_space(1))) *)(p))
#define AS3(p) ((void __attribute__((address_space(3))) *)(p))

__device__ __forceinline__ void st_entry(u64 *p, uint32_t payload, uint32_t tag) {
  __hip_atomic_store(p, ((u64)tag << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// coherent 128-bit load (two entries); the result is valid only after wait_vm
__device__ __forceinline__ uint4_t ld2(const void *p) {
  uint4_t v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ void wait_vm(uint4_t &a) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(a)::"memory"); }
__device__ __forceinline__ void wait_vm(uint4_t &a, uint4_t &b) {
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(a), "+v"(b)::"memory");
}
__device__ __forceinline__ void wait_vm(uint4_t &a, uint4_t &b, uint4_t &c, uint4_t &d) {
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d)::"memory");
}
__device__ __forceinline__ void wait_vm8(uint4_t *v) {
  asm volatile("s_waitcnt vmcnt(0)"
               : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])::"memory");
}
// LDS word access that the compiler does not order against outstanding global->LDS loads
__device__ __forceinline__ uint32_t lds_peek(uint32_t addr) {
  uint32_t v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ void lds_poke(uint32_t addr, uint32_t v) {
  asm volatile("ds_write_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" ::"v"(addr), "v"(v) : "memory");
}
// tags are compared on their low 24 bits; the top byte of the tag word may carry a block exponent
__device__ __forceinline__ bool tag_ok(uint32_t word, uint32_t tag) { return ((word ^ tag) & 0xFFFFFFu) == 0; }
__device__ __forceinline__ bool aborted(const PersistModel &m) {
  return __hip_atomic_load(m.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
}
__device__ __forceinline__ void set_abort(const PersistModel &m) {
  __hip_atomic_store(m.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
  a = fminf(fmaxf(a, -65504.0f), 65504.0f);
  b = fminf(fmaxf(b, -65504.0f), 65504.0f);
  U32H2 u;
  u.h = half2_t{(_Float16)a, (_Float16)b};
  return u.u;
}
__device__ __forceinline__ float h2_lo(uint32_t w) {
  U32H2 u;
  u.u = w;
  return (float)u.h[0];
}
__device__ __forceinline__ float h2_hi(uint32_t w) {
  U32H2 u;
  u.u = w;
  return (float)u.h[1];
}
__device__ __forceinline__ half8_t as_half8(uint4_t v) {
  union {
    uint4_t u;
    half8_t h;
  } x;
  x.u = v;
  return x.h;
}
// position of value i (even) of a k-vector inside its exchange buffer: fragment order of the consumer
__device__ __forceinline__ int xidx(int i, int ks, int frags) {
  const int v = i / ks;
  const int kk = i - v * ks;
  const int f = kk >> 9, k2 = kk & 511;
  const int r = k2 >> 5, c = (k2 >> 3) & 3, q = (k2 & 7) >> 1;
  return ((v * frags + f) << 8) + ((q >> 1) << 7) + 2 * (16 * c + r) + (q & 1);
}
__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + __expf(-g)); }
// order of the greedy pick: higher value wins, equal (or unordered) values -> larger index
__device__ __forceinline__ bool better(float va, int ia, float vb, int ib) {
  if (ia < 0) return false;
  if (ib < 0) return true;
  if (va > vb) return true;
  if (vb > va) return false;
  return ia > ib;
}

typedef __attribute__((address_space(3))) uint32_t lds_u32;
typedef __attribute__((address_space(3))) float lds_f32;
typedef __attribute__((address_space(3))) _Float16 lds_f16;

// state of the bounded waits and of the compute-wave barrier, carried by value through the noinline stages
struct WaitState {
  unsigned spin_budget;
  unsigned bar_gen;
};
__device__ __forceinline__ bool poll_backoff_ws(WaitState &ws, uint32_t *abort_flag) {
  __builtin_amdgcn_s_sleep(2);
  if (ws.spin_budget <= 1 ||
      ((ws.spin_budget & 63u) == 0 && __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
    __hip_atomic_store(abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ws.spin_budget = 1;
    return false;
  }
  ws.spin_budget--;
  return true;
}
// barrier of the compute waves (the producer waves never join, so s_barrier cannot be used)
// Every other wait of a compute wave is bounded, so every wave reaches its barriers; the bound here (minutes) only
// keeps a wave from spinning for ever should one of its workgroup have died.
__device__ __forceinline__ void compute_barrier(WaitState &ws, lds_u32 *ctr, int n_waves) {
  ws.bar_gen += n_waves;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  if ((threadIdx.x & 63) == 0) {
    __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    unsigned n = 0;
    while ((int)(__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) - ws.bar_gen) < 0 && ++n < 0x40000000u)
      __builtin_amdgcn_s_sleep(0);
  }
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
__device__ __forceinline__ half8_t gload_h8(const _Float16 *p) {
  return *reinterpret_cast<const half8_t __attribute__((address_space(1))) *>(reinterpret_cast<uintptr_t>(p));
}

struct AttnArgs {
  u64 *qkv, *part, *ao;
  _Float16 *kc, *vc;       // caches of this layer, batch row 0
  uint32_t *abort_flag;
  int HQ, HKV, GROUP, max_ctx, G, pos, pos0, wg;
  int ks_o, frags_o;       // k slice / fragments of the output projection (layout of `ao`)
  uint32_t tag;
  uint32_t att_off, bar_off;  // LDS byte offsets: attention scratch, barrier counter
  unsigned long long *dbg_t;  // null or timestamp slots
};

// Attention of the new token over the cached positions [0, pos): one work item = (kv head, 128 positions),
// four waves x 32 positions; writes one (max, sum, o[128]) partial per query head of the group.
__device__ ATTN_INL WaitState attn_items(AttnArgs a, WaitState ws) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  lds_f16 *p_lds = (lds_f16 *)(uintptr_t)a.att_off;                 // [4 waves][4 heads][32]
  lds_f32 *w_m = (lds_f32 *)(uintptr_t)(a.att_off + 1024);          // [4][4]
  lds_f32 *w_l = (lds_f32 *)(uintptr_t)(a.att_off + 1024 + 64);     // [4][4]
  lds_f32 *w_o = (lds_f32 *)(uintptr_t)(a.att_off + 1024 + 128);    // [4][4][128]
  lds_u32 *bar = (lds_u32 *)(uintptr_t)a.bar_off;
  const int pos = a.pos, GROUP = a.GROUP, HKV = a.HKV;
  const int nchunks = (pos + ACHUNK - 1) / ACHUNK;
  const int items = HKV * nchunks;
  const int max_chunks = a.max_ctx / ACHUNK;
  const uint32_t tag = a.tag;
  const float scale = 0.08838834764831845f;  // 1 / sqrt(128)
  if (YSCV_PERSIST_TRACE && a.dbg_t && tid == 0) a.dbg_t[14] = wall_clock64();
#pragma unroll 1
  for (int id = a.wg; id < items; id += a.G) {
    const int chunk = id / HKV, kvh = id - chunk * HKV;
    float m_h = -INFINITY, l_h = 0.0f;
    float o_acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++) o_acc[t] = 0.0f;
    const int p0 = chunk * ACHUNK + wave * 32;
    if (p0 < pos) {
      const _Float16 *kbase = a.kc + ((size_t)kvh * a.max_ctx + p0) * 128;
      const _Float16 *vbase = a.vc + (((size_t)kvh * (a.max_ctx / 8) + p0 / 8) * 128) * 8;
      half8_t kf[2][4], vf[8];
      const half8_t hz = {0, 0, 0, 0, 0, 0, 0, 0};
      // Blocks that were complete before this launch never change and are read with plain loads (issued
      // before the wait for q).  Positions appended during this launch were written with agent-scope
      // stores by another workgroup: their blocks are read with coherent loads, and only where valid.
      const bool recent = p0 + 32 > a.pos0;
      if (!recent) {
#pragma unroll
        for (int pbk = 0; pbk < 2; pbk++)
#pragma unroll
          for (int j = 0; j < 4; j++) kf[pbk][j] = gload_h8(kbase + (size_t)(pbk * 16 + r) * 128 + 32 * c + 8 * j);
#pragma unroll
        for (int t = 0; t < 8; t++) vf[t] = gload_h8(vbase + ((size_t)c * 128 + t * 16 + r) * 8);
      } else {
        uint4_t tmp[8];
#pragma unroll
        for (int pbk = 0; pbk < 2; pbk++)
#pragma unroll
          for (int j = 0; j < 4; j++) tmp[pbk * 4 + j] = ld2(kbase + (size_t)(pbk * 16 + r) * 128 + 32 * c + 8 * j);
        wait_vm8(tmp);
#pragma unroll
        for (int pbk = 0; pbk < 2; pbk++)
#pragma unroll
          for (int j = 0; j < 4; j++) kf[pbk][j] = (p0 + pbk * 16 + r) < pos ? as_half8(tmp[pbk * 4 + j]) : hz;
#pragma unroll
        for (int t = 0; t < 8; t++) tmp[t] = ld2(vbase + ((size_t)c * 128 + t * 16 + r) * 8);
        wait_vm8(tmp);
#pragma unroll
        for (int t = 0; t < 8; t++) vf[t] = as_half8(tmp[t]);
      }
      // Q operand: MFMA row 4*hh carries head hh of this group; lane (r, c) holds d = 32c + 8j + 0..7.
      // q arrives as fp16-pair entries in natural order: entry (head*128 + d) / 2.
      half8_t qa[4];
      {
        const int hh = r >> 2;
        const bool valid = ((r & 3) == 0) && hh < GROUP;
        const u64 *qsrc = a.qkv + ((size_t)(kvh * GROUP + (valid ? hh : 0)) * 128 + 32 * c) / 2;
        uint4_t qv[8];
        while (true) {
#pragma unroll
          for (int i = 0; i < 8; i++) qv[i] = ld2(qsrc + 2 * i);
          wait_vm8(qv);
          bool ok = true;
#pragma unroll
          for (int i = 0; i < 8; i++) ok = ok && tag_ok(qv[i][1], tag) && tag_ok(qv[i][3], tag);
          if (__all(ok || !valid)) break;
          if (!poll_backoff_ws(ws, a.abort_flag)) break;
        }
        if (YSCV_PERSIST_TRACE && a.dbg_t && tid == 0) a.dbg_t[15] = wall_clock64();
#pragma unroll
        for (int j = 0; j < 4; j++) {
          U32H2 e0, e1, e2, e3;
          e0.u = valid ? qv[2 * j][0] : 0u;
          e1.u = valid ? qv[2 * j][2] : 0u;
          e2.u = valid ? qv[2 * j + 1][0] : 0u;
          e3.u = valid ? qv[2 * j + 1][2] : 0u;
          qa[j] = half8_t{e0.h[0], e0.h[1], e1.h[0], e1.h[1], e2.h[0], e2.h[1], e3.h[0], e3.h[1]};
        }
      }
      float sc2[2];
#pragma unroll
      for (int pbk = 0; pbk < 2; pbk++) {
        float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; j++) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[j], kf[pbk][j], d, 0, 0, 0);
        const int p = p0 + pbk * 16 + r;  // lane (r, c): score of head c at position p
        sc2[pbk] = (p < pos) ? d[0] * scale : -INFINITY;
      }
      float mx = fmaxf(sc2[0], sc2[1]);
      mx = row_max16(mx);
      const float e0 = (sc2[0] == -INFINITY) ? 0.0f : __expf(sc2[0] - mx);
      const float e1 = (sc2[1] == -INFINITY) ? 0.0f : __expf(sc2[1] - mx);
      float sum = e0 + e1;
      sum = row_sum16(sum);
      m_h = mx;
      l_h = sum;
      lds_f16 *pw = p_lds + (size_t)wave * 4 * 32;
      pw[c * 32 + r] = (_Float16)e0;
      pw[c * 32 + 16 + r] = (_Float16)e1;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
      half8_t pa = {0, 0, 0, 0, 0, 0, 0, 0};
      if ((r & 3) == 0 && (r >> 2) < GROUP) {
        typedef __attribute__((address_space(3))) half8_t lds_h8;
        pa = *(const lds_h8 *)(pw + (r >> 2) * 32 + 8 * c);
      }
#pragma unroll
      for (int t = 0; t < 8; t++) {
        half8_t vv = vf[t];
        if (p0 + 8 * c >= pos) vv = hz;
        else if (p0 + 8 * c + 8 > pos) {
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (p0 + 8 * c + e >= pos) vv[e] = (_Float16)0.0f;
        }
        float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vv, d, 0, 0, 0);
        o_acc[t] = d[0];  // lane (r, c): o of head c at d = 16 t + r
      }
    }
    if (r == 0) {
      w_m[wave * 4 + c] = m_h;
      w_l[wave * 4 + c] = l_h;
    }
#pragma unroll
    for (int t = 0; t < 8; t++) w_o[((size_t)wave * 4 + c) * 128 + t * 16 + r] = o_acc[t];
    compute_barrier(ws, bar, CW);
    for (int idx = tid; idx < GROUP * 128; idx += 64 * CW) {
      const int hh = idx >> 7, dd = idx & 127;
      float mx = -INFINITY;
#pragma unroll
      for (int w = 0; w < 4; w++) mx = fmaxf(mx, w_m[w * 4 + hh]);
      float l = 0.0f, o = 0.0f;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        const float wm = w_m[w * 4 + hh];
        const float f = (wm == -INFINITY) ? 0.0f : __expf(wm - mx);
        l += w_l[w * 4 + hh] * f;
        o += w_o[((size_t)w * 4 + hh) * 128 + dd] * f;
      }
      u64 *dst = a.part + ((size_t)(kvh * GROUP + hh) * max_chunks + chunk) * PART_REC;
      st_entry(dst + 2 + dd, __float_as_uint(o), tag);
      if (dd == 0) {
        st_entry(dst, __float_as_uint(mx), tag);
        st_entry(dst + 1, __float_as_uint(l), tag);
      }
    }
    compute_barrier(ws, bar, CW);
  }
  return ws;
}

// Merge the chunk partials of one head with the token of this step (its k / v come straight from the qkv
// exchange buffer), publish the head's output, and append k / v to the cache (first head of each group).
// All compute waves of the workgroup take part: wave w merges chunks w, w + CW, ... (one round trip for up
// to five of them), the last wave also takes the token of this step, and wave 0 merges the CW states.
__device__ ATTN_INL WaitState attn_combine(AttnArgs a, WaitState ws, int head) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int pos = a.pos;
  const uint32_t tag = a.tag;
  const int nchunks = (pos + ACHUNK - 1) / ACHUNK;
  const int max_chunks = a.max_ctx / ACHUNK;
  const int kvh = head / a.GROUP;
  lds_f32 *cst = (lds_f32 *)(uintptr_t)(a.att_off + 1024 + 128);  // [CW][4][64] merge states (the w_o area)
  lds_u32 *bar = (lds_u32 *)(uintptr_t)a.bar_off;
  float M = -INFINITY, Ls = 0.0f, O0 = 0.0f, O1 = 0.0f;
  auto merge = [&](float mc, float lc, float o0, float o1) {
    if (mc == -INFINITY) return;
    const float Mn = fmaxf(M, mc);
    const float fa = (M == -INFINITY) ? 0.0f : __expf(M - Mn);
    const float fb = __expf(mc - Mn);
    Ls = Ls * fa + lc * fb;
    O0 = O0 * fa + o0 * fb;
    O1 = O1 * fa + o1 * fb;
    M = Mn;
  };
#pragma unroll 1
  for (int c0 = wave; c0 < nchunks; c0 += 5 * CW) {
    uint4_t v[10];
    while (true) {
#pragma unroll
      for (int i = 0; i < 5; i++) {
        const int ch = c0 + i * CW < nchunks ? c0 + i * CW : c0;
        const u64 *rec = a.part + ((size_t)head * max_chunks + ch) * PART_REC;
        v[2 * i] = ld2(rec);
        v[2 * i + 1] = ld2(rec + 2 + 2 * lane);
      }
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]),
                     "+v"(v[9])::"memory");
      bool ok = true;
#pragma unroll
      for (int i = 0; i < 10; i++) ok = ok && tag_ok(v[i][1], tag) && tag_ok(v[i][3], tag);
      if (__all(ok)) break;
      if (!poll_backoff_ws(ws, a.abort_flag)) break;
    }
#pragma unroll
    for (int i = 0; i < 5; i++)
      if (c0 + i * CW < nchunks)
        merge(__uint_as_float(v[2 * i][0]), __uint_as_float(v[2 * i][2]), __uint_as_float(v[2 * i + 1][0]),
              __uint_as_float(v[2 * i + 1][2]));
  }
  uint32_t kw = 0, vw = 0;
  if (wave == CW - 1) {
    const u64 *qe = a.qkv + (size_t)head * 64 + lane;
    const u64 *ke = a.qkv + (size_t)(a.HQ + kvh) * 64 + lane;
    const u64 *ve = a.qkv + (size_t)(a.HQ + a.HKV + kvh) * 64 + lane;
    u64 q, k, v;
    while (true) {
      q = __hip_atomic_load(qe, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      k = __hip_atomic_load(ke, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v = __hip_atomic_load(ve, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool ok = tag_ok((uint32_t)(q >> 32), tag) && tag_ok((uint32_t)(k >> 32), tag) && tag_ok((uint32_t)(v >> 32), tag);
      if (__all(ok)) break;
      if (!poll_backoff_ws(ws, a.abort_flag)) break;
    }
    const uint32_t qw = (uint32_t)q;
    kw = (uint32_t)k;
    vw = (uint32_t)v;
    const float s = wave_sum(h2_lo(qw) * h2_lo(kw) + h2_hi(qw) * h2_hi(kw)) * 0.08838834764831845f;
    merge(s, 1.0f, h2_lo(vw), h2_hi(vw));
    if (head == kvh * a.GROUP) {
      // append: other workgroups read these lines in later steps of this launch -> agent-scope stores
      uint32_t *krow = reinterpret_cast<uint32_t *>(a.kc + ((size_t)kvh * a.max_ctx + pos) * 128);
      __hip_atomic_store(krow + lane, kw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      uint16_t *vslab = reinterpret_cast<uint16_t *>(a.vc + (((size_t)kvh * (a.max_ctx / 8) + pos / 8) * 128) * 8) + (pos & 7);
      __hip_atomic_store(vslab + (size_t)(2 * lane) * 8, (uint16_t)(vw & 0xFFFFu), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(vslab + (size_t)(2 * lane + 1) * 8, (uint16_t)(vw >> 16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  lds_f32 *mine = cst + (size_t)wave * 256;
  mine[lane] = M;
  mine[64 + lane] = Ls;
  mine[128 + lane] = O0;
  mine[192 + lane] = O1;
  compute_barrier(ws, bar, CW);
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < CW; w++) {
      const lds_f32 *o = cst + (size_t)w * 256;
      merge(o[lane], o[64 + lane], o[128 + lane], o[192 + lane]);
    }
    const float inv = Ls > 0.0f ? 1.0f / Ls : 0.0f;
    st_entry(a.ao + xidx(head * 128 + 2 * lane, a.ks_o, a.frags_o), pack_h2(O0 * inv, O1 * inv), tag);
  }
  compute_barrier(ws, bar, CW);  // the merge states are reused by the next head / the next attention item
  return ws;
}

struct GemvArgs {
  const u64 *in_buf, *ss;        // exchange vector of the activation; sum-of-squares entries behind it or null
  uint32_t *abort_flag;
  unsigned long long *dbg_t;     // null or two timestamp slots (input arrived, blocks done)
  uint32_t tag;
  int ks, frags, pairs, odd, nb, ss_count, d_model;
  float eps;
  uint32_t ring_off, part_off, sync_off;  // LDS byte addresses: this wave's ring, its row-sum slots, sync words
};
struct GemvState {
  unsigned crec;   // weight records this wave has consumed in this launch
  WaitState ws;
};

// One projection for one compute wave: waits for its slice of the activation, then consumes the records
// of every 8-row block this workgroup owns and leaves one partial row sum per row in LDS (the caller adds
// the CW slices).  Ends with the barrier of the compute waves.
__device__ GEMV_INL GemvState gemv_stage(GemvArgs a, GemvState st) {
  // arguments of a non-kernel function arrive in vector registers: tell the compiler which are wave-uniform
  a.tag = __builtin_amdgcn_readfirstlane(a.tag);
  a.ks = __builtin_amdgcn_readfirstlane(a.ks);
  a.frags = __builtin_amdgcn_readfirstlane(a.frags);
  a.pairs = __builtin_amdgcn_readfirstlane(a.pairs);
  a.odd = __builtin_amdgcn_readfirstlane(a.odd);
  a.nb = __builtin_amdgcn_readfirstlane(a.nb);
  a.ss_count = __builtin_amdgcn_readfirstlane(a.ss_count);
  a.ring_off = __builtin_amdgcn_readfirstlane(a.ring_off);
  a.part_off = __builtin_amdgcn_readfirstlane(a.part_off);
  a.sync_off = __builtin_amdgcn_readfirstlane(a.sync_off);
  st.crec = __builtin_amdgcn_readfirstlane(st.crec);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, c = lane >> 4;
  lds_u32 *sync = (lds_u32 *)(uintptr_t)a.sync_off;
  lds_f32 *dst = (lds_f32 *)(uintptr_t)a.part_off;
  // The decode constants are kept in registers the compiler cannot see through, so that (s & mask) | magic
  // becomes one three-register v_and_or_b32 instead of two literal-operand instructions.  (An inline-asm
  // v_and_or_b32 is not an option: the hazard recognizer does not see it overwrite a register that a
  // matrix instruction is still writing.)
  uint32_t magic = 0x64006400u, mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u;
  asm volatile("" : "+v"(magic), "+v"(mask_lo), "+v"(mask_hi));
  const uint32_t tag = a.tag;
  half8_t xa[MAXF];
  float4_t z[MAXF];
  float rstd = 1.0f;
  const half8_t bc = {(_Float16)1032.0f, (_Float16)1032.0f, (_Float16)1152.0f, (_Float16)1152.0f,
                      (_Float16)1032.0f, (_Float16)1032.0f, (_Float16)1152.0f, (_Float16)1152.0f};
  const bool normed = a.ss != nullptr;
  // ---- activation fragments (A operand: row i = k-block i of the fragment) ------------------------------
  // A `normed` vector holds fp16(h * gamma * 2^-e) with the exponent e of each 8-row block in the top byte
  // of its tag words; the operand is then fp16(h * gamma / rms), the activation RMSNorm feeds
  // (crates/yscv-kernels/src/ops/norm.rs:1497-1518); 1/rms comes from the sum-of-squares entries.
  {
    uint4_t qa[MAXF], qb[MAXF], sa, sb;
    const bool v0 = normed && 4 * lane < a.ss_count, v1 = normed && 4 * lane + 1 < a.ss_count,
               v2 = normed && 4 * lane + 2 < a.ss_count, v3 = normed && 4 * lane + 3 < a.ss_count;
    const u64 *sp = normed ? a.ss + 4 * lane : a.in_buf;
    const u64 *p0 = a.in_buf + (((size_t)wave * a.frags) << 8) + 2 * lane;
    if (a.nb > 0) {
      while (true) {  // one round trip for all fragments and the sum-of-squares entries
#pragma unroll
        for (int f = 0; f < MAXF; f++) {
          if (f < a.frags) {  // wave-uniform
            qa[f] = ld2(p0 + ((size_t)f << 8));
            qb[f] = ld2(p0 + ((size_t)f << 8) + 128);
          }
        }
        sa = ld2(sp);
        sb = ld2(sp + 2);
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(qa[0]), "+v"(qa[1]), "+v"(qa[2]), "+v"(qa[3]), "+v"(qa[4]), "+v"(qa[5]), "+v"(qa[6]), "+v"(qa[7]),
                       "+v"(qb[0]), "+v"(qb[1]), "+v"(qb[2]), "+v"(qb[3]), "+v"(qb[4]), "+v"(qb[5]), "+v"(qb[6]), "+v"(qb[7]),
                       "+v"(sa), "+v"(sb)::"memory");
        bool ok = (!v0 || tag_ok(sa[1], tag)) && (!v1 || tag_ok(sa[3], tag)) && (!v2 || tag_ok(sb[1], tag)) &&
                  (!v3 || tag_ok(sb[3], tag));
#pragma unroll
        for (int f = 0; f < MAXF; f++) {
          const bool valid = f < a.frags && (512 * f + 32 * r) < a.ks;
          ok = ok && (!valid || (tag_ok(qa[f][1], tag) && tag_ok(qa[f][3], tag) && tag_ok(qb[f][1], tag) && tag_ok(qb[f][3], tag)));
        }
        if (__all(ok)) break;
        if (!poll_backoff_ws(st.ws, a.abort_flag)) break;
      }
    }
    if (normed) {
      const float sq = (v0 ? __uint_as_float(sa[0]) : 0.0f) + (v1 ? __uint_as_float(sa[2]) : 0.0f) +
                       (v2 ? __uint_as_float(sb[0]) : 0.0f) + (v3 ? __uint_as_float(sb[2]) : 0.0f);
      rstd = 1.0f / sqrtf(wave_sum(sq) / (float)a.d_model + a.eps);
    }
#pragma unroll
    for (int f = 0; f < MAXF; f++) {
      if (f < a.frags && a.nb > 0) {
        const bool valid = (512 * f + 32 * r) < a.ks;
        U32H2 u0, u1, u2, u3;
        u0.u = valid ? qa[f][0] : 0u;
        u1.u = valid ? qa[f][2] : 0u;
        u2.u = valid ? qb[f][0] : 0u;
        u3.u = valid ? qb[f][2] : 0u;
        if (normed) {
          const float fac = valid ? ldexpf(rstd, (int)(qa[f][1] >> 24) - 128) : 0.0f;
          u0.h = half2_t{(_Float16)((float)u0.h[0] * fac), (_Float16)((float)u0.h[1] * fac)};
          u1.h = half2_t{(_Float16)((float)u1.h[0] * fac), (_Float16)((float)u1.h[1] * fac)};
          u2.h = half2_t{(_Float16)((float)u2.h[0] * fac), (_Float16)((float)u2.h[1] * fac)};
          u3.h = half2_t{(_Float16)((float)u3.h[0] * fac), (_Float16)((float)u3.h[1] * fac)};
        }
        // the slots that meet 1024 + 16 q carry x / 16 (exact: a power of two)
        const half2_t sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
        u1.h = u1.h * sixteenth;
        u3.h = u3.h * sixteenth;
        xa[f] = half8_t{u0.h[0], u0.h[1], u1.h[0], u1.h[1], u2.h[0], u2.h[1], u3.h[0], u3.h[1]};
        const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
        z[f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[f], bc, zero, 0, 0, 0);  // offset term of every k-block
      } else {
        xa[f] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        z[f] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
  }
  if (YSCV_PERSIST_TRACE && a.dbg_t && threadIdx.x == 0) a.dbg_t[0] = wall_clock64();

  // ---- one record: 8 rows x 512 k against fragment xa ------------------------------------------------------
  unsigned crec = st.crec;
  unsigned landed_seen = st.crec;  // the producer's count as last read: while it is ahead, no record waits for a poll
  unsigned spins = 0;              // one budget for all records of the stage: a stalled stream costs it once, not per record
  auto consume = [&](bool single, const half8_t &xf, const float4_t &zf, float &acc) {
    if ((int)(landed_seen - (crec + 1)) < 0) {
      while ((int)((landed_seen = __builtin_amdgcn_readfirstlane(
                        __hip_atomic_load(sync + wave, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP))) -
                   (crec + 1)) < 0) {
        __builtin_amdgcn_s_sleep(0);
        // the stream stalled (never expected) or another wave has given up: no wait here is unbounded
        if (++spins > 40000000u ||
            ((spins & 4095u) == 0 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
          __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          spins = 40000000u;
          break;
        }
      }
    }
    const uint32_t slot = crec % RING;
    const uint32_t a_w = a.ring_off + slot * SLOT + lane * 16;
    const uint32_t a_s = a.ring_off + slot * SLOT + (c >> 1) * 128 + r * 8;
    uint4_t w0, w1;
    typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
    uint2_t sc;
    asm volatile(
        "ds_read_b128 %0, %3\n\tds_read_b128 %1, %3 offset:1024\n\tds_read_b64 %2, %4 offset:2048\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(w0), "=&v"(w1), "=&v"(sc)
        : "v"(a_w), "v"(a_s)
        : "memory");
    crec++;
    if (lane == 0) __hip_atomic_store(sync + 8 + wave, crec, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
    float d0[4], d1[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      U32H2 q0, q1, q2, q3;
      const uint32_t s = w0[j], s2 = s >> 8;
      q0.u = (s & mask_lo) | magic;
      q1.u = (s & mask_hi) | magic;
      q2.u = (s2 & mask_lo) | magic;
      q3.u = (s2 & mask_hi) | magic;
      const half8_t b = {q0.h[0], q0.h[1], q1.h[0], q1.h[1], q2.h[0], q2.h[1], q3.h[0], q3.h[1]};
      const float4_t dd = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf, b, zero, 0, 0, 0);
      d0[j] = dd[j];
    }
    if (!single) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        U32H2 q0, q1, q2, q3;
        const uint32_t s = w1[j], s2 = s >> 8;
        q0.u = (s & mask_lo) | magic;
        q1.u = (s & mask_hi) | magic;
        q2.u = (s2 & mask_lo) | magic;
        q3.u = (s2 & mask_hi) | magic;
        const half8_t b = {q0.h[0], q0.h[1], q1.h[0], q1.h[1], q2.h[0], q2.h[1], q3.h[0], q3.h[1]};
        const float4_t dd = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf, b, zero, 0, 0, 0);
        d1[j] = dd[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) d1[j] = 0.0f;
    }
    const bool second = (c >> 1) != 0;
    const float s0 = h2_lo(sc[0]), s1 = h2_hi(sc[0]), s2 = h2_lo(sc[1]), s3 = h2_hi(sc[1]);
    acc = fmaf(s0, (second ? d1[0] : d0[0]) - zf[0], acc);
    acc = fmaf(s1, (second ? d1[1] : d0[1]) - zf[1], acc);
    acc = fmaf(s2, (second ? d1[2] : d0[2]) - zf[2], acc);
    acc = fmaf(s3, (second ? d1[3] : d0[3]) - zf[3], acc);
  };

  const bool useful = (c & 1) == (r >> 3);
#pragma unroll 1
  for (int blk = 0; blk < a.nb; blk++) {
    float acc = 0.0f;
#pragma unroll
    for (int p = 0; p < MAXF; p++)
      if (p < a.pairs) consume(a.odd && p == a.pairs - 1, xa[p], z[p], acc);
    acc = useful ? acc : 0.0f;
    acc += dpp_move<DPP_ROR8>(acc);
    acc = sum_xor16_xor32(acc);
    if (lane < 8) dst[blk * 8 + lane] = acc;
  }
  if (YSCV_PERSIST_TRACE && a.dbg_t && threadIdx.x == 0) a.dbg_t[1] = wall_clock64();
  st.crec = crec;
  compute_barrier(st.ws, sync + 16, CW);
  return st;
}

__global__ void __launch_bounds__(THREADS, 1)
decode_persistent_kernel(PersistModel m, int n_steps, int pos0, int step0, int max_steps, uint32_t epoch0) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  float *part_lds = reinterpret_cast<float *>(lds + RING_BYTES);                 // [2][8][PART_ROWS]
  unsigned char *att_lds = lds + RING_BYTES + PART_BYTES;
  int *tok_lds = reinterpret_cast<int *>(att_lds + 1024 + 128 + 8192);            // [1]
  float *arg_v = reinterpret_cast<float *>(att_lds + 1024 + 128 + 8192 + 64);     // [8]
  int *arg_i = reinterpret_cast<int *>(att_lds + 1024 + 128 + 8192 + 128);        // [8]
  lds_u32 *sync = (lds_u32 *)(lds + RING_BYTES + PART_BYTES + ATT_BYTES);  // [0..CW) landed, [8..8+CW) consumed, [16] barrier

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wg = blockIdx.x;
  const int G = m.G;
  const int L = m.n_layers;
  const int D = m.d_model;
  const int HQ = m.n_heads, HKV = m.n_kv_heads, GROUP = HQ / HKV;

  auto nbw = [&](int kind) { return wg < m.ph[kind].nb ? (m.ph[kind].nb - wg + G - 1) / G : 0; };
  int dbg_layer = 0;
  auto mark = [&](int idx) {
    if (YSCV_PERSIST_TRACE && m.dbg_t && tid == 0) m.dbg_t[((size_t)wg * L + dbg_layer) * PERSIST_TRACE_SLOTS + idx] = wall_clock64();
  };
  if (tid < 32) sync[tid] = 0;
  __syncthreads();

  // ---- producer waves: stream the weight records of their compute waves into the LDS rings -------------
  // A producer issues a record (3 direct global->LDS loads) whenever a ring of one of its waves has a free
  // slot, and publishes how many records have landed, which it reads from its own outstanding-load counter
  // (loads return in order).  Compute waves never have a weight load of their own in flight, so their polls
  // are not queued behind the stream.  The LDS words shared with the compute waves are accessed with explicit
  // ds instructions: a compiler-visible LDS read would be ordered behind every outstanding LDS-bound load.
  if (wave >= CW) {
    const uint32_t sync_lds = (uint32_t)(size_t)(lds + RING_BYTES + PART_BYTES + ATT_BYTES);
  {
    constexpr int SERVED = CW / PW;
    const int p = wave - CW;
    const uint32_t lds_base = (uint32_t)(size_t)lds;
    int nb_k[PK_COUNT], pairs_k[PK_COUNT], odd_k[PK_COUNT];
    unsigned per_step = 0;
#pragma unroll
    for (int k = 0; k < PK_COUNT; k++) {
      nb_k[k] = nbw(k);
      pairs_k[k] = m.ph[k].pairs;
      odd_k[k] = m.ph[k].tiles & 1;
      per_step += (unsigned)nb_k[k] * pairs_k[k] * (k == PK_LM ? 1 : L);
    }
    const unsigned total = per_step * (unsigned)n_steps;  // records per compute wave in this launch
    const unsigned char *base[SERVED], *ptr[SERVED];
    int kind[SERVED], layer[SERVED], blk[SERVED], pair[SERVED];
    unsigned issued[SERVED], landed_cnt[SERVED], consumed_seen[SERVED];
#pragma unroll
    for (int j = 0; j < SERVED; j++) {
      const int w = p * SERVED + j;
      base[j] = ptr[j] = m.stream + m.wg_off[wg] + (size_t)w * m.wave_bytes[wg];
      kind[j] = layer[j] = blk[j] = pair[j] = 0;
      issued[j] = landed_cnt[j] = consumed_seen[j] = 0;
    }
    unsigned long long fifo = 0;  // bit (i & 63): which served wave the i-th issued record belongs to
    unsigned n_issued = 0, n_retired = 0;
    auto kv = [&](const int *arr, int k) {  // 5-entry table lookup without dynamic register indexing
      return k == 0 ? arr[0] : (k == 1 ? arr[1] : (k == 2 ? arr[2] : (k == 3 ? arr[3] : arr[4])));
    };
    if (total > 0) {
      while (n_retired < total * SERVED) {
        bool did = false;
#pragma unroll
        for (int jj = 0; jj < SERVED * ISSUE_PER_ITER; jj++) {
          const int j = jj % SERVED;
          const int w = p * SERVED + j;
          // the consumer's count is read again only when the last value read leaves no free slot
          if (issued[j] < total && n_issued - n_retired < INFLIGHT_CAP && issued[j] - consumed_seen[j] >= RING)
            consumed_seen[j] = __builtin_amdgcn_readfirstlane(lds_peek(sync_lds + 4 * (8 + w)));  // uniform: keeps the state machine scalar
          if (issued[j] < total && n_issued - n_retired < INFLIGHT_CAP && issued[j] - consumed_seen[j] < RING) {
            while (kv(nb_k, kind[j]) == 0) {  // kinds this workgroup has no rows of
              if (kind[j] == PK_DOWN) { layer[j]++; kind[j] = layer[j] == L ? PK_LM : PK_QKV; }
              else if (kind[j] == PK_LM) { layer[j] = 0; kind[j] = PK_QKV; ptr[j] = base[j]; }
              else kind[j]++;
            }
            const int pairs = kv(pairs_k, kind[j]);
            const bool single = (pair[j] == pairs - 1) && kv(odd_k, kind[j]);
            const uint32_t dst = lds_base + (uint32_t)((w * RING + issued[j] % RING) * SLOT);
            const unsigned char *src = ptr[j];
            __builtin_amdgcn_global_load_lds(AS1(src + lane * 16), (void __attribute__((address_space(3))) *)(uintptr_t)(dst), 16, 0, 2);
            __builtin_amdgcn_global_load_lds(AS1(src + (single ? 0 : 1024) + lane * 16), (void __attribute__((address_space(3))) *)(uintptr_t)(dst + 1024), 16, 0, 2);
            __builtin_amdgcn_global_load_lds(AS1(src + (single ? 1024 : 2048) + lane * 4), (void __attribute__((address_space(3))) *)(uintptr_t)(dst + 2048), 4, 0, 2);
            ptr[j] += single ? PS_REC_SINGLE : PS_REC_FULL;
            issued[j]++;
            fifo = (fifo & ~(1ull << (n_issued & 63))) | ((unsigned long long)j << (n_issued & 63));
            n_issued++;
            did = true;
            if (++pair[j] == pairs) {
              pair[j] = 0;
              if (++blk[j] >= kv(nb_k, kind[j])) {
                blk[j] = 0;
                if (kind[j] == PK_DOWN) { layer[j]++; kind[j] = layer[j] == L ? PK_LM : PK_QKV; }
                else if (kind[j] == PK_LM) { layer[j] = 0; kind[j] = PK_QKV; ptr[j] = base[j]; }
                else kind[j]++;
              }
            }
          }
        }
        // outstanding vector-memory operations of this wave: IB_STS.vm_cnt (bits 3:0 and 23:22)
        // (read after the issues above: the clobber keeps the compiler from moving it across them)
        unsigned ib_sts;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_IB_STS)" : "=s"(ib_sts)::"memory");
        const unsigned vm = (ib_sts & 15u) | (((ib_sts >> 22) & 3u) << 4);
        const unsigned done = n_issued - (vm + 2) / 3;
        bool dirty = false;
        while ((int)(done - n_retired) > 0) {
          const int j = (int)((fifo >> (n_retired & 63)) & 1ull);
          if (j == 0) landed_cnt[0]++; else landed_cnt[SERVED - 1]++;
          n_retired++;
          dirty = true;
        }
        if (dirty) {
#pragma unroll
          for (int j = 0; j < SERVED; j++)
            lds_poke(sync_lds + 4 * (p * SERVED + j), landed_cnt[j]);
        }
        if (!did && !dirty) __builtin_amdgcn_s_sleep(1);
      }
    }
  }
    return;
  }

  // ---- compute waves ---------------------------------------------------------------------------------
  const uint32_t ring_lds = (uint32_t)(size_t)(lds + (size_t)wave * RING * SLOT);  // LDS byte address of this wave's ring
  WaitState ws{SPIN_LIMIT, 0};
  auto cbar = [&]() { compute_barrier(ws, sync + 16, CW); };

  int pb = 0;
  const int ss_count = m.ph[PK_O].nb < G ? m.ph[PK_O].nb : G;
  unsigned crec = 0;  // weight records this wave has consumed in this launch
  auto gemv = [&](int kind, const u64 *in_buf, uint32_t tag, bool with_ss, int mk) {
    GemvArgs ga;
    ga.in_buf = in_buf;
    ga.ss = with_ss ? in_buf + persist_vec_entries(m.ph[kind].k) : nullptr;
    ga.abort_flag = m.abort_flag;
    ga.dbg_t = (YSCV_PERSIST_TRACE && m.dbg_t) ? m.dbg_t + ((size_t)wg * L + dbg_layer) * PERSIST_TRACE_SLOTS + mk : nullptr;
    ga.tag = tag;
    ga.ks = m.ph[kind].ks;
    ga.frags = m.ph[kind].frags;
    ga.pairs = m.ph[kind].pairs;
    ga.odd = m.ph[kind].tiles & 1;
    ga.nb = nbw(kind);
    ga.ss_count = ss_count;
    ga.d_model = D;
    ga.eps = m.eps;
    ga.ring_off = ring_lds;
    ga.part_off = (uint32_t)(size_t)(part_lds + ((size_t)pb * CW + wave) * PART_ROWS);
    ga.sync_off = (uint32_t)(size_t)(lds + RING_BYTES + PART_BYTES + ATT_BYTES);
    const GemvState gs = gemv_stage(ga, GemvState{crec, ws});
    crec = gs.crec;
    ws = gs.ws;
  };
  auto row_sum = [&](int row_slot) -> float {
    const float *src = part_lds + (size_t)pb * CW * PART_ROWS + row_slot;
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < CW; w++) v += src[w * PART_ROWS];
    return v;
  };

  // ---- residual stream: thread t < 8 * nbw(PK_O) owns row 8 * (wg + G * (t >> 3)) + (t & 7) ---------
  const int nb_d = nbw(PK_O);
  const bool own = tid < 8 * nb_d;  // 8 * nb_d <= 64: all owners sit in wave 0
  const int own_row = 8 * (wg + G * (tid >> 3)) + (tid & 7);
  float h = 0.0f;
  // publish fp16(h * gamma * 2^-e) pairs (fragment order of a k = d_model consumer; e = exponent of the largest
  // value of the 8-row block, carried in the top byte of the tag word) + this workgroup's sum of squares
  auto publish_h = [&](u64 *buf, float gamma, uint32_t tag) {
    if (tid < 64) {
      const float xs = own ? h * gamma : 0.0f;
      float mx = fabsf(xs);
      mx = fmaxf(mx, dpp_move<DPP_XOR1>(mx));
      mx = fmaxf(mx, dpp_move<DPP_XOR2>(mx));
      mx = fmaxf(mx, dpp_move<DPP_HALF_MIRROR>(mx));
      int e = (mx > 0.0f && mx < INFINITY) ? ilogbf(mx) + 1 : 0;
      e = e < -100 ? -100 : (e > 100 ? 100 : e);
      const float sc = ldexpf(xs, -e);
      const float nxt = dpp_move<DPP_NEXT1>(sc);  // used by even lanes only
      if (own && !(tid & 1))
        st_entry(buf + xidx(own_row, m.ph[PK_QKV].ks, m.ph[PK_QKV].frags), pack_h2(sc, nxt), tag | ((uint32_t)(e + 128) << 24));
      const float ss = wave_sum(own ? h * h : 0.0f);
      if (tid == 0 && nb_d > 0) st_entry(buf + persist_vec_entries(D) + wg, __float_as_uint(ss), tag);
    }
  };

  // ---- the decode loop ---------------------------------------------------------------------------------
  if (tid == 0) tok_lds[0] = m.tokens[0];
  cbar();
  int token = tok_lds[0];
  const float *gam = m.gammas;

#pragma unroll 1
  for (int s = 0; s < n_steps; s++) {
    const int pos = pos0 + s;
    const uint32_t tag_base = (epoch0 + (uint32_t)s) * (uint32_t)(L + 2) + 1u;  // used modulo 2^24
    ws.spin_budget = ws.spin_budget > 1 ? SPIN_LIMIT : 1;
    token = token < 0 ? 0 : (token >= m.vocab ? m.vocab - 1 : token);
    if (own) h = (float)m.emb[(size_t)token * D + own_row];
    publish_h(m.xn, own ? gam[own_row] : 0.0f, tag_base & 0xFFFFFFu);

#pragma unroll 1
    for (int l = 0; l < L; l++) {
      const uint32_t tag = (tag_base + (uint32_t)l) & 0xFFFFFFu;
      dbg_layer = l;
      mark(0);
      // ---- q/k/v projection + rotary embedding ------------------------------------------------------------
      {
        const int nb = nbw(PK_QKV);
        const bool act = tid < 8 * nb;
        const int pr = 8 * (wg + G * (tid >> 3)) + (tid & 7);  // row in stream order
        const bool rot = act && pr < (HQ + HKV) * 128;
        float sn = 0.0f, cs = 1.0f;
        if (rot) {
          const int i = (pr & 127) >> 1;
          const float inv_freq = 1.0f / powf(m.theta, (float)(2 * i) / 128.0f);
          sincosf(inv_freq * (float)pos, &sn, &cs);
        }
        gemv(PK_QKV, m.xn, tag, true, 1);
        const float val = act ? row_sum(tid) : 0.0f;
        const float partner = dpp_move<DPP_XOR1>(val);
        const int which = pr & 1;
        const float x0 = which ? partner : val, x1 = which ? val : partner;
        const float rotated = which ? x0 * sn + x1 * cs : x0 * cs - x1 * sn;
        const float out = rot ? rotated : val;
        const float out2 = dpp_move<DPP_NEXT2>(out);  // same member of the next rotary pair (read by lanes 0, 1 of a quad)
        const float out1 = dpp_move<DPP_NEXT1>(out);  // next row (v rows are in natural order; read by even lanes)
        if (act) {
          if (rot) {
            if (!(tid & 2)) {
              const int head = pr >> 7, i = (pr & 127) >> 1;
              const int dim = i + 64 * which;
              st_entry(m.qkv + (head * 128 + dim) / 2, pack_h2(out, out2), tag);
            }
          } else if (!(tid & 1)) {
            st_entry(m.qkv + pr / 2, pack_h2(out, out1), tag);
          }
        }
        pb ^= 1;
        mark(3);
      }
      // ---- attention -------------------------------------------------------------------------------------
      {
        AttnArgs aa;
        aa.qkv = m.qkv; aa.part = m.part; aa.ao = m.ao;
        aa.kc = m.kc[l]; aa.vc = m.vc[l];
        aa.abort_flag = m.abort_flag;
        aa.HQ = HQ; aa.HKV = HKV; aa.GROUP = GROUP; aa.max_ctx = m.max_ctx; aa.G = G; aa.pos = pos; aa.pos0 = pos0; aa.wg = wg;
        aa.ks_o = m.ph[PK_O].ks; aa.frags_o = m.ph[PK_O].frags;
        aa.tag = tag;
        aa.att_off = (uint32_t)(size_t)att_lds;
        aa.bar_off = (uint32_t)(size_t)(lds + RING_BYTES + PART_BYTES + ATT_BYTES) + 64;
        aa.dbg_t = (YSCV_PERSIST_TRACE && m.dbg_t) ? m.dbg_t + ((size_t)wg * L + l) * PERSIST_TRACE_SLOTS : nullptr;
        ws = attn_items(aa, ws);
        mark(4);
        for (int head = G - 1 - wg; head < HQ; head += G) ws = attn_combine(aa, ws, head);
        mark(16);
      }
      // ---- output projection + residual ------------------------------------------------------------------
      {
        const float g_next = own ? gam[(size_t)(2 * l + 1) * D + own_row] : 0.0f;  // in flight during the stage
        gemv(PK_O, m.ao, tag, false, 5);
        if (own) h += row_sum(tid);
        publish_h(m.xn2, g_next, tag);
        pb ^= 1;
        mark(7);
      }
      // ---- gate / up projection + SwiGLU (rows interleaved: 2i = gate_i, 2i+1 = up_i) ---------------------
      {
        const int nb = nbw(PK_GU);
        gemv(PK_GU, m.xn2, tag, true, 8);
        const bool act = tid < 8 * nb;
        const int pr = 8 * (wg + G * (tid >> 3)) + (tid & 7);
        const float val = act ? row_sum(tid) : 0.0f;
        const float up = dpp_move<DPP_NEXT1>(val);
        const float a = silu_f(val) * up;          // meaningful in even threads
        const float a2 = dpp_move<DPP_NEXT2>(a);   // act value of the next pair of rows (read by lane 0 of a quad)
        if (act && !(tid & 3)) st_entry(m.act + xidx(pr / 2, m.ph[PK_DOWN].ks, m.ph[PK_DOWN].frags), pack_h2(a, a2), tag);
        pb ^= 1;
        mark(10);
      }
      // ---- down projection + residual; publishes the input of the next layer (or of lm_head) ---------------
      {
        const float g_next = own ? gam[(size_t)(l + 1 < L ? 2 * (l + 1) : 2 * L) * D + own_row] : 0.0f;
        gemv(PK_DOWN, m.act, tag, false, 11);
        if (own) h += row_sum(tid);
        publish_h(m.xn, g_next, (tag + 1) & 0xFFFFFFu);
        pb ^= 1;
        mark(13);
      }
    }
    // ---- lm_head + greedy pick -----------------------------------------------------------------------------
    {
      const uint32_t tag = (tag_base + (uint32_t)L) & 0xFFFFFFu;
      const int nb = nbw(PK_LM);
      gemv(PK_LM, m.xn, tag, true, 14);
      const bool act = tid < 8 * nb;
      const int row = 8 * (wg + G * (tid >> 3)) + (tid & 7);
      float best = 0.0f;
      int bi = -1;
      if (act) {
        best = row_sum(tid);
        bi = row;
        m.logits[row] = best;
      }
      pb ^= 1;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (better(ov, oi, best, bi)) {
          best = ov;
          bi = oi;
        }
      }
      if (lane == 0) {
        arg_v[wave] = best;
        arg_i[wave] = bi;
      }
      cbar();
      if (wave == 0) {
        if (lane == 0 && nb > 0) {
          for (int w = 1; w < CW; w++)
            if (better(arg_v[w], arg_i[w], best, bi)) {
              best = arg_v[w];
              bi = arg_i[w];
            }
          st_entry(m.arg + 2 * wg, __float_as_uint(best), tag);
          st_entry(m.arg + 2 * wg + 1, (uint32_t)bi, tag);
        }
        // every workgroup merges the per-workgroup picks itself: no second exchange for the token
        const int cnt = m.ph[PK_LM].nb < G ? m.ph[PK_LM].nb : G;
        float gv = 0.0f;
        int gi = -1;
        for (int w0 = 0; w0 < cnt; w0 += 64) {
          const int w = w0 + lane;
          uint4_t e;
          while (true) {
            e = ld2(m.arg + 2 * (w < cnt ? w : 0));
            wait_vm(e);
            const bool ok = w >= cnt || (tag_ok(e[1], tag) && tag_ok(e[3], tag));
            if (__all(ok)) break;
            if (!poll_backoff_ws(ws, m.abort_flag)) break;
          }
          if (w < cnt && better(__uint_as_float(e[0]), (int)e[2], gv, gi)) {
            gv = __uint_as_float(e[0]);
            gi = (int)e[2];
          }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
          const float ov = __shfl_xor(gv, off, 64);
          const int oi = __shfl_xor(gi, off, 64);
          if (better(ov, oi, gv, gi)) {
            gv = ov;
            gi = oi;
          }
        }
        if (lane == 0) {
          tok_lds[0] = gi;
          if (wg == 0) {
            m.tokens[0] = gi;
            if (step0 + s < max_steps) m.history[step0 + s] = gi;
          }
        }
      }
      cbar();
      token = tok_lds[0];
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---- stream packing --------------------------------------------------------------------------------------
__device__ __forceinline__ int pk_nbw(const PersistModel &m, int kind, int w) {
  return w < m.ph[kind].nb ? (m.ph[kind].nb - w + m.G - 1) / m.G : 0;
}
__device__ __host__ inline size_t pk_seq_offset(const PersistModel &m, int w, int layer, int kind) {
  size_t per_layer = 0, before = 0;
  for (int k = 0; k < 4; k++) {
    const int nb = w < m.ph[k].nb ? (m.ph[k].nb - w + m.G - 1) / m.G : 0;
    const size_t b = (size_t)nb * m.ph[k].blk_bytes;
    per_layer += b;
    if (k < kind) before += b;
  }
  if (kind == PK_LM) return (size_t)m.n_layers * per_layer;
  return (size_t)layer * per_layer + before;
}

__global__ void __launch_bounds__(256) persist_pack_kernel(PersistModel m, int layer, int kind,
                                                           const uint8_t *__restrict__ packed,
                                                           const _Float16 *__restrict__ scales, uint8_t *stream) {
  const int gb = blockIdx.x;   // global 8-row block
  const int v = blockIdx.y;    // wave (k slice)
  const PersistPhase ph = m.ph[kind];
  const int w = gb % m.G, bi = gb / m.G;
  uint8_t *dest = stream + m.wg_off[w] + (size_t)v * m.wave_bytes[w] + pk_seq_offset(m, w, layer, kind) +
                  (size_t)bi * ph.blk_bytes;
  const int tid = threadIdx.x;
  const size_t row_bytes = (size_t)ph.k / 2, row_groups = (size_t)ph.k / 32;
  const int rot_rows = kind == PK_QKV ? (m.n_heads + m.n_kv_heads) * 128 : 0;
  auto logical_row = [&](int pr) {
    if (pr < rot_rows) {
      const int head = pr >> 7, p2 = pr & 127;
      return head * 128 + (p2 >> 1) + 64 * (p2 & 1);
    }
    return pr;
  };
  for (int p = 0; p < ph.pairs; p++) {
    const bool single = (ph.tiles & 1) && p == ph.pairs - 1;
    uint8_t *rec = dest + (size_t)p * PS_REC_FULL;
    if (tid < 128) {
      const int t = tid >> 6, ln = tid & 63;
      if (!(t == 1 && single)) {
        const int r = ln & 15, c = ln >> 4;
        const int row = logical_row(8 * gb + (r & 7));
        const int kbase = v * ph.ks + 256 * (2 * p + t);
        uint4_t out;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const int kb = (r < 8) ? j : 4 + j;
          const int k = kbase + 32 * kb + 8 * c;
          const uint32_t raw = *reinterpret_cast<const uint32_t *>(packed + (size_t)row * row_bytes + k / 2);
          // raw: element i in bits [4i, 4i+4)  ->  e0 e2 e4 e6 | e1 e3 e5 e7 (int4_common.hpp)
          uint32_t wv = 0;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const uint32_t q = (raw >> (4 * e)) & 0xFu;
            const int slot = (e & 1) ? 4 + (e >> 1) : (e >> 1);
            wv |= q << (4 * slot);
          }
          out[j] = wv;
        }
        *reinterpret_cast<uint4_t *>(rec + t * 1024 + ln * 16) = out;
      }
    } else if (tid < 192) {
      const int sl = tid - 128;  // two fp16 scales at byte sl * 4 of the 256-byte scale block
      const int t = sl >> 5, r = (sl & 31) >> 1, j0 = (sl & 1) * 2;
      uint32_t word = 0;
      if (!(t == 1 && single)) {
        const int row = logical_row(8 * gb + (r & 7));
        const int kbase = v * ph.ks + 256 * (2 * p + t);
        U32H2 u;
#pragma unroll
        for (int jj = 0; jj < 2; jj++) {
          const int kb = (r < 8) ? (j0 + jj) : 4 + j0 + jj;
          u.h[jj] = scales[(size_t)row * row_groups + (kbase + 32 * kb) / 32];
        }
        word = u.u;
      }
      *reinterpret_cast<uint32_t *>(rec + (single ? 1024 : 2048) + sl * 4) = word;
    }
  }
}

// ---- host side ---------------------------------------------------------------------------------------------
bool persist_supported(const yscv_hip_decoder_config &c, int num_cus, const char **why) {
  const char *dummy;
  if (!why) why = &dummy;
  const int G = num_cus;
  const int hq = c.n_heads * c.head_dim;
  auto bad_k = [](int k) { return k % (256 * PS_WAVES) != 0 || k > PS_WAVES * 512 * MAXF || k <= 0; };
  if (c.head_dim != 128) { *why = "head_dim must be 128"; return false; }
  if (c.group_size != 32) { *why = "group size must be 32"; return false; }
  if (bad_k(c.d_model) || bad_k(hq) || bad_k(c.d_ff)) { *why = "d_model, n_heads*128 and d_ff must be multiples of 1024, at most 16384"; return false; }
  if (c.vocab % 8 != 0) { *why = "vocab must be a multiple of 8"; return false; }
  if (c.n_heads % c.n_kv_heads != 0 || c.n_heads / c.n_kv_heads > 4) { *why = "1..4 query heads per kv head"; return false; }
  if (G < 16 || G > 1024) { *why = "unsupported CU count"; return false; }
  auto rows_per_wg = [&](int n) { return ((n / 8 + G - 1) / G) * 8; };
  if (rows_per_wg(c.d_model) > 64) { *why = "d_model too large for the CU count"; return false; }
  const int qkv_n = (c.n_heads + 2 * c.n_kv_heads) * 128;
  if (rows_per_wg(qkv_n) > PART_ROWS || rows_per_wg(2 * c.d_ff) > PART_ROWS || rows_per_wg(c.vocab) > PART_ROWS) {
    *why = "a projection has more rows per workgroup than the reduction buffer holds";
    return false;
  }
  if (c.max_ctx % 128 != 0) { *why = "max_ctx must be a multiple of 128"; return false; }
  return true;
}

void persist_fill_phases(const yscv_hip_decoder_config &c, int G, PersistModel *m) {
  m->n_layers = c.n_layers;
  m->d_model = c.d_model;
  m->n_heads = c.n_heads;
  m->n_kv_heads = c.n_kv_heads;
  m->d_ff = c.d_ff;
  m->vocab = c.vocab;
  m->max_ctx = c.max_ctx;
  m->theta = c.rope_theta;
  m->eps = c.rms_eps;
  m->G = G;
  const int hq = c.n_heads * 128;
  const int n[PK_COUNT] = {(c.n_heads + 2 * c.n_kv_heads) * 128, c.d_model, 2 * c.d_ff, c.d_model, c.vocab};
  const int k[PK_COUNT] = {c.d_model, hq, c.d_model, c.d_ff, c.d_model};
  for (int i = 0; i < PK_COUNT; i++) {
    PersistPhase &p = m->ph[i];
    p.n = n[i];
    p.k = k[i];
    p.ks = k[i] / PS_WAVES;
    p.tiles = p.ks / 256;
    p.pairs = (p.tiles + 1) / 2;
    p.frags = p.pairs;
    p.nb = n[i] / 8;
    p.blk_bytes = (p.tiles / 2) * PS_REC_FULL + (p.tiles & 1) * PS_REC_SINGLE;
  }
}

size_t persist_wave_bytes(const PersistModel &m, int w) { return pk_seq_offset(m, w, 0, PK_LM) + (size_t)(w < m.ph[PK_LM].nb ? (m.ph[PK_LM].nb - w + m.G - 1) / m.G : 0) * m.ph[PK_LM].blk_bytes; }
size_t persist_seq_offset(const PersistModel &m, int w, int layer, int kind) { return pk_seq_offset(m, w, layer, kind); }

int32_t launch_persist_pack(const PersistModel &m, int layer, int kind, const uint8_t *packed_dev,
                            const _Float16 *scales_dev, uint8_t *stream, hipStream_t s) {
  if (kind < 0 || kind >= PK_COUNT) return set_error(YSCV_HIP_ERR_INVALID_ARG, "bad projection kind %d", kind);
  hipLaunchKernelGGL(persist_pack_kernel, dim3(m.ph[kind].nb, CW), dim3(256), 0, s, m, layer, kind, packed_dev,
                     scales_dev, stream);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_persist_decode(const PersistModel &m, int n_steps, int pos0, int step0, int max_steps,
                              uint32_t epoch0, hipStream_t s) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void *>(decode_persistent_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, PERSIST_LDS);
  });
  if (attr_err != hipSuccess)
    return set_error(YSCV_HIP_ERR_DEVICE, "cannot reserve %d bytes of LDS: %s", PERSIST_LDS, hipGetErrorString(attr_err));
  int max_blocks = 0;
  YSCV_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&max_blocks, decode_persistent_kernel, THREADS, PERSIST_LDS));
  if (max_blocks < 1) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "the persistent decode kernel does not fit a CU");
  PersistModel mm = m;
  void *args[] = {&mm, &n_steps, &pos0, &step0, &max_steps, &epoch0};
  YSCV_HIP_TRY(hipLaunchCooperativeKernel(reinterpret_cast<const void *>(decode_persistent_kernel), dim3(m.G), dim3(THREADS),
                                          args, PERSIST_LDS, s));
  return YSCV_HIP_OK;
}

}  // namespace yscv
