// The operators between the MatMuls of an exported LLM graph, as stand-alone entry points on device tensors, so
// that a graph executor stays on the GPU from one projection to the next:
//   rms_norm   crates/yscv-kernels/src/ops/norm.rs:1431-1518   y = x * (1 / sqrt(mean(x^2) + eps)) * gamma, last axis
//   rope       crates/yscv-kernels/src/ops/rope.rs:24-117      rotate-half pairs (i, i + d/2), in place on q and k
//   GroupQueryAttention  crates/yscv-onnx/src/runner/linear.rs:552-646   q [B][Sq][Hq d], k / v [B][Sk][Hkv d],
//              kv_h = q_h / groups, scores * 1/sqrt(d), max-subtracted softmax, no mask
// and the general attention kernel behind the last one, which the decoder also uses where its specialised kernels
// do not apply: any head width that is a multiple of 32 up to 128, any number of query heads per kv head, several
// query positions per call with a causal limit (prompt ingestion), K / V either as the operator's tensors or as the
// decoder's fp16 cache.
//
// Three forms of the attention kernel share the arithmetic below: gqa_generic_kernel (a workgroup owns 16 queries of
// one head, the key blocks are split over its waves: decode and short query counts), gqa_rows_kernel (a wave owns 32
// queries and walks every key block: the operator from 64 queries on) and gqa_shared_kv_kernel (the prompt pass over
// the decoder's cache: the waves of a workgroup share each stage of K / V through LDS).
// gqa_generic_kernel: a workgroup of four waves owns 16 query positions of one head.  Wave w walks the key blocks
// w, w + 4, ... of 16 positions each:
//   S^T = K Q^T   rows = positions, columns = queries: hd / 32 x v_mfma_f32_16x16x32_f16, A = 16 cache rows as they lie
//                 in memory, B = the 16 query rows as they lie in memory; lane (r, c) then holds positions 4c .. 4c+3
//                 of query r, which is exactly the B operand of the second product
//   online softmax per query (= per lane column r; the four lane groups c are reduced with two permlane swaps)
//   O^T += V^T P^T  hd / 16 x v_mfma_f32_16x16x16_f16, A = V^T (the cache keeps eight consecutive positions of one
//                 channel together, so a lane's four positions are one 8-byte load)
// and the four waves merge their (max, sum, O) through LDS.  Scores and sums are f32; q, k, v and the softmax weights
// enter the MFMAs as fp16, like the decoder's own kernels (tolerance-checked against the f32 restatement).
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>

#include "int4_common.hpp"
#include "decoder.hpp"
#include "kernels.hpp"

namespace yscv {

namespace {

struct GqaArgs {
  const void *q, *k, *v;
  void *out;
  // element strides: q[b * q_b + s * q_s + h * hd + d], same for k (h = kv head) and out; v natural like k, or
  // v slab: v[b * v_b + kvh * v_h + ((pos / 8) * hd + d) * 8 + pos % 8]
  long long q_b, q_s, k_b, k_s, k_h, v_b, v_s, v_h, o_b, o_s;
  int B, Sq, Sk, Hq, Hkv;
  int causal_base;            // < 0: every query sees all Sk positions; else query s sees positions <= causal_base + s
  const int32_t *sk_minus_1;  // null, or device word holding Sk - 1 (the decoder's position counter)
  float scale;
  // Decode with the rotary embedding and the cache append inside the kernel (FUSE): q is [B][(Hq + 2 Hkv) HD] with
  // q, k and v of the new position unrotated; the workgroups rotate what they need themselves, the first query head
  // of a kv group also writes the new k / v row to the cache (k, v are then written through), the rotated q goes to qrot
  float theta;
  _Float16 *qrot;
};

template <typename T>
__device__ __forceinline__ half8_t load8(const T *p);
template <>
__device__ __forceinline__ half8_t load8<_Float16>(const _Float16 *p) {
  return *reinterpret_cast<const half8_t *>(p);
}
template <>
__device__ __forceinline__ half8_t load8<float>(const float *p) {
  const float4_t a = *reinterpret_cast<const float4_t *>(p), b = *reinterpret_cast<const float4_t *>(p + 4);
  return half8_t{(_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3],
                 (_Float16)b[0], (_Float16)b[1], (_Float16)b[2], (_Float16)b[3]};
}
template <typename T>
__device__ __forceinline__ void store4(T *p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<_Float16>(_Float16 *p, float a, float b, float c, float d) {
  *reinterpret_cast<half4_t *>(p) = half4_t{(_Float16)a, (_Float16)b, (_Float16)c, (_Float16)d};
}
template <>
__device__ __forceinline__ void store4<float>(float *p, float a, float b, float c, float d) {
  *reinterpret_cast<float4_t *>(p) = float4_t{a, b, c, d};
}

constexpr int GQA_WAVES = 4;

template <int HD, typename TQ, typename TKV, typename TO, bool V_SLAB, bool FUSE = false>
__global__ void __launch_bounds__(64 * GQA_WAVES) gqa_generic_kernel(GqaArgs p) {
  static_assert(HD % 32 == 0 && HD >= 32 && HD <= 128, "head width (the merge buffer must fit the static LDS limit)");
  static_assert(!FUSE || (V_SLAB && std::is_same<TQ, _Float16>::value && std::is_same<TKV, _Float16>::value),
                "the fused form works on the decoder's fp16 buffers");
  constexpr int KK = HD / 32, DT = HD / 16;
  __shared__ float m_s[GQA_WAVES][16], l_s[GQA_WAVES][16];
  __shared__ float o_s[GQA_WAVES][16][HD + 4];
  __shared__ __attribute__((aligned(16))) _Float16 q_rot[FUSE ? HD : 8], k_new[FUSE ? HD : 8], v_new[FUSE ? HD : 8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int q0 = blockIdx.x * 16, h = blockIdx.y, b = blockIdx.z;
  const int kvh = h / (p.Hq / p.Hkv);
  const int Sk = p.sk_minus_1 ? *p.sk_minus_1 + 1 : p.Sk;
  // query r of this tile (rows past the end repeat the last one and are not stored)
  const int qi = min(q0 + r, p.Sq - 1);
  const int lim_q = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + qi);           // last position query r sees
  const int lim_tile = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + min(q0 + 15, p.Sq - 1));
  const int nblocks = lim_tile / 16 + 1;

  const TQ *qrow = static_cast<const TQ *>(p.q) + (size_t)b * p.q_b + (size_t)qi * p.q_s + (size_t)h * HD;
  const TKV *kbase = static_cast<const TKV *>(p.k) + (size_t)b * p.k_b + (size_t)kvh * p.k_h;
  const TKV *vbase = static_cast<const TKV *>(p.v) + (size_t)b * p.v_b + (size_t)kvh * p.v_h;
  half8_t qf[KK];
  if constexpr (FUSE) {
    // One query position per sequence (Sq = 1, the position is Sk - 1).  Wave 0 rotates this head's q, wave 1 the new
    // k row of its kv head, waves 2 and 3 fetch the new v row: the arithmetic of the separate rope + append launch.
    // Every workgroup of a kv group works out the same k / v row (it cannot wait for another workgroup's append) and
    // patches it into the key block that holds the position; one of them stores it.
    const int pos = Sk - 1, half_d = HD / 2, wave_u = __builtin_amdgcn_readfirstlane(wave);
    const bool writer = h % (p.Hq / p.Hkv) == 0;
    const _Float16 *row = reinterpret_cast<const _Float16 *>(p.q) + (size_t)b * p.q_b;
    if (wave_u < 2) {
      const int i = lane;
      if (i < half_d) {
        const float inv_freq = 1.0f / powf(p.theta, (float)(2 * i) / (float)HD);
        float sn, cs;
        sincosf(inv_freq * (float)pos, &sn, &cs);
        const _Float16 *src = row + (size_t)(wave_u == 0 ? h : p.Hq + kvh) * HD;
        const float x0 = (float)src[i], x1 = (float)src[i + half_d];
        float f0 = fmaf(x0, cs, -(x1 * sn)), f1 = fmaf(x0, sn, x1 * cs);
        asm volatile("" : "+v"(f0), "+v"(f1));  // the f32 value exists before it is narrowed (no mixed-precision fma)
        const _Float16 y0 = (_Float16)f0, y1 = (_Float16)f1;
        if (wave_u == 0) {
          q_rot[i] = y0;
          q_rot[i + half_d] = y1;
          _Float16 *qd = p.qrot + ((size_t)b * p.Hq + h) * HD;
          qd[i] = y0;
          qd[i + half_d] = y1;
        } else {
          k_new[i] = y0;
          k_new[i + half_d] = y1;
          if (writer) {
            _Float16 *kd = const_cast<_Float16 *>(reinterpret_cast<const _Float16 *>(kbase)) + (size_t)pos * p.k_s;
            kd[i] = y0;
            kd[i + half_d] = y1;
          }
        }
      }
    } else {
      const int dd = tid - 128;
      if (dd < HD) {
        const _Float16 v = row[(size_t)(p.Hq + p.Hkv + kvh) * HD + dd];
        v_new[dd] = v;
        if (writer)
          const_cast<_Float16 *>(reinterpret_cast<const _Float16 *>(vbase))[((size_t)(pos >> 3) * HD + dd) * 8 + (pos & 7)] = v;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KK; kk++) qf[kk] = *reinterpret_cast<const half8_t *>(&q_rot[32 * kk + 8 * c]);
  } else {
#pragma unroll
    for (int kk = 0; kk < KK; kk++) qf[kk] = load8<TQ>(qrow + 32 * kk + 8 * c);
  }

  float m_run = -INFINITY, l_run = 0.0f;
  float4_t o_acc[DT];
#pragma unroll
  for (int t = 0; t < DT; t++) o_acc[t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

  // operands of one key block: 16 cache rows as the A operand of S^T (lane (r, c): row p0 + r, channels 32 kk + 8c .. + 7;
  // rows past the end repeat the last one) and V^T as the A operand of the second product (lane (r, c): channel
  // 16 t + r at positions p0 + 4c .. + 3).  The next block's are requested before this block's arithmetic.
  auto load_block = [&](int blk, half8_t (&kf)[KK], half4_t (&vf)[DT]) {
    const int p0 = blk * 16;
    const TKV *krow = kbase + (size_t)min(p0 + r, Sk - 1) * p.k_s;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) kf[kk] = load8<TKV>(krow + 32 * kk + 8 * c);
#pragma unroll
    for (int t = 0; t < DT; t++) {
      if constexpr (V_SLAB) {
        const _Float16 *vp = reinterpret_cast<const _Float16 *>(vbase) + ((size_t)((p0 + 4 * c) >> 3) * HD + 16 * t + r) * 8 + ((4 * c) & 7);
        vf[t] = *reinterpret_cast<const half4_t *>(vp);
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int pos = min(p0 + 4 * c + e, Sk - 1);
          vf[t][e] = (_Float16)vbase[(size_t)pos * p.v_s + 16 * t + r];
        }
      }
    }
  };
  half8_t kf[KK], kn[KK];
  half4_t vf[DT], vn[DT];
  if (wave < nblocks) load_block(wave, kf, vf);
  for (int blk = wave; blk < nblocks; blk += GQA_WAVES) {
    const int p0 = blk * 16;
    const bool more = blk + GQA_WAVES < nblocks;  // uniform in the wave
    if (more) load_block(blk + GQA_WAVES, kn, vn);
    if constexpr (FUSE) {
      // the row appended in this launch: the loads saw whatever the cache held before
      const int rel = Sk - 1 - p0;
      if (rel >= 0 && rel < 16) {  // uniform in the wave
        if (r == rel) {
#pragma unroll
          for (int kk = 0; kk < KK; kk++) kf[kk] = *reinterpret_cast<const half8_t *>(&k_new[32 * kk + 8 * c]);
        }
        const int e_new = rel - 4 * c;
        if (e_new >= 0 && e_new < 4) {
#pragma unroll
          for (int t = 0; t < DT; t++) {
            const _Float16 nv = v_new[16 * t + r];
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (e == e_new) vf[t][e] = nv;
          }
        }
      }
    }
    float4_t s = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int kk = 0; kk < KK; kk++) s = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[kk], qf[kk], s, 0, 0, 0);
    // lane (r, c): query r, positions p0 + 4c + e
    float sv[4], mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      sv[e] = (p0 + 4 * c + e <= lim_q) ? s[e] * p.scale : -INFINITY;
      mx = fmaxf(mx, sv[e]);
    }
    mx = max_xor16_xor32(mx);
    const float m_new = fmaxf(m_run, mx);
    float pe[4], sum = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      pe[e] = (sv[e] == -INFINITY) ? 0.0f : __expf(sv[e] - m_new);
      sum += pe[e];
    }
    sum = sum_xor16_xor32(sum);
    const float alpha = (m_run == -INFINITY) ? 0.0f : __expf(m_run - m_new);
    l_run = l_run * alpha + sum;
    m_run = m_new;
    const half4_t pf = {(_Float16)pe[0], (_Float16)pe[1], (_Float16)pe[2], (_Float16)pe[3]};
#pragma unroll
    for (int t = 0; t < DT; t++) {
      // positions past the end of the context meet weight 0 -- but 0 * NaN would poison the sum (the slab may hold
      // anything there), so they are blanked
      half4_t vv = vf[t];
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (p0 + 4 * c + e >= Sk) vv[e] = (_Float16)0.0f;
      o_acc[t] = o_acc[t] * alpha;
      o_acc[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(vv, pf, o_acc[t], 0, 0, 0);
    }
    if (more) {
#pragma unroll
      for (int kk = 0; kk < KK; kk++) kf[kk] = kn[kk];
#pragma unroll
      for (int t = 0; t < DT; t++) vf[t] = vn[t];
    }
  }
  // ---- merge the four waves: lane (r, c) holds O^T[16 t + 4c + e][query r]
  if (c == 0) {
    m_s[wave][r] = m_run;
    l_s[wave][r] = l_run;
  }
#pragma unroll
  for (int t = 0; t < DT; t++)
#pragma unroll
    for (int e = 0; e < 4; e++) o_s[wave][r][16 * t + 4 * c + e] = o_acc[t][e];
  __syncthreads();
  TO *obase = static_cast<TO *>(p.out) + (size_t)b * p.o_b + (size_t)h * HD;
  for (int idx = tid; idx < 16 * (HD / 4); idx += 64 * GQA_WAVES) {
    const int qq = idx / (HD / 4), d4 = (idx % (HD / 4)) * 4;
    if (q0 + qq >= p.Sq) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < GQA_WAVES; w++) M = fmaxf(M, m_s[w][qq]);
    float L = 0.0f, o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int w = 0; w < GQA_WAVES; w++) {
      const float f = (m_s[w][qq] == -INFINITY) ? 0.0f : __expf(m_s[w][qq] - M);
      L += l_s[w][qq] * f;
#pragma unroll
      for (int e = 0; e < 4; e++) o[e] += o_s[w][qq][d4 + e] * f;
    }
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
    store4<TO>(obase + (size_t)(q0 + qq) * p.o_s + d4, o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv);
  }
}

// Many query positions (prompt pass, or the operator with a long seq_q): a wave owns 32 consecutive queries of one
// head and walks every key block itself -- each K / V load then feeds two query tiles, and nothing is merged at the
// end.  A workgroup's four waves take neighbouring query ranges of the same head, so their K / V requests meet in
// the CU's cache.  Same arithmetic per (query, position) as gqa_generic_kernel.
template <int HD, typename TQ, typename TKV, typename TO, bool V_SLAB>
__global__ void __launch_bounds__(64 * GQA_WAVES) gqa_rows_kernel(GqaArgs p) {
  static_assert(HD % 32 == 0 && HD >= 32 && HD <= 128, "head width");
  constexpr int KK = HD / 32, DT = HD / 16, QT = 2;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  // late query ranges see the most keys: they are dispatched first, so that the grid does not end on its longest workgroups
  const int q0 = (((int)gridDim.x - 1 - (int)blockIdx.x) * GQA_WAVES + wave) * 16 * QT, h = blockIdx.y, b = blockIdx.z;
  if (q0 >= p.Sq) return;  // no barrier in this kernel
  const int kvh = h / (p.Hq / p.Hkv);
  const int Sk = p.Sk;
  int qi[QT], lim_q[QT];
  half8_t qf[QT][KK];
#pragma unroll
  for (int u = 0; u < QT; u++) {
    qi[u] = min(q0 + 16 * u + r, p.Sq - 1);
    lim_q[u] = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + qi[u]);
    const TQ *qrow = static_cast<const TQ *>(p.q) + (size_t)b * p.q_b + (size_t)qi[u] * p.q_s + (size_t)h * HD;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) qf[u][kk] = load8<TQ>(qrow + 32 * kk + 8 * c);
  }
  const int lim_wave = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + min(q0 + 16 * QT - 1, p.Sq - 1));
  const int nblocks = lim_wave / 16 + 1;
  const TKV *kbase = static_cast<const TKV *>(p.k) + (size_t)b * p.k_b + (size_t)kvh * p.k_h;
  const TKV *vbase = static_cast<const TKV *>(p.v) + (size_t)b * p.v_b + (size_t)kvh * p.v_h;
  float m_run[QT], l_run[QT];
  float4_t o_acc[QT][DT];
#pragma unroll
  for (int u = 0; u < QT; u++) {
    m_run[u] = -INFINITY;
    l_run[u] = 0.0f;
#pragma unroll
    for (int t = 0; t < DT; t++) o_acc[u][t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }
  auto load_block = [&](int blk, half8_t (&kf)[KK], half4_t (&vf)[DT]) {
    const int p0 = blk * 16;
    const TKV *krow = kbase + (size_t)min(p0 + r, Sk - 1) * p.k_s;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) kf[kk] = load8<TKV>(krow + 32 * kk + 8 * c);
#pragma unroll
    for (int t = 0; t < DT; t++) {
      if constexpr (V_SLAB) {
        const _Float16 *vp = reinterpret_cast<const _Float16 *>(vbase) + ((size_t)((p0 + 4 * c) >> 3) * HD + 16 * t + r) * 8 + ((4 * c) & 7);
        vf[t] = *reinterpret_cast<const half4_t *>(vp);
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int pos = min(p0 + 4 * c + e, Sk - 1);
          vf[t][e] = (_Float16)vbase[(size_t)pos * p.v_s + 16 * t + r];
        }
      }
    }
  };
  half8_t kf[KK], kn[KK];
  half4_t vf[DT], vn[DT];
  load_block(0, kf, vf);
  for (int blk = 0; blk < nblocks; blk++) {
    const int p0 = blk * 16;
    const bool more = blk + 1 < nblocks;
    if (more) load_block(blk + 1, kn, vn);
    half4_t vv[DT];
#pragma unroll
    for (int t = 0; t < DT; t++) {
      vv[t] = vf[t];
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (p0 + 4 * c + e >= Sk) vv[t][e] = (_Float16)0.0f;  // 0 * NaN would poison the sum
    }
#pragma unroll
    for (int u = 0; u < QT; u++) {
      float4_t s = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kk = 0; kk < KK; kk++) s = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[kk], qf[u][kk], s, 0, 0, 0);
      float sv[4], mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        sv[e] = (p0 + 4 * c + e <= lim_q[u]) ? s[e] * p.scale : -INFINITY;
        mx = fmaxf(mx, sv[e]);
      }
      mx = max_xor16_xor32(mx);
      const float m_new = fmaxf(m_run[u], mx);
      float pe[4], sum = 0.0f;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        pe[e] = (sv[e] == -INFINITY) ? 0.0f : __expf(sv[e] - m_new);
        sum += pe[e];
      }
      sum = sum_xor16_xor32(sum);
      const float alpha = (m_run[u] == -INFINITY) ? 0.0f : __expf(m_run[u] - m_new);
      l_run[u] = l_run[u] * alpha + sum;
      m_run[u] = m_new;
      const half4_t pf = {(_Float16)pe[0], (_Float16)pe[1], (_Float16)pe[2], (_Float16)pe[3]};
#pragma unroll
      for (int t = 0; t < DT; t++) {
        o_acc[u][t] = o_acc[u][t] * alpha;
        o_acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x16f16(vv[t], pf, o_acc[u][t], 0, 0, 0);
      }
    }
    if (more) {
#pragma unroll
      for (int kk = 0; kk < KK; kk++) kf[kk] = kn[kk];
#pragma unroll
      for (int t = 0; t < DT; t++) vf[t] = vn[t];
    }
  }
  // lane (r, c) holds O^T[16 t + 4c + e][query r] of each query tile: four consecutive channels per store
  TO *obase = static_cast<TO *>(p.out) + (size_t)b * p.o_b + (size_t)h * HD;
#pragma unroll
  for (int u = 0; u < QT; u++) {
    if (q0 + 16 * u + r >= p.Sq) continue;
    const float inv = l_run[u] > 0.0f ? 1.0f / l_run[u] : 0.0f;
    TO *orow = obase + (size_t)(q0 + 16 * u + r) * p.o_s;
#pragma unroll
    for (int t = 0; t < DT; t++)
      store4<TO>(orow + 16 * t + 4 * c, o_acc[u][t][0] * inv, o_acc[u][t][1] * inv, o_acc[u][t][2] * inv, o_acc[u][t][3] * inv);
  }
}

// Prompt pass over the decoder's fp16 cache: the four waves of a workgroup take the same key range -- query heads
// that share a kv head (as many of them as divide four), else neighbouring 32-query ranges of one head -- so a
// stage of 32 cache positions is fetched once per workgroup into LDS (K rows with their 16-byte pieces XOR-swizzled
// so that the 16 rows a fragment read touches fall into 16 different bank groups; V as its slabs lie in memory) and
// read from there by all four: a quarter of the L2 traffic of gqa_rows_kernel, which is what bounds that kernel at
// prompt lengths in the thousands.  Two stage buffers: the next stage's pieces are requested into registers before
// this stage's arithmetic and written to the other buffer behind it, one barrier per stage.  Arithmetic per
// (query, position) as in gqa_generic_kernel; the running output is rescaled only where some query's maximum moved
// (a factor of exactly one otherwise).
template <int HD>
__global__ void __launch_bounds__(64 * GQA_WAVES, 2) gqa_shared_kv_kernel(GqaArgs p, int hw_log2) {
  static_assert(HD % 32 == 0 && HD >= 32 && HD <= 128, "head width");
  constexpr int KK = HD / 32, DT = HD / 16, QT = 2, KB = 32;  // KB: cache positions per stage
  constexpr int CPR = HD / 8;                                  // 16-byte pieces of a K row
  constexpr int PITCH = HD > 64 ? 16 : (HD > 32 ? 8 : 4);      // row pitch in pieces (a power of two)
  constexpr int RPW = 16 / PITCH;                              // rows per 256 bytes
  constexpr int K_BYTES = KB * PITCH * 16, V_BYTES = (KB / 8) * HD * 16, ST_BYTES = K_BYTES + V_BYTES;
  constexpr int K_PIECES = KB * CPR, V_PIECES = (KB / 8) * HD;
  constexpr int THREADS = 64 * GQA_WAVES;
  constexpr int K_LD = (K_PIECES + THREADS - 1) / THREADS, V_LD = (V_PIECES + THREADS - 1) / THREADS;
  __shared__ __attribute__((aligned(16))) uint8_t stage[2 * ST_BYTES];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int hw = 1 << hw_log2, qw = GQA_WAVES >> hw_log2;  // heads x query ranges of a workgroup
  const int group = p.Hq / p.Hkv, chunks = group >> hw_log2;
  const int kvh = (int)blockIdx.x / chunks, b = blockIdx.z;
  const int h = kvh * group + ((int)blockIdx.x % chunks) * hw + (wave & (hw - 1));
  // Workgroups start in the order of blockIdx.y.  The first half takes the late query ranges (most positions), the
  // second half the early ones in rising order: two workgroups that start half a grid apart, and so tend to share
  // a CU, carry about the same work together as any other such pair.
  const int T = gridDim.y, first_half = (T + 1) / 2;
  const int tile = (int)blockIdx.y < first_half ? T - 1 - (int)blockIdx.y : (int)blockIdx.y - first_half;
  const int q0 = (tile * qw + (wave >> hw_log2)) * 16 * QT;
  const bool active = q0 < p.Sq;
  const int Sk = p.Sk;
  int qi[QT], lim_q[QT];
  half8_t qf[QT][KK];
#pragma unroll
  for (int u = 0; u < QT; u++) {
    qi[u] = min(q0 + 16 * u + r, p.Sq - 1);
    lim_q[u] = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + qi[u]);
    const _Float16 *qrow = static_cast<const _Float16 *>(p.q) + (size_t)b * p.q_b + (size_t)qi[u] * p.q_s + (size_t)h * HD;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) qf[u][kk] = load8<_Float16>(qrow + 32 * kk + 8 * c);
  }
  const int lim_wave = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + min(q0 + 16 * QT - 1, p.Sq - 1));
  const int lim_first = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + min(q0, p.Sq - 1));  // what the wave's first query sees
  const int q_last = min((tile + 1) * qw * 16 * QT, p.Sq) - 1;  // last query of the workgroup
  const int lim_wg = p.causal_base < 0 ? Sk - 1 : min(Sk - 1, p.causal_base + q_last);
  const int nstages = lim_wg / KB + 1;
  const _Float16 *kbase = static_cast<const _Float16 *>(p.k) + (size_t)b * p.k_b + (size_t)kvh * p.k_h;
  const _Float16 *vbase = static_cast<const _Float16 *>(p.v) + (size_t)b * p.v_b + (size_t)kvh * p.v_h;
  float m_run[QT], l_run[QT];
  float4_t o_acc[QT][DT];
#pragma unroll
  for (int u = 0; u < QT; u++) {
    m_run[u] = -INFINITY;
    l_run[u] = 0.0f;
#pragma unroll
    for (int t = 0; t < DT; t++) o_acc[u][t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }
  // piece idx of a stage's K: row idx / CPR, piece idx % CPR; of its V: slab idx / HD, channel idx % HD.  Rows and
  // slabs past the end of the context repeat the last one (never used: their positions are masked)
  auto fetch = [&](int st, uint4_t (&kr)[K_LD], uint4_t (&vr)[V_LD]) {
#pragma unroll
    for (int j = 0; j < K_LD; j++) {
      const int idx = tid + THREADS * j;
      if (K_PIECES % THREADS == 0 || idx < K_PIECES) {
        const int pos = min(st * KB + idx / CPR, Sk - 1);
        kr[j] = *reinterpret_cast<const uint4_t *>(kbase + (size_t)pos * p.k_s + (idx % CPR) * 8);
      }
    }
#pragma unroll
    for (int j = 0; j < V_LD; j++) {
      const int idx = tid + THREADS * j;
      if (V_PIECES % THREADS == 0 || idx < V_PIECES) {
        const int slab = min(st * (KB / 8) + idx / HD, (Sk - 1) >> 3);
        vr[j] = *reinterpret_cast<const uint4_t *>(vbase + ((size_t)slab * HD + idx % HD) * 8);
      }
    }
  };
  auto stash = [&](int buf, const uint4_t (&kr)[K_LD], const uint4_t (&vr)[V_LD]) {
    uint8_t *base = stage + buf * ST_BYTES;
#pragma unroll
    for (int j = 0; j < K_LD; j++) {
      const int idx = tid + THREADS * j;
      if (K_PIECES % THREADS == 0 || idx < K_PIECES) {
        const int row = idx / CPR, piece = idx % CPR;
        *reinterpret_cast<uint4_t *>(base + (row * PITCH + (piece ^ ((((row >> 3) & 3) * 4 + (row & 3)) / RPW))) * 16) = kr[j];
      }
    }
#pragma unroll
    for (int j = 0; j < V_LD; j++) {
      const int idx = tid + THREADS * j;
      if (V_PIECES % THREADS == 0 || idx < V_PIECES) *reinterpret_cast<uint4_t *>(base + K_BYTES + idx * 16) = vr[j];
    }
  };
  auto compute = [&](int st) {
    const uint8_t *base = stage + (st & 1) * ST_BYTES;
    const int p0 = st * KB;
    if (active && p0 <= lim_wave) {  // uniform in the wave
      // Two S^T tiles per stage.  Row rho of tile j is stage position 8 (rho / 4) + 4 j + rho % 4, so lane (r, c)
      // ends up with the weights of positions 8c .. 8c+7 (tile 0: the first four, tile 1: the last four): one 16-byte
      // slab piece of V^T per channel, and the B operand of one 32-deep MFMA.
      half8_t kf[2][KK], vv[DT];
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int row = 8 * (r >> 2) + 4 * j + (r & 3);
#pragma unroll
        for (int kk = 0; kk < KK; kk++)
          kf[j][kk] = *reinterpret_cast<const half8_t *>(base + (row * PITCH + ((4 * kk + c) ^ (r / RPW))) * 16);
      }
#pragma unroll
      for (int t = 0; t < DT; t++) vv[t] = *reinterpret_cast<const half8_t *>(base + K_BYTES + (c * HD + 16 * t + r) * 16);
      if (p0 + KB > Sk) {  // 0 * NaN would poison the sum: positions past the context are blanked
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (p0 + 8 * c + e >= Sk) vv[t][e] = (_Float16)0.0f;
      }
#pragma unroll
      for (int u = 0; u < QT; u++) {
        float4_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[0][kk], qf[u][kk], s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[1][kk], qf[u][kk], s1, 0, 0, 0);
        }
        float sv[8], mx = -INFINITY, pe[8], sum = 0.0f, m_new;
        if (p0 + KB - 1 <= lim_first) {  // uniform in the wave: every query of the wave sees the whole stage
#pragma unroll
          for (int e = 0; e < 8; e++) {
            sv[e] = (e < 4 ? s0[e & 3] : s1[e & 3]) * p.scale;
            mx = fmaxf(mx, sv[e]);
          }
          m_new = fmaxf(m_run[u], max_xor16_xor32(mx));
#pragma unroll
          for (int e = 0; e < 8; e++) {
            pe[e] = __expf(sv[e] - m_new);
            sum += pe[e];
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float raw = (e < 4 ? s0[e & 3] : s1[e & 3]) * p.scale;
            sv[e] = (p0 + 8 * c + e <= lim_q[u]) ? raw : -INFINITY;
            mx = fmaxf(mx, sv[e]);
          }
          m_new = fmaxf(m_run[u], max_xor16_xor32(mx));
#pragma unroll
          for (int e = 0; e < 8; e++) {
            pe[e] = (sv[e] == -INFINITY) ? 0.0f : __expf(sv[e] - m_new);
            sum += pe[e];
          }
        }
        sum = sum_xor16_xor32(sum);
        const float alpha = (m_run[u] == -INFINITY) ? 0.0f : __expf(m_run[u] - m_new);
        l_run[u] = l_run[u] * alpha + sum;
        m_run[u] = m_new;
        const half8_t pf = {(_Float16)pe[0], (_Float16)pe[1], (_Float16)pe[2], (_Float16)pe[3],
                            (_Float16)pe[4], (_Float16)pe[5], (_Float16)pe[6], (_Float16)pe[7]};
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
          for (int t = 0; t < DT; t++) o_acc[u][t] = o_acc[u][t] * alpha;
        }
#pragma unroll
        for (int t = 0; t < DT; t++) o_acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vv[t], pf, o_acc[u][t], 0, 0, 0);
      }
    }
  };
  uint4_t kr[K_LD], vr[V_LD];
  fetch(0, kr, vr);
  stash(0, kr, vr);
  __syncthreads();
  for (int st = 0; st < nstages; st++) {
    const bool more = st + 1 < nstages;  // uniform in the workgroup
    if (more) fetch(st + 1, kr, vr);
    compute(st);
    if (more) stash((st + 1) & 1, kr, vr);
    __syncthreads();
  }
  if (!active) return;
  _Float16 *obase = static_cast<_Float16 *>(p.out) + (size_t)b * p.o_b + (size_t)h * HD;
#pragma unroll
  for (int u = 0; u < QT; u++) {
    if (q0 + 16 * u + r >= p.Sq) continue;
    const float inv = l_run[u] > 0.0f ? 1.0f / l_run[u] : 0.0f;
    _Float16 *orow = obase + (size_t)(q0 + 16 * u + r) * p.o_s;
#pragma unroll
    for (int t = 0; t < DT; t++)
      store4<_Float16>(orow + 16 * t + 4 * c, o_acc[u][t][0] * inv, o_acc[u][t][1] * inv, o_acc[u][t][2] * inv, o_acc[u][t][3] * inv);
  }
}

// heads of one kv group that share a workgroup of gqa_shared_kv_kernel: the largest of 4, 2, 1 that divides the group
inline int shared_kv_hw_log2(int group) { return group % 4 == 0 ? 2 : (group % 2 == 0 ? 1 : 0); }

int32_t gqa_launch_shared_kv(const GqaArgs &a, int hd, hipStream_t s) {
  const int hw_log2 = shared_kv_hw_log2(a.Hq / a.Hkv);
  const int q_per_wg = 32 * (GQA_WAVES >> hw_log2);
  const dim3 grid((unsigned)(a.Hq >> hw_log2), (unsigned)((a.Sq + q_per_wg - 1) / q_per_wg), (unsigned)a.B), block(64 * GQA_WAVES);
  switch (hd) {
    case 32: hipLaunchKernelGGL((gqa_shared_kv_kernel<32>), grid, block, 0, s, a, hw_log2); break;
    case 64: hipLaunchKernelGGL((gqa_shared_kv_kernel<64>), grid, block, 0, s, a, hw_log2); break;
    case 96: hipLaunchKernelGGL((gqa_shared_kv_kernel<96>), grid, block, 0, s, a, hw_log2); break;
    case 128: hipLaunchKernelGGL((gqa_shared_kv_kernel<128>), grid, block, 0, s, a, hw_log2); break;
    default: return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention: head width %d (supported: 32, 64, 96, 128)", hd);
  }
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

template <typename TQ, typename TKV, typename TO, bool V_SLAB>
int32_t gqa_launch(const GqaArgs &a, int hd, hipStream_t s) {
  // many queries and a host-known context: one wave per 32 queries, no split over the keys
  if (a.Sq >= 64 && a.sk_minus_1 == nullptr) {
    const dim3 grid((unsigned)((a.Sq + 32 * GQA_WAVES - 1) / (32 * GQA_WAVES)), (unsigned)a.Hq, (unsigned)a.B), block(64 * GQA_WAVES);
    switch (hd) {
      case 32: hipLaunchKernelGGL((gqa_rows_kernel<32, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
      case 64: hipLaunchKernelGGL((gqa_rows_kernel<64, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
      case 96: hipLaunchKernelGGL((gqa_rows_kernel<96, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
      case 128: hipLaunchKernelGGL((gqa_rows_kernel<128, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
      default: return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention: head width %d (supported: 32, 64, 96, 128)", hd);
    }
    YSCV_HIP_TRY(hipGetLastError());
    return YSCV_HIP_OK;
  }
  const dim3 grid((unsigned)((a.Sq + 15) / 16), (unsigned)a.Hq, (unsigned)a.B), block(64 * GQA_WAVES);
  switch (hd) {
    case 32: hipLaunchKernelGGL((gqa_generic_kernel<32, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
    case 64: hipLaunchKernelGGL((gqa_generic_kernel<64, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
    case 96: hipLaunchKernelGGL((gqa_generic_kernel<96, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
    case 128: hipLaunchKernelGGL((gqa_generic_kernel<128, TQ, TKV, TO, V_SLAB>), grid, block, 0, s, a); break;
    default: return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention: head width %d (supported: 32, 64, 96, 128)", hd);
  }
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// decode step on the decoder's fp16 buffers with the rotary embedding and the cache append inside the kernel
int32_t gqa_launch_fused_decode(const GqaArgs &a, int hd, hipStream_t s) {
  const dim3 grid(1, (unsigned)a.Hq, (unsigned)a.B), block(64 * GQA_WAVES);
  switch (hd) {
    case 32: hipLaunchKernelGGL((gqa_generic_kernel<32, _Float16, _Float16, _Float16, true, true>), grid, block, 0, s, a); break;
    case 64: hipLaunchKernelGGL((gqa_generic_kernel<64, _Float16, _Float16, _Float16, true, true>), grid, block, 0, s, a); break;
    case 96: hipLaunchKernelGGL((gqa_generic_kernel<96, _Float16, _Float16, _Float16, true, true>), grid, block, 0, s, a); break;
    case 128: hipLaunchKernelGGL((gqa_generic_kernel<128, _Float16, _Float16, _Float16, true, true>), grid, block, 0, s, a); break;
    default: return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention: head width %d (supported: 32, 64, 96, 128)", hd);
  }
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// ---- RMSNorm over the last axis, f32 in and out ---------------------------------------------------------------
__global__ void __launch_bounds__(256) rms_norm_f32_kernel(const float *__restrict__ x, const float *__restrict__ gamma, int d,
                                                           float eps, float *__restrict__ y) {
  __shared__ float red[4];
  const float *row = x + (size_t)blockIdx.x * d;
  float *out = y + (size_t)blockIdx.x * d;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < d; i += 256) ss += row[i] * row[i];
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = red[0] + red[1] + red[2] + red[3];
  // rms = sqrt(sum / n + eps); inv_rms = 1 / rms; y = x * inv_rms * gamma (ops/norm.rs:1507-1516, in that order)
  const float inv_rms = 1.0f / sqrtf(ss / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += 256) out[i] = row[i] * inv_rms * gamma[i];
}

// ---- rotate-half RoPE in place on [seq][heads][d] f32 ------------------------------------------------------------
__global__ void __launch_bounds__(64) rope_f32_kernel(float *__restrict__ x, int heads, int d, int seq_offset, float theta) {
  const int pos = blockIdx.y, head = blockIdx.x;
  float *row = x + ((size_t)pos * heads + head) * d;
  const int half_d = d / 2;
  const float abs_pos = (float)(pos + seq_offset);
  for (int i = threadIdx.x; i < half_d; i += 64) {
    const float inv_freq = 1.0f / powf(theta, 2.0f * (float)i / (float)d);
    float sn, cs;
    sincosf(inv_freq * abs_pos, &sn, &cs);
    const float x0 = row[i], x1 = row[i + half_d];
    row[i] = x0 * cs - x1 * sn;
    row[i + half_d] = x0 * sn + x1 * cs;
  }
}


// ---- small kernels of the prompt pass (rows = consecutive positions of one sequence) ------------------------------
// RoPE on the q and k heads of every row (row i sits at position start_pos + i), k and v appended to batch row 0 of
// the cache: the arithmetic of the decode step's rope + append, one launch for all rows.  A workgroup takes the (up
// to eight) rows whose positions share one 8-position slab of the V layout: the angle of a pair is worked out once per
// position for all heads, and the values of a channel at the slab's positions leave as one 16-byte store where the
// whole slab is new.
__global__ void __launch_bounds__(256) prefill_rope_append_kernel(_Float16 *__restrict__ qkv, int rows, int start_pos, int hq, int hkv,
                                                                  int hd, float theta, int max_ctx, _Float16 *__restrict__ kc,
                                                                  _Float16 *__restrict__ vc) {
  const int tid = threadIdx.x;
  const int slab = start_pos / 8 + (int)blockIdx.x;
  const int p_lo = max(start_pos, slab * 8), p_hi = min(start_pos + rows, slab * 8 + 8);  // positions [p_lo, p_hi)
  const size_t row_elems = (size_t)(hq + 2 * hkv) * hd;
  const int half_d = hd / 2;
  // the angle of pair i at each of the slab's positions, once for all heads
  __shared__ float cs_s[8][64], sn_s[8][64];
  const int n_pos = p_hi - p_lo;
  for (int idx = tid; idx < n_pos * half_d; idx += 256) {
    const int e = idx / half_d, i = idx % half_d;
    const float inv_freq = 1.0f / powf(theta, (float)(2 * i) / (float)hd);
    sincosf(inv_freq * (float)(p_lo + e), &sn_s[e][i], &cs_s[e][i]);
  }
  __syncthreads();
  const int slots = hq + hkv, vecs = half_d / 8;  // eight pairs per item: 16-byte loads and stores
#pragma unroll 2
  // blockIdx.y takes every gridDim.y-th item of the slab (short prompts have few slabs and would leave the CUs idle)
  for (int item = tid + 256 * (int)blockIdx.y; item < n_pos * slots * vecs; item += 256 * (int)gridDim.y) {
    const int i0 = (item % vecs) * 8, slot = (item / vecs) % slots, e = item / (vecs * slots);
    const int pos = p_lo + e;
    _Float16 *src = qkv + (size_t)(pos - start_pos) * row_elems + (size_t)slot * hd;
    const half8_t x0 = *reinterpret_cast<const half8_t *>(src + i0), x1 = *reinterpret_cast<const half8_t *>(src + i0 + half_d);
    half8_t y0, y1;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float cs = cs_s[e][i0 + j], sn = sn_s[e][i0 + j];
      const float a = (float)x0[j], b = (float)x1[j];
      float f0 = fmaf(a, cs, -(b * sn)), f1 = fmaf(a, sn, b * cs);
      asm volatile("" : "+v"(f0), "+v"(f1));  // the f32 value exists before it is narrowed (no mixed-precision fma)
      y0[j] = (_Float16)f0;
      y1[j] = (_Float16)f1;
    }
    _Float16 *dst = slot < hq ? src : kc + ((size_t)(slot - hq) * max_ctx + pos) * hd;
    *reinterpret_cast<half8_t *>(dst + i0) = y0;
    *reinterpret_cast<half8_t *>(dst + i0 + half_d) = y1;
  }
  // v: channel ch of kv head kvh at the slab's positions
  const _Float16 *vsrc = qkv + (size_t)(hq + hkv) * hd;
  const bool whole = p_hi - p_lo == 8;
  for (int idx = tid + 256 * (int)blockIdx.y; idx < hkv * hd; idx += 256 * (int)gridDim.y) {
    const int kvh = idx / hd, ch = idx % hd;
    _Float16 *dst = vc + (((size_t)kvh * (max_ctx / 8) + slab) * hd + ch) * 8;
    if (whole) {
      half8_t v;
#pragma unroll
      for (int e = 0; e < 8; e++) v[e] = vsrc[(size_t)(p_lo - start_pos + e) * row_elems + idx];
      *reinterpret_cast<half8_t *>(dst) = v;
    } else {
      for (int pos = p_lo; pos < p_hi; pos++) dst[pos & 7] = vsrc[(size_t)(pos - start_pos) * row_elems + idx];
    }
  }
}

__global__ void bias_add_f16_kernel(_Float16 *__restrict__ x, const _Float16 *__restrict__ bias, size_t rows, size_t n) {
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < rows * n; idx += (size_t)gridDim.x * blockDim.x)
    x[idx] = (_Float16)((float)x[idx] + (float)bias[idx % n]);
}

unsigned flat_grid(size_t n) {
  const size_t b = (n + 255) / 256;
  return (unsigned)(b > 65535 ? 65535 : (b < 1 ? 1 : b));
}

}  // namespace

int32_t launch_prefill_rope_append(_Float16 *qkv, int rows, int start_pos, int hq, int hkv, int hd, float theta, int max_ctx,
                                   _Float16 *kc, _Float16 *vc, hipStream_t s) {
  if (hd > 128 || hd % 16 != 0) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "rope + append: head width %d", hd);
  const int slabs = (start_pos + rows - 1) / 8 - start_pos / 8 + 1;
  int parts = 512 / slabs;  // about two workgroups per CU
  parts = parts < 1 ? 1 : (parts > 16 ? 16 : parts);
  hipLaunchKernelGGL(prefill_rope_append_kernel, dim3(slabs, parts), dim3(256), 0, s, qkv, rows, start_pos, hq, hkv, hd, theta, max_ctx,
                     kc, vc);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}
int32_t launch_bias_add_f16(_Float16 *x, const _Float16 *bias, size_t rows, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(bias_add_f16_kernel, dim3(flat_grid(rows * n)), dim3(256), 0, s, x, bias, rows, n);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

// Attention of `rows` query rows against the decoder's fp16 cache of one layer.  qkv: [rows][(hq + 2 hkv) hd] with
// the query heads already rotated; out: [rows][hq hd].
//   decode (pos_ptr != null): row b is batch row b at the position *pos_ptr, cache rows [0, *pos_ptr];
//   prompt ingestion (pos_ptr == null): the rows are consecutive positions start_pos .. of batch row 0, row i sees
//   cache rows [0, start_pos + i].
int32_t launch_gqa_cache(const _Float16 *qkv, const _Float16 *kc, const _Float16 *vc, const int32_t *pos_ptr, int rows,
                         int start_pos, int hq, int hkv, int hd, int max_ctx, _Float16 *out, hipStream_t s, float rope_theta,
                         _Float16 *qrot) {
  GqaArgs a{};
  a.theta = rope_theta;
  a.qrot = qrot;
  const long long row_elems = (long long)(hq + 2 * hkv) * hd;
  a.q = qkv;
  a.k = kc;
  a.v = vc;
  a.out = out;
  a.k_s = hd;
  a.k_h = (long long)max_ctx * hd;
  a.v_h = (long long)max_ctx * hd;
  a.v_s = 0;
  a.Hq = hq;
  a.Hkv = hkv;
  a.scale = 1.0f / sqrtf((float)hd);
  if (pos_ptr) {
    a.B = rows;
    a.Sq = 1;
    a.Sk = 1;
    a.sk_minus_1 = pos_ptr;
    a.causal_base = -1;
    a.q_b = row_elems;
    a.q_s = 0;
    a.k_b = (long long)hkv * max_ctx * hd;
    a.v_b = a.k_b;
    a.o_b = (long long)hq * hd;
    a.o_s = 0;
  } else {
    a.B = 1;
    a.Sq = rows;
    a.Sk = start_pos + rows;
    a.sk_minus_1 = nullptr;
    a.causal_base = start_pos;
    a.q_b = 0;
    a.q_s = row_elems;
    a.k_b = 0;
    a.v_b = 0;
    a.o_b = 0;
    a.o_s = (long long)hq * hd;
  }
  // decode mode with qrot given: q / k / v of the new position come unrotated, rope + append happen in the kernel
  if (pos_ptr && qrot) return gqa_launch_fused_decode(a, hd, s);
  // prompt mode with enough rows: the kernel that stages K / V in LDS for four waves (its K rows must be contiguous
  // 16-byte pieces, which the cache's are)
  if (!pos_ptr && rows >= 64 && (max_ctx & 7) == 0) return gqa_launch_shared_kv(a, hd, s);
  return gqa_launch<_Float16, _Float16, _Float16, true>(a, hd, s);
}

extern "C" {

int32_t yscv_hip_rms_norm_dev(const float *x, const float *gamma, size_t rows, size_t d, float eps, float *y, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(x && gamma && y, "null argument");
  YSCV_REQUIRE(std::isfinite(eps) && eps > 0.0f, "rms_norm: epsilon must be finite and > 0");
  YSCV_REQUIRE(d > 0 && d < ((size_t)1 << 31) && rows < ((size_t)1 << 31), "rms_norm: bad shape %zu x %zu", rows, d);
  if (rows == 0) return YSCV_HIP_OK;
  hipLaunchKernelGGL(rms_norm_f32_kernel, dim3((unsigned)rows), dim3(256), 0, as_stream(stream), x, gamma, (int)d, eps, y);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t yscv_hip_rope_dev(float *q, float *k, size_t num_q_heads, size_t num_kv_heads, size_t d_head, size_t seq_len,
                          size_t seq_offset, float theta, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(q && k, "null argument");
  YSCV_REQUIRE(d_head % 2 == 0 && d_head > 0, "rope: d_head must be even (got %zu)", d_head);
  YSCV_REQUIRE(seq_len + seq_offset < ((size_t)1 << 24), "rope: position beyond 2^24");
  YSCV_REQUIRE(seq_len < 65536 && num_q_heads < ((size_t)1 << 31) && num_kv_heads < ((size_t)1 << 31), "rope: shape too large");
  if (seq_len == 0) return YSCV_HIP_OK;
  hipStream_t s = as_stream(stream);
  if (num_q_heads > 0) {
    hipLaunchKernelGGL(rope_f32_kernel, dim3((unsigned)num_q_heads, (unsigned)seq_len), dim3(64), 0, s, q, (int)num_q_heads, (int)d_head,
                       (int)seq_offset, theta);
    YSCV_HIP_TRY(hipGetLastError());
  }
  if (num_kv_heads > 0) {
    hipLaunchKernelGGL(rope_f32_kernel, dim3((unsigned)num_kv_heads, (unsigned)seq_len), dim3(64), 0, s, k, (int)num_kv_heads, (int)d_head,
                       (int)seq_offset, theta);
    YSCV_HIP_TRY(hipGetLastError());
  }
  return YSCV_HIP_OK;
}

int32_t yscv_hip_gqa_attention_dev(const float *q, const float *k, const float *v, size_t batch, size_t seq_q, size_t seq_k,
                                   size_t num_q_heads, size_t num_kv_heads, size_t d_head, float *out, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(q && k && v && out, "null argument");
  YSCV_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
               "GroupQueryAttention: %zu query heads over %zu kv heads", num_q_heads, num_kv_heads);
  YSCV_REQUIRE(batch < 65536 && num_q_heads < 65536 && seq_q < ((size_t)1 << 24) && seq_k < ((size_t)1 << 24),
               "GroupQueryAttention: shape too large");
  YSCV_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(out)) & 15) == 0,
               "GroupQueryAttention: tensors must be 16-byte aligned");
  if (batch == 0 || seq_q == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(seq_k > 0, "GroupQueryAttention: no key positions");
  GqaArgs a{};
  a.q = q;
  a.k = k;
  a.v = v;
  a.out = out;
  a.q_s = (long long)(num_q_heads * d_head);
  a.q_b = (long long)seq_q * a.q_s;
  a.k_s = (long long)(num_kv_heads * d_head);
  a.k_b = (long long)seq_k * a.k_s;
  a.k_h = (long long)d_head;
  a.v_s = a.k_s;
  a.v_b = a.k_b;
  a.v_h = a.k_h;
  a.o_s = a.q_s;
  a.o_b = a.q_b;
  a.B = (int)batch;
  a.Sq = (int)seq_q;
  a.Sk = (int)seq_k;
  a.Hq = (int)num_q_heads;
  a.Hkv = (int)num_kv_heads;
  a.causal_base = -1;
  a.sk_minus_1 = nullptr;
  a.scale = 1.0f / sqrtf((float)d_head);
  return gqa_launch<float, float, float, false>(a, (int)d_head, as_stream(stream));
}

}  // extern "C"

}  // namespace yscv
