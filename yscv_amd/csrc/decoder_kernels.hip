// Glue kernels of the Llama-style decode step around the int4 projections: embedding lookup,
// RMSNorm, rotary embedding + KV-cache append, single-token grouped-query attention over an fp16
// KV cache, greedy pick.  Reference semantics (tolerance-checked, these use libm-class functions):
//   RMSNorm  y = x * (1/sqrt(mean(x^2) + eps)) * gamma   crates/yscv-kernels/src/ops/norm.rs:1497-1518
//   RoPE     rotate-half pairs (i, i + d/2), inv_freq[i] = 1/theta^(2i/d), angle = pos * inv_freq[i]
//                                                        crates/yscv-kernels/src/ops/rope.rs:24-117
//   GQA      kv_h = q_h / (Hq/Hkv), scores * 1/sqrt(d), max-subtracted softmax
//                                                        crates/yscv-onnx/src/runner/linear.rs:552-646
//   greedy   last index among equal maxima              apps/llm-bench/src/main.rs:538-543
// The reference GQA op has no mask and no cache; attending to every cached position up to and
// including the current token is the causal decode the llm-bench harness gets from its ONNX graph.
//
// KV cache layout (per layer, fp16), chosen so that both attention matmuls run on the matrix
// cores with fully coalesced loads:
//   K: [batch][kv_head][pos][head_dim]                      one 256 B row per position
//   V: [batch][kv_head][pos / 8][head_dim][8]               8 positions interleaved per d
// so a lane of v_mfma_f32_16x16x32_f16 reads 8 consecutive d of one position (K, B operand of
// Q K^T) or 8 consecutive positions of one d (V, B operand of P V) as one 128-bit load.
#include "decoder.hpp"
#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

// ---- embedding: h[b][:] = table[token[b]][:] (fp16 -> f32 residual stream) ----------------------
__global__ void embed_kernel(const int32_t *__restrict__ tokens, const _Float16 *__restrict__ table, int d,
                             int vocab, float *__restrict__ h) {
  const int b = blockIdx.x;
  int tok = tokens[b];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  for (int i = threadIdx.x; i < d; i += blockDim.x) h[(size_t)b * d + i] = (float)table[(size_t)tok * d + i];
}

// embedding lookup that also feeds the first norm in its folded form (NormFold, kernels.hpp): the row stays in
// registers (d <= 4096) until its sum of squares is known, which gives the power of two pre[b] near 1 / (4 rms);
// xg = fp16(h * gamma * pre[b]), and the sum as the row's single partial
__global__ void __launch_bounds__(256) embed_norm_kernel(const int32_t *__restrict__ tokens, const _Float16 *__restrict__ table,
                                                         int d, int vocab, float eps, float *__restrict__ h,
                                                         const float *__restrict__ gamma, _Float16 *__restrict__ xg,
                                                         float *__restrict__ ss_out, int ss_stride, float *__restrict__ pre) {
  __shared__ float red4[4];
  const int b = blockIdx.x;
  int tok = tokens[b];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  // eight consecutive values per thread and piece, two pieces: 4096 values at most (d is a multiple of 8)
  constexpr int PIECES = 2;
  half8_t raw[PIECES];
  float4_t gam[PIECES][2];
#pragma unroll
  for (int u = 0; u < PIECES; u++) {
    const int i = (u * 256 + (int)threadIdx.x) * 8;
    const bool in = i < d;
    raw[u] = in ? *reinterpret_cast<const half8_t *>(table + (size_t)tok * d + i) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    // gamma is requested with the row, not after the sum
    gam[u][0] = in ? *reinterpret_cast<const float4_t *>(gamma + i) : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    gam[u][1] = in ? *reinterpret_cast<const float4_t *>(gamma + i + 4) : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }
  float sq = 0.0f;
#pragma unroll
  for (int u = 0; u < PIECES; u++) {
    const int i = (u * 256 + (int)threadIdx.x) * 8;
    if (i < d) {
      float4_t lo, hi;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        lo[e] = (float)raw[u][e];
        hi[e] = (float)raw[u][4 + e];
      }
      *reinterpret_cast<float4_t *>(h + (size_t)b * d + i) = lo;
      *reinterpret_cast<float4_t *>(h + (size_t)b * d + i + 4) = hi;
    }
#pragma unroll
    for (int e = 0; e < 8; e++) sq += (float)raw[u][e] * (float)raw[u][e];
  }
  sq = wave_sum(sq);
  if ((threadIdx.x & 63) == 0) red4[threadIdx.x >> 6] = sq;
  __syncthreads();
  const float total = ((red4[0] + red4[1]) + red4[2]) + red4[3];
  const float scale = norm_fold_prescale(1.0f / sqrtf(total / (float)d + eps));
#pragma unroll
  for (int u = 0; u < PIECES; u++) {
    const int i = (u * 256 + (int)threadIdx.x) * 8;
    if (i < d) {
      half8_t o;
#pragma unroll
      for (int e = 0; e < 8; e++)
        o[e] = (_Float16)fminf(fmaxf((float)raw[u][e] * gam[u][e >> 2][e & 3] * scale, -65504.0f), 65504.0f);
      *reinterpret_cast<half8_t *>(xg + (size_t)b * d + i) = o;
    }
  }
  if (threadIdx.x == 0) {
    ss_out[(size_t)b * ss_stride] = total;
    pre[b] = scale;
  }
}

// ---- RMSNorm: f32 residual -> fp16 normalised activations -----------------------------------------
__global__ void __launch_bounds__(256) rmsnorm_kernel(const float *__restrict__ h, const float *__restrict__ gamma,
                                                      int d, float eps, _Float16 *__restrict__ out) {
  __shared__ float red[4];
  const int b = blockIdx.x;
  const float *row = h + (size_t)b * d;
  // a row of up to 8192 values stays in registers between the two passes (one memory round trip instead of two);
  // longer rows are read again
  constexpr int KEEP = 8;
  float4_t keep[KEEP];
  const bool fits = d <= KEEP * 256 * 4;
  float ss = 0.0f;
  if (fits) {
#pragma unroll
    for (int u = 0; u < KEEP; u++) {
      const int i = (u * 256 + (int)threadIdx.x) * 4;
      keep[u] = i < d ? *reinterpret_cast<const float4_t *>(row + i) : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int u = 0; u < KEEP; u++) {
      const float4_t v = keep[u];
      if ((u * 256 + (int)threadIdx.x) * 4 < d) ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
  } else {
    for (int i = threadIdx.x * 4; i < d; i += blockDim.x * 4) {
      float4_t v = *reinterpret_cast<const float4_t *>(row + i);
      ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
  }
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = red[0] + red[1] + red[2] + red[3];
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  if (fits) {
#pragma unroll
    for (int u = 0; u < KEEP; u++) {
      const int i = (u * 256 + (int)threadIdx.x) * 4;
      if (i < d) {
        const float4_t v = keep[u];
        const float4_t g = *reinterpret_cast<const float4_t *>(gamma + i);
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (_Float16)(v[e] * inv * g[e]);
        *reinterpret_cast<half4_t *>(out + (size_t)b * d + i) = o;
      }
    }
    return;
  }
  for (int i = threadIdx.x * 4; i < d; i += blockDim.x * 4) {
    float4_t v = *reinterpret_cast<const float4_t *>(row + i);
    float4_t g = *reinterpret_cast<const float4_t *>(gamma + i);
    half4_t o;
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = (_Float16)(v[e] * inv * g[e]);
    *reinterpret_cast<half4_t *>(out + (size_t)b * d + i) = o;
  }
}

// sin and cos of the angle of pair i at position pos: inv_freq[i] = 1 / theta^(2i / d)
struct SinCos {
  float sn, cs;
};
__device__ __forceinline__ SinCos rope_sincos(float theta, int i, int d, int pos) {
  const float inv_freq = 1.0f / powf(theta, (float)(2 * i) / (float)d);
  SinCos r;
  sincosf(inv_freq * (float)pos, &r.sn, &r.cs);
  return r;
}

// rotate-half of one pair, written with explicit fused multiply-adds so that every kernel that rotates rounds alike
__device__ __forceinline__ void rope_pair_f32(float x0, float x1, float cs, float sn, float &y0, float &y1) {
  y0 = fmaf(x0, cs, -(x1 * sn));
  y1 = fmaf(x0, sn, x1 * cs);
}
// f32 -> fp16 of a value that exists as an f32 first.  Without the empty asm the compiler may merge the conversion
// into the multiply-add that produced the value (a mixed-precision fma that rounds once, straight to fp16), in one
// kernel and not in another: one rotated q element in a few thousand then differs by an fp16 ulp between them.
__device__ __forceinline__ _Float16 f16_of_f32(float v) {
  asm volatile("" : "+v"(v));
  return (_Float16)v;
}
__device__ __forceinline__ void rope_pair(float x0, float x1, float cs, float sn, _Float16 &y0, _Float16 &y1) {
  float f0, f1;
  rope_pair_f32(x0, x1, cs, sn, f0, f1);
  y0 = f16_of_f32(f0);
  y1 = f16_of_f32(f1);
}

// ---- RoPE on q (in place) and k, then append k / v to the cache -------------------------------------
// qkv: [batch][(Hq + 2*Hkv) * D] fp16, q heads first, then k heads, then v heads.
// one workgroup per (batch row, head slot); head slots: Hq q heads, Hkv k heads, Hkv v heads.
__global__ void __launch_bounds__(64) rope_append_kernel(_Float16 *__restrict__ qkv, const int32_t *__restrict__ pos_ptr,
                                                         int hq, int hkv, int hd, float theta, int max_ctx,
                                                         _Float16 *__restrict__ kc, _Float16 *__restrict__ vc) {
  const int b = blockIdx.y;
  const int slot = blockIdx.x;
  const int pos = *pos_ptr;
  const int row_elems = (hq + 2 * hkv) * hd;
  _Float16 *src = qkv + (size_t)b * row_elems + (size_t)slot * hd;
  const int half_d = hd / 2;
  if (slot < hq + hkv) {
    // rotate-half: (x[i], x[i + d/2]) -> (x0 cos - x1 sin, x0 sin + x1 cos)
    for (int i = threadIdx.x; i < half_d; i += blockDim.x) {
      const SinCos sc = rope_sincos(theta, i, hd, pos);
      const float sn = sc.sn, cs = sc.cs;
      const float x0 = (float)src[i], x1 = (float)src[i + half_d];
      _Float16 y0, y1;
      rope_pair(x0, x1, cs, sn, y0, y1);
      if (slot < hq) {
        src[i] = y0;
        src[i + half_d] = y1;
      } else {
        const int kvh = slot - hq;
        _Float16 *dst = kc + (((size_t)b * hkv + kvh) * max_ctx + pos) * hd;
        dst[i] = y0;
        dst[i + half_d] = y1;
      }
    }
  } else {
    const int kvh = slot - hq - hkv;
    _Float16 *dst = vc + ((((size_t)b * hkv + kvh) * (max_ctx / 8) + pos / 8) * hd) * 8 + (pos & 7);
    for (int i = threadIdx.x; i < hd; i += blockDim.x) dst[(size_t)i * 8] = src[i];
  }
}

// natural [batch][pos][kv_head][d] fp16 (host order) -> the two cache layouts, for positions [0, npos)
__global__ void kv_relayout_kernel(const _Float16 *__restrict__ k_nat, const _Float16 *__restrict__ v_nat, int batch,
                                   int npos, int hkv, int hd, int max_ctx, _Float16 *__restrict__ kc,
                                   _Float16 *__restrict__ vc) {
  const size_t total = (size_t)batch * npos * hkv * hd;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const int i = idx % hd;
    const int kvh = (idx / hd) % hkv;
    const int pos = (idx / hd / hkv) % npos;
    const int b = idx / hd / hkv / npos;
    kc[(((size_t)b * hkv + kvh) * max_ctx + pos) * hd + i] = k_nat[idx];
    vc[((((size_t)b * hkv + kvh) * (max_ctx / 8) + pos / 8) * hd + i) * 8 + (pos & 7)] = v_nat[idx];
  }
}

// ---- single-token GQA attention, split over the context ----------------------------------------------
// grid (chunks, Hkv, batch), 4 waves per workgroup, each wave owns 32 consecutive positions and the
// GROUP = Hq/Hkv (<= 4) query heads that share this kv head.  Per wave:
//   S = Q K^T   two 16-position blocks x 4 MFMAs (k = 128 d), Q rows sit at MFMA rows 4*h
//   online-softmax statistics per head over its 32 positions
//   O = P V     eight 16-wide d tiles x 1 MFMA (k = 32 positions), P as fp16 through LDS
// then the 4 waves merge in LDS and write one (max, sum, o[128]) partial per (batch, head, chunk).
constexpr int ATT_WAVES = 4;
constexpr int ATT_POS_PER_WAVE = 32;
constexpr int ATT_CHUNK = ATT_WAVES * ATT_POS_PER_WAVE;  // 128 positions per workgroup

// KV8: the cache holds int8 rows with one f32 scale per (batch row, position) for K and for V (KvCache with
// KvDtype::I8, crates/yscv-onnx/src/runner/kv_cache.rs:45-79: values read back as q * scale).  int8 values are exact in
// fp16, so both operands carry the bare int8 values: the K scale multiplies the finished score, the V scale the
// softmax weight of its position before that is rounded to fp16 (one rounding per product, where scaling V itself
// would round twice).  Eight bytes -> eight fp16 values: b ^ 0x80 is b + 128 as an unsigned byte u, the fp16 with bits
// 0x6400 | u is 1024 + u, and subtracting 1152 leaves b (two byte permutes and two packed adds per four values).
typedef int int2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ half8_t i8x8_to_half8(int2_t raw) {
  const half2_t bias = {(_Float16)(-1152.0f), (_Float16)(-1152.0f)};
  half8_t h;
#pragma unroll
  for (int w = 0; w < 2; w++) {
    const uint32_t x = (uint32_t)raw[w] ^ 0x80808080u;
    // v_perm_b32: result byte i = byte sel[i] of {0x64646464 (bytes 4..7), x (bytes 0..3)}
    const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);
    const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);
    const half2_t a = __builtin_bit_cast(half2_t, lo) + bias;
    const half2_t c = __builtin_bit_cast(half2_t, hi) + bias;
    h[4 * w + 0] = a[0];
    h[4 * w + 1] = a[1];
    h[4 * w + 2] = c[0];
    h[4 * w + 3] = c[1];
  }
  return h;
}

// int8 cache: the value scale of a position rides on its softmax weight, which the second MFMA takes as fp16.  The
// largest scale among the wave's live positions, rounded up to a power of two S, is taken out first: the weights carry
// v_scale / S <= 1 (a row of small values, absmax 1e-4 say, would otherwise push them into fp16's subnormals) and the
// f32 result is multiplied by S.  Returns S; *inv = 1 / S (both exact).
__device__ __forceinline__ float v_scale_pow2(float v0, float v1, bool live0, bool live1, float *inv) {
  const float m = row_max16(fmaxf(live0 ? v0 : 0.0f, live1 ? v1 : 0.0f));
  int e = 0;
  if (m > 0.0f && m < INFINITY) (void)frexpf(m, &e);  // m = f * 2^e, f in [0.5, 1)
  *inv = ldexpf(1.0f, -e);
  return ldexpf(1.0f, e);
}

template <bool KV8>
__global__ void __launch_bounds__(256) attn_partial_kernel(const _Float16 *__restrict__ qkv,
                                                           const void *__restrict__ kc_v,
                                                           const void *__restrict__ vc_v,
                                                           const float *__restrict__ ks, const float *__restrict__ vs,
                                                           const int32_t *__restrict__ pos_ptr, int hq, int hkv,
                                                           int max_ctx, int max_chunks, float scale,
                                                           float *__restrict__ part) {
  constexpr int HD = 128;
  __shared__ __attribute__((aligned(16))) _Float16 p_lds[ATT_WAVES][4][32];
  __shared__ float w_m[ATT_WAVES][4], w_l[ATT_WAVES][4];
  __shared__ float w_o[ATT_WAVES][4][HD];
  const int chunk = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int group = hq / hkv;
  const int n_ctx = *pos_ptr + 1;  // the current token was appended before this kernel
  const int p0 = chunk * ATT_CHUNK + wave * ATT_POS_PER_WAVE;
  const int row_elems = (hq + 2 * hkv) * HD;
  const bool wave_live = p0 < n_ctx;

  float m_h = -INFINITY, l_h = 0.0f;   // statistics of head c (lane group) -- valid for c < group
  float o_acc[8];
#pragma unroll
  for (int t = 0; t < 8; t++) o_acc[t] = 0.0f;

  if (wave_live) {
    // Q operand: MFMA row 4*h carries head h of this group; lane (r, c) holds d = 32c + 8j + 0..7
    half8_t qa[4];
    {
      const int h = r >> 2;
      const bool valid = ((r & 3) == 0) && h < group;
      const _Float16 *qsrc = qkv + (size_t)b * row_elems + (size_t)(kvh * group + h) * HD + 32 * c;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
        qa[j] = valid ? *reinterpret_cast<const half8_t *>(qsrc + 8 * j) : z;
      }
    }
    const size_t k_off = (((size_t)b * hkv + kvh) * max_ctx + p0) * HD;
    const size_t v_off = ((((size_t)b * hkv + kvh) * (max_ctx / 8) + p0 / 8) * HD) * 8;
    // issue every load of this wave up front: 8 KiB of K, 8 KiB of V (half of that from an int8 cache)
    half8_t kf[2][4], vf[8];
    float k_scale[2] = {1.0f, 1.0f}, v_scale[2] = {1.0f, 1.0f};  // of position p0 + 16 pb + r
    if constexpr (KV8) {
      const int8_t *kbase = static_cast<const int8_t *>(kc_v) + k_off;
      const int8_t *vbase = static_cast<const int8_t *>(vc_v) + v_off;
      int2_t kraw[2][4], vraw[8];
#pragma unroll
      for (int pb = 0; pb < 2; pb++) {
        k_scale[pb] = ks[(size_t)b * max_ctx + p0 + pb * 16 + r];
        v_scale[pb] = vs[(size_t)b * max_ctx + p0 + pb * 16 + r];
#pragma unroll
        for (int j = 0; j < 4; j++)
          kraw[pb][j] = *reinterpret_cast<const int2_t *>(kbase + (size_t)(pb * 16 + r) * HD + 32 * c + 8 * j);
      }
#pragma unroll
      for (int t = 0; t < 8; t++) vraw[t] = *reinterpret_cast<const int2_t *>(vbase + ((size_t)c * HD + t * 16 + r) * 8);
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
#pragma unroll
        for (int j = 0; j < 4; j++) kf[pb][j] = i8x8_to_half8(kraw[pb][j]);
#pragma unroll
      for (int t = 0; t < 8; t++) vf[t] = i8x8_to_half8(vraw[t]);
    } else {
      const _Float16 *kbase = static_cast<const _Float16 *>(kc_v) + k_off;
      const _Float16 *vbase = static_cast<const _Float16 *>(vc_v) + v_off;
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
#pragma unroll
        for (int j = 0; j < 4; j++)
          kf[pb][j] = *reinterpret_cast<const half8_t *>(kbase + (size_t)(pb * 16 + r) * HD + 32 * c + 8 * j);
#pragma unroll
      for (int t = 0; t < 8; t++)
        vf[t] = *reinterpret_cast<const half8_t *>(vbase + ((size_t)c * HD + t * 16 + r) * 8);
    }

    float s[2];
#pragma unroll
    for (int pb = 0; pb < 2; pb++) {
      float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 4; j++) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[j], kf[pb][j], d, 0, 0, 0);
      // lane (r, c): score of head c at position p0 + 16*pb + r
      const int p = p0 + pb * 16 + r;
      s[pb] = (p < n_ctx) ? d[0] * scale * k_scale[pb] : -INFINITY;
    }
    const float mx = row_max16(fmaxf(s[0], s[1]));  // over the 16 lanes of a group: DPP moves, no LDS round trips
    const float e0 = (s[0] == -INFINITY) ? 0.0f : __expf(s[0] - mx);
    const float e1 = (s[1] == -INFINITY) ? 0.0f : __expf(s[1] - mx);
    const float sum = row_sum16(e0 + e1);
    m_h = mx;
    l_h = sum;
    float vS = 1.0f, vS_inv = 1.0f;
    if constexpr (KV8) vS = v_scale_pow2(v_scale[0], v_scale[1], p0 + r < n_ctx, p0 + 16 + r < n_ctx, &vS_inv);
    if (c < 4) {
      // int8 cache: the V scale of the position rides on its weight (a dead position has weight 0 whatever its scale)
      p_lds[wave][c][r] = KV8 ? (e0 == 0.0f ? (_Float16)0.0f : (_Float16)(e0 * (v_scale[0] * vS_inv))) : (_Float16)e0;
      p_lds[wave][c][16 + r] = KV8 ? (e1 == 0.0f ? (_Float16)0.0f : (_Float16)(e1 * (v_scale[1] * vS_inv))) : (_Float16)e1;
    }
    __builtin_amdgcn_wave_barrier();  // LDS is in order per wave: the reads below see the writes above
    // P operand: MFMA row 4*h = head h, lane (r, c) holds positions 8c .. 8c+7 of this wave's 32
    half8_t pa = {0, 0, 0, 0, 0, 0, 0, 0};
    if ((r & 3) == 0 && (r >> 2) < group) pa = *reinterpret_cast<const half8_t *>(&p_lds[wave][r >> 2][8 * c]);
    // V rows past the context hold stale or unwritten bits; their weights are exactly 0, but 0 * NaN
    // would poison the sum, so blank the operand where the whole 8-position slab is out of range.
#pragma unroll
    for (int t = 0; t < 8; t++) {
      half8_t vv = vf[t];
      if (p0 + 8 * c >= n_ctx) vv = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      else if (p0 + 8 * c + 8 > n_ctx) {
#pragma unroll
        for (int e = 0; e < 8; e++)
          if (p0 + 8 * c + e >= n_ctx) vv[e] = (_Float16)0.0f;
      }
      float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
      d = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vv, d, 0, 0, 0);
      o_acc[t] = KV8 ? d[0] * vS : d[0];  // lane (r, c): o of head c at d = 16 t + r
    }
  }

  // ---- merge the 4 waves ---------------------------------------------------------------------------
  if (c < 4) {
    if (r == 0) {
      w_m[wave][c] = m_h;
      w_l[wave][c] = l_h;
    }
#pragma unroll
    for (int t = 0; t < 8; t++) w_o[wave][c][t * 16 + r] = o_acc[t];
  }
  __syncthreads();
  // thread -> (head h = tid / 64 ... ) : 4 heads x 128 d = 512 values, 256 threads -> 2 each
  for (int idx = threadIdx.x; idx < group * HD; idx += blockDim.x) {
    const int h = idx / HD, dd = idx % HD;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; w++) mx = fmaxf(mx, w_m[w][h]);
    float l = 0.0f, o = 0.0f;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; w++) {
      const float f = (w_m[w][h] == -INFINITY) ? 0.0f : __expf(w_m[w][h] - mx);
      l += w_l[w][h] * f;
      o += w_o[w][h][dd] * f;
    }
    const int head = kvh * group + h;
    float *dst = part + (((size_t)b * hq + head) * max_chunks + chunk) * (HD + 2);
    dst[2 + dd] = o;
    if (dd == 0) {
      dst[0] = mx;
      dst[1] = l;
    }
  }
}

// merge the per-chunk partials: one workgroup per (batch, head), 128 threads = one per d.  The chunk maxima and
// sums are fetched by one thread each (one memory round trip instead of one per chunk), the softmax weights of the
// chunks go through LDS, and the weighted sum over the chunks keeps several loads in flight.
__global__ void __launch_bounds__(128) attn_combine_kernel(const float *__restrict__ part,
                                                           const int32_t *__restrict__ pos_ptr, int hq,
                                                           int max_chunks, _Float16 *__restrict__ out) {
  constexpr int HD = 128;
  constexpr int CAP = 256;  // chunks whose weights fit the LDS table; longer contexts take the tail loop below
  __shared__ float wgt[CAP];
  __shared__ float red_m[2], red_l[2];
  const int head = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int n_ctx = *pos_ptr + 1;
  const int chunks = (n_ctx + ATT_CHUNK - 1) / ATT_CHUNK;
  const float *src = part + (((size_t)b * hq + head) * max_chunks) * (HD + 2);
  constexpr int FAST = 32;  // contexts up to 32 chunks: every load of the kernel is requested at once
  if (chunks <= FAST) {
    float po[FAST];
#pragma unroll
    for (int ch = 0; ch < FAST; ch++) po[ch] = src[(size_t)(ch < chunks ? ch : chunks - 1) * (HD + 2) + 2 + tid];
    // both waves fetch the (maximum, sum) pairs of all chunks, one chunk per lane: each wave then has the merge
    // statistics without LDS or a barrier, and a chunk's weight reaches every lane as a scalar read of its lane
    const int ln = tid & 63;
    float pm = -INFINITY, pl = 0.0f;
    if (ln < chunks) {
      pm = src[(size_t)ln * (HD + 2)];
      pl = src[(size_t)ln * (HD + 2) + 1];
    }
    const float mx = wave_max(pm);
    const float f = (pm == -INFINITY) ? 0.0f : __expf(pm - mx);
    const float l = wave_sum(pl * f);
    float o = 0.0f;
#pragma unroll
    for (int ch = 0; ch < FAST; ch++)
      if (ch < chunks) o += po[ch] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), ch));
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    out[((size_t)b * hq + head) * HD + tid] = (_Float16)(o * inv);
    return;
  }
  // maximum over all chunks
  float mx = -INFINITY;
  for (int ch = tid; ch < chunks; ch += 128) mx = fmaxf(mx, src[(size_t)ch * (HD + 2)]);
  mx = wave_max(mx);
  if ((tid & 63) == 0) red_m[tid >> 6] = mx;
  __syncthreads();
  mx = fmaxf(red_m[0], red_m[1]);
  // weights exp(m_ch - mx) and the normaliser
  float l = 0.0f;
  for (int ch = tid; ch < chunks; ch += 128) {
    const float *p = src + (size_t)ch * (HD + 2);
    const float f = (p[0] == -INFINITY) ? 0.0f : __expf(p[0] - mx);
    if (ch < CAP) wgt[ch] = f;
    l += p[1] * f;
  }
  l = wave_sum(l);
  if ((tid & 63) == 0) red_l[tid >> 6] = l;
  __syncthreads();
  l = red_l[0] + red_l[1];
  float o = 0.0f;
  const int fast = chunks < CAP ? chunks : CAP;
#pragma unroll 8
  for (int ch = 0; ch < fast; ch++) o += src[(size_t)ch * (HD + 2) + 2 + tid] * wgt[ch];
  for (int ch = CAP; ch < chunks; ch++) {
    const float *p = src + (size_t)ch * (HD + 2);
    const float f = (p[0] == -INFINITY) ? 0.0f : __expf(p[0] - mx);
    o += p[2 + tid] * f;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  out[((size_t)b * hq + head) * HD + tid] = (_Float16)(o * inv);
}

// ---- rotary embedding + cache append + attention partials in ONE launch (fp16 cache) ------------------------------
// Same arithmetic as rope_append_kernel -> attn_partial_kernel<false>, without the kernel boundary between them:
//   * every workgroup rotates the query heads of its kv head itself (one (i, i + 64) pair per thread, through LDS)
//     while its K / V loads are in flight; the rotated q is never written back (the workgroups of the other chunks
//     read the unrotated one at the same time), only the workgroup of chunk 0 leaves a copy in `qrot` for diagnostics;
//   * the workgroup whose chunk holds the current position rotates k, appends k and v to the cache and patches the
//     new row into the registers of the wave that owns the position (the loads issued up front saw the old bytes).
// attn_combine_kernel follows as a launch of its own.  (Merging the chunks in the same launch as well -- partials
// through agent-scope stores, an arrival counter per (batch row, kv head), the last workgroup merges -- computed the
// same values but was slower than the separate launch: 36.9 against 29.2 + 4.7 us at batch 16, context 2048; with an
// acquire-release counter, whose cache write-back every workgroup pays, 113 us.)
__global__ void __launch_bounds__(256) attn_fused_kernel(const _Float16 *__restrict__ qkv, _Float16 *kc, _Float16 *vc,
                                                         const int32_t *__restrict__ pos_ptr, int hq, int hkv, int max_ctx,
                                                         int max_chunks, float scale, float theta,
                                                         float *__restrict__ part, _Float16 *__restrict__ qrot) {
  constexpr int HD = 128;
  __shared__ __attribute__((aligned(16))) _Float16 q_lds[4][HD];
  __shared__ __attribute__((aligned(16))) _Float16 knew[HD], vnew[HD];
  __shared__ __attribute__((aligned(16))) _Float16 p_lds[ATT_WAVES][4][32];
  __shared__ float w_m[ATT_WAVES][4], w_l[ATT_WAVES][4];
  __shared__ float w_o[ATT_WAVES][4][HD];
  // chunk index slowest: the workgroups of the last, partly filled chunk (a quarter of the loads or less) are the
  // ones that run while the grid drains
  const int kvh = blockIdx.x, b = blockIdx.y, chunk = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int group = hq / hkv;
  const int pos = *pos_ptr;
  const int n_ctx = pos + 1;
  const int live_chunks = (n_ctx + ATT_CHUNK - 1) / ATT_CHUNK;
  if (chunk >= live_chunks) return;  // uniform in the workgroup, before any barrier
  const int p0 = chunk * ATT_CHUNK + wave * ATT_POS_PER_WAVE;
  const int row_elems = (hq + 2 * hkv) * HD;
  const bool wave_live = p0 < n_ctx;
  const bool owner = (pos / ATT_CHUNK) == chunk;  // this workgroup's positions include the current token

  // ---- K / V of this wave's 32 positions: requested before anything else ----
  const size_t k_off = (((size_t)b * hkv + kvh) * max_ctx + p0) * HD;
  const size_t v_off = ((((size_t)b * hkv + kvh) * (max_ctx / 8) + p0 / 8) * HD) * 8;
  half8_t kf[2][4], vf[8];
  if (wave_live) {
    const _Float16 *kbase = kc + k_off;
    const _Float16 *vbase = vc + v_off;
#pragma unroll
    for (int pb = 0; pb < 2; pb++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        kf[pb][j] = *reinterpret_cast<const half8_t *>(kbase + (size_t)(pb * 16 + r) * HD + 32 * c + 8 * j);
#pragma unroll
    // V arrives in whole lines that nothing reads again in this launch: streaming loads keep them from displacing the
    // K lines, which four requests share (K through streaming loads costs more than it saves: a line evicted between
    // two of its requests is fetched again)
    for (int t = 0; t < 8; t++)
      vf[t] = __builtin_nontemporal_load(reinterpret_cast<const half8_t *>(vbase + ((size_t)c * HD + t * 16 + r) * 8));
  }

  // ---- rotary embedding: thread (h = tid / 64, i = tid % 64) turns the pair (i, i + 64) of query head h ----
  {
    const int h = tid >> 6, i = tid & 63;
    const SinCos sc = rope_sincos(theta, i, HD, pos);
    const float sn = sc.sn, cs = sc.cs;
    if (h < group) {
      const int head = kvh * group + h;
      const _Float16 *src = qkv + (size_t)b * row_elems + (size_t)head * HD;
      const float x0 = (float)src[i], x1 = (float)src[i + HD / 2];
      _Float16 y0, y1;
      rope_pair(x0, x1, cs, sn, y0, y1);
      q_lds[h][i] = y0;
      q_lds[h][i + HD / 2] = y1;
      if (chunk == 0) {
        qrot[((size_t)b * hq + head) * HD + i] = y0;
        qrot[((size_t)b * hq + head) * HD + i + HD / 2] = y1;
      }
    }
    if (owner) {
      if (h == 0) {
        const _Float16 *src = qkv + (size_t)b * row_elems + (size_t)(hq + kvh) * HD;
        const float x0 = (float)src[i], x1 = (float)src[i + HD / 2];
        _Float16 y0, y1;
      rope_pair(x0, x1, cs, sn, y0, y1);
        knew[i] = y0;
        knew[i + HD / 2] = y1;
        _Float16 *dst = kc + (((size_t)b * hkv + kvh) * max_ctx + pos) * HD;
        dst[i] = y0;
        dst[i + HD / 2] = y1;
      } else if (h == 1 || h == 2) {
        const int dd = (h - 1) * 64 + i;
        const _Float16 v = qkv[(size_t)b * row_elems + (size_t)(hq + hkv + kvh) * HD + dd];
        vnew[dd] = v;
        vc[((((size_t)b * hkv + kvh) * (max_ctx / 8) + pos / 8) * HD + dd) * 8 + (pos & 7)] = v;
      }
    }
  }
  __syncthreads();

  float m_h = -INFINITY, l_h = 0.0f;
  float o_acc[8];
#pragma unroll
  for (int t = 0; t < 8; t++) o_acc[t] = 0.0f;

  if (wave_live) {
    half8_t qa[4];
    {
      const int h = r >> 2;
      const bool valid = ((r & 3) == 0) && h < group;
      const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 4; j++)
        qa[j] = valid ? *reinterpret_cast<const half8_t *>(&q_lds[h & 3][32 * c + 8 * j]) : z;
    }
    // the row appended in this launch: the loads above read whatever the cache held before
    const int rel = pos - p0;
    if (owner && rel >= 0 && rel < ATT_POS_PER_WAVE) {
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
        if (rel == pb * 16 + r) {
#pragma unroll
          for (int j = 0; j < 4; j++) kf[pb][j] = *reinterpret_cast<const half8_t *>(&knew[32 * c + 8 * j]);
        }
      const int e_new = rel - 8 * c;
      if (e_new >= 0 && e_new < 8) {
#pragma unroll
        for (int t = 0; t < 8; t++) {
          const _Float16 nv = vnew[t * 16 + r];
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (e == e_new) vf[t][e] = nv;
        }
      }
    }

    float s[2];
#pragma unroll
    for (int pb = 0; pb < 2; pb++) {
      float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 4; j++) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[j], kf[pb][j], d, 0, 0, 0);
      const int p = p0 + pb * 16 + r;
      s[pb] = (p < n_ctx) ? d[0] * scale : -INFINITY;
    }
    const float mx = row_max16(fmaxf(s[0], s[1]));  // over the 16 lanes of a group: DPP moves, no LDS round trips
    const float e0 = (s[0] == -INFINITY) ? 0.0f : __expf(s[0] - mx);
    const float e1 = (s[1] == -INFINITY) ? 0.0f : __expf(s[1] - mx);
    const float sum = row_sum16(e0 + e1);
    m_h = mx;
    l_h = sum;
    if (c < 4) {
      p_lds[wave][c][r] = (_Float16)e0;
      p_lds[wave][c][16 + r] = (_Float16)e1;
    }
    __builtin_amdgcn_wave_barrier();
    half8_t pa = {0, 0, 0, 0, 0, 0, 0, 0};
    if ((r & 3) == 0 && (r >> 2) < group) pa = *reinterpret_cast<const half8_t *>(&p_lds[wave][r >> 2][8 * c]);
#pragma unroll
    for (int t = 0; t < 8; t++) {
      half8_t vv = vf[t];
      if (p0 + 8 * c >= n_ctx) vv = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      else if (p0 + 8 * c + 8 > n_ctx) {
#pragma unroll
        for (int e = 0; e < 8; e++)
          if (p0 + 8 * c + e >= n_ctx) vv[e] = (_Float16)0.0f;
      }
      float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
      d = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vv, d, 0, 0, 0);
      o_acc[t] = d[0];
    }
  }

  // ---- merge the 4 waves, write this chunk's partial ----
  if (c < 4) {
    if (r == 0) {
      w_m[wave][c] = m_h;
      w_l[wave][c] = l_h;
    }
#pragma unroll
    for (int t = 0; t < 8; t++) w_o[wave][c][t * 16 + r] = o_acc[t];
  }
  __syncthreads();
  for (int idx = tid; idx < group * HD; idx += blockDim.x) {
    const int h = idx / HD, dd = idx % HD;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; w++) mx = fmaxf(mx, w_m[w][h]);
    float l = 0.0f, o = 0.0f;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; w++) {
      const float f = (w_m[w][h] == -INFINITY) ? 0.0f : __expf(w_m[w][h] - mx);
      l += w_l[w][h] * f;
      o += w_o[w][h][dd] * f;
    }
    const int head = kvh * group + h;
    float *dst = part + (((size_t)b * hq + head) * max_chunks + chunk) * (HD + 2);
    dst[2 + dd] = o;
    if (dd == 0) {
      dst[0] = mx;
      dst[1] = l;
    }
  }

}

// ---- greedy pick: last index among equal maxima; also records the token and advances the position ------
__global__ void __launch_bounds__(1024) argmax_kernel(const float *__restrict__ logits, int vocab,
                                                      int32_t *__restrict__ tokens, int32_t *__restrict__ history,
                                                      int32_t *__restrict__ step_ptr, int batch, int max_steps) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int b = blockIdx.x;
  const float *row = logits + (size_t)b * vocab;
  float best = -INFINITY;
  int bi = -1;
  // max_by keeps the later element unless the earlier one compares Greater; NaN compares Equal
  auto take = [&](float v, int i) {
    if (bi < 0 || !(best > v)) {
      best = v;
      bi = i;
    }
  };
  if ((vocab & 3) == 0) {
    // four consecutive values per thread and request, eight requests in flight, visited in index order
    const float4_t *row4 = reinterpret_cast<const float4_t *>(row);
    const int n4 = vocab >> 2;
    for (int i0 = 0; i0 < n4; i0 += 8 * (int)blockDim.x) {
      float4_t v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = i0 + u * (int)blockDim.x + (int)threadIdx.x;
        v[u] = i < n4 ? row4[i] : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = i0 + u * (int)blockDim.x + (int)threadIdx.x;
        if (i < n4) {
#pragma unroll
          for (int e = 0; e < 4; e++) take(v[u][e], 4 * i + e);
        }
      }
    }
  } else {
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) take(row[i], i);
  }
  // combine: higher value wins, equal values -> larger index; an unordered pair keeps the larger index too
  auto better = [](float va, int ia, float vb, int ib) {
    if (ia < 0) return false;
    if (ib < 0) return true;
    if (va > vb) return true;
    if (vb > va) return false;
    return ia > ib;
  };
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    if (better(ov, oi, best, bi)) {
      best = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = best;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (unsigned w = 1; w < (blockDim.x >> 6); w++)
      if (better(sv[w], si[w], best, bi)) {
        best = sv[w];
        bi = si[w];
      }
    tokens[b] = bi;
    const int step = *step_ptr;
    if (history && step < max_steps) history[(size_t)step * batch + b] = bi;
  }
}

// pos += 1, step += 1 (one thread) -- separate so every other kernel of the step sees one value
__global__ void advance_kernel(int32_t *pos_ptr, int32_t *step_ptr) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    *pos_ptr += 1;
    *step_ptr += 1;
  }
}

// deterministic pseudo-random fill of a cache region with ~N(0,1) fp16 (sum of uniforms), for benchmarks
__global__ void kv_random_fill_kernel(_Float16 *__restrict__ buf, size_t n, uint64_t seed) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    // four 16-bit uniforms -> approximately normal with unit variance
    float u = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; e++) u += (float)((z >> (16 * e)) & 0xFFFF) * (1.0f / 65536.0f);
    buf[i] = (_Float16)((u - 2.0f) * 1.7320508f);
  }
}

// ---- int8 cache: KvCache with KvDtype::I8 (crates/yscv-onnx/src/runner/kv_cache.rs:45-61) --------------------------------
// A row = the kv_dim = Hkv * 128 values one position adds to K (or V): scale = absmax / 127 (1.0 when absmax <=
// f32::EPSILON), q = clamp(round_half_away(v * (1 / scale)), -127, 127).
__device__ __forceinline__ float block_max_256(float v, float *red) {
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  return v;
}
__device__ __forceinline__ int8_t kv_quant_one(float v, float inv) {
#pragma clang fp contract(off)  // the product is rounded before the rounding rule looks at it, as in the reference
  const float x = v * inv;
  const float t = truncf(x);
  const float rr = (fabsf(x - t) >= 0.5f) ? t + copysignf(1.0f, x) : t;
  if (rr != rr) return 0;
  return (int8_t)(int)fminf(fmaxf(rr, -127.0f), 127.0f);
}
__device__ __forceinline__ void kv_row_scale(float amax, float *scale, float *inv) {
  *scale = (amax <= 1.1920929e-7f) ? 1.0f : __fdiv_rn(amax, 127.0f);
  *inv = __fdiv_rn(1.0f, *scale);
}

// RoPE on q (in place) and k, then per-row int8 quantisation of the rotated k row and of the v row of this position.
// One workgroup per batch row; dynamic LDS: 2 * Hkv * 128 floats.
__global__ void __launch_bounds__(256) rope_append_i8_kernel(_Float16 *__restrict__ qkv, const int32_t *__restrict__ pos_ptr,
                                                             int hq, int hkv, float theta, int max_ctx,
                                                             int8_t *__restrict__ kc, float *__restrict__ ks,
                                                             int8_t *__restrict__ vc, float *__restrict__ vs) {
  constexpr int HD = 128, HALF = 64;
  extern __shared__ float kv_lds[];
  __shared__ float red[4];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int pos = *pos_ptr;
  const int kv_dim = hkv * HD;
  float *kbuf = kv_lds, *vbuf = kv_lds + kv_dim;
  _Float16 *row = qkv + (size_t)b * (hq + 2 * hkv) * HD;
  float kmax = 0.0f, vmax = 0.0f;
  for (int idx = tid; idx < (hq + hkv) * HALF; idx += 256) {
    const int slot = idx / HALF, i = idx % HALF;
    const SinCos sc = rope_sincos(theta, i, HD, pos);
    const float sn = sc.sn, cs = sc.cs;
    _Float16 *src = row + (size_t)slot * HD;
    const float x0 = (float)src[i], x1 = (float)src[i + HALF];
    float y0, y1;
    rope_pair_f32(x0, x1, cs, sn, y0, y1);
    if (slot < hq) {
      src[i] = f16_of_f32(y0);
      src[i + HALF] = f16_of_f32(y1);
    } else {
      kbuf[(slot - hq) * HD + i] = y0;
      kbuf[(slot - hq) * HD + i + HALF] = y1;
      kmax = fmaxf(kmax, fmaxf(fabsf(y0), fabsf(y1)));
    }
  }
  for (int idx = tid; idx < kv_dim; idx += 256) {
    const float v = (float)row[(size_t)(hq + hkv) * HD + idx];
    vbuf[idx] = v;
    vmax = fmaxf(vmax, fabsf(v));
  }
  __syncthreads();
  kmax = block_max_256(kmax, red);
  vmax = block_max_256(vmax, red);
  float k_scale, k_inv, v_scale, v_inv;
  kv_row_scale(kmax, &k_scale, &k_inv);
  kv_row_scale(vmax, &v_scale, &v_inv);
  if (tid == 0) {
    ks[(size_t)b * max_ctx + pos] = k_scale;
    vs[(size_t)b * max_ctx + pos] = v_scale;
  }
  for (int idx = tid; idx < kv_dim; idx += 256) {
    const int kvh = idx / HD, i = idx % HD;
    kc[(((size_t)b * hkv + kvh) * max_ctx + pos) * HD + i] = kv_quant_one(kbuf[idx], k_inv);
    vc[((((size_t)b * hkv + kvh) * (max_ctx / 8) + pos / 8) * HD + i) * 8 + (pos & 7)] = kv_quant_one(vbuf[idx], v_inv);
  }
}

// Prompt pass on the int8 cache: the same rotation, row scales and quantisation for `rows` consecutive positions of
// batch row 0 (one workgroup per position), and what the cache now returns for each appended value (q * scale of its
// row, LayerStorage::dequantise_to_vec, crates/yscv-onnx/src/runner/kv_cache.rs:64-79) as fp16 in a scratch K / V
// pair laid out like the fp16 cache with t_ctx positions: the prompt's attention reads that pair.
__global__ void __launch_bounds__(256) prefill_rope_append_i8_kernel(_Float16 *__restrict__ qkv, int start_pos, int hq, int hkv,
                                                                     float theta, int max_ctx, int8_t *__restrict__ kc,
                                                                     float *__restrict__ ks, int8_t *__restrict__ vc,
                                                                     float *__restrict__ vs, int t_ctx, _Float16 *__restrict__ tk,
                                                                     _Float16 *__restrict__ tv) {
  constexpr int HD = 128, HALF = 64;
  extern __shared__ float kv_lds[];
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int pos = start_pos + (int)blockIdx.x;
  const int kv_dim = hkv * HD;
  float *kbuf = kv_lds, *vbuf = kv_lds + kv_dim;
  _Float16 *row = qkv + (size_t)blockIdx.x * (hq + 2 * hkv) * HD;
  float kmax = 0.0f, vmax = 0.0f;
  for (int idx = tid; idx < (hq + hkv) * HALF; idx += 256) {
    const int slot = idx / HALF, i = idx % HALF;
    const SinCos sc = rope_sincos(theta, i, HD, pos);
    _Float16 *src = row + (size_t)slot * HD;
    const float x0 = (float)src[i], x1 = (float)src[i + HALF];
    float y0, y1;
    rope_pair_f32(x0, x1, sc.cs, sc.sn, y0, y1);
    if (slot < hq) {
      src[i] = f16_of_f32(y0);
      src[i + HALF] = f16_of_f32(y1);
    } else {
      kbuf[(slot - hq) * HD + i] = y0;
      kbuf[(slot - hq) * HD + i + HALF] = y1;
      kmax = fmaxf(kmax, fmaxf(fabsf(y0), fabsf(y1)));
    }
  }
  for (int idx = tid; idx < kv_dim; idx += 256) {
    const float v = (float)row[(size_t)(hq + hkv) * HD + idx];
    vbuf[idx] = v;
    vmax = fmaxf(vmax, fabsf(v));
  }
  __syncthreads();
  kmax = block_max_256(kmax, red);
  vmax = block_max_256(vmax, red);
  float k_scale, k_inv, v_scale, v_inv;
  kv_row_scale(kmax, &k_scale, &k_inv);
  kv_row_scale(vmax, &v_scale, &v_inv);
  if (tid == 0) {
    ks[pos] = k_scale;
    vs[pos] = v_scale;
  }
  for (int idx = tid; idx < kv_dim; idx += 256) {
    const int kvh = idx / HD, i = idx % HD;
    const int8_t kq = kv_quant_one(kbuf[idx], k_inv), vq = kv_quant_one(vbuf[idx], v_inv);
    kc[((size_t)kvh * max_ctx + pos) * HD + i] = kq;
    vc[(((size_t)kvh * (max_ctx / 8) + pos / 8) * HD + i) * 8 + (pos & 7)] = vq;
    tk[((size_t)kvh * t_ctx + pos) * HD + i] = (_Float16)((float)kq * k_scale);
    tv[(((size_t)kvh * (t_ctx / 8) + pos / 8) * HD + i) * 8 + (pos & 7)] = (_Float16)((float)vq * v_scale);
  }
}

// positions 0 .. npos-1 of batch row 0 of the int8 cache, dequantised into the scratch pair of the prompt pass
__global__ void __launch_bounds__(256) kv_dequant_i8_kernel(const int8_t *__restrict__ kc, const float *__restrict__ ks,
                                                            const int8_t *__restrict__ vc, const float *__restrict__ vs, int hkv,
                                                            int max_ctx, int t_ctx, _Float16 *__restrict__ tk,
                                                            _Float16 *__restrict__ tv) {
  constexpr int HD = 128;
  const int pos = blockIdx.x;
  const float k_scale = ks[pos], v_scale = vs[pos];
  for (int idx = threadIdx.x; idx < hkv * HD; idx += 256) {
    const int kvh = idx / HD, i = idx % HD;
    tk[((size_t)kvh * t_ctx + pos) * HD + i] = (_Float16)((float)kc[((size_t)kvh * max_ctx + pos) * HD + i] * k_scale);
    tv[(((size_t)kvh * (t_ctx / 8) + pos / 8) * HD + i) * 8 + (pos & 7)] =
        (_Float16)((float)vc[(((size_t)kvh * (max_ctx / 8) + pos / 8) * HD + i) * 8 + (pos & 7)] * v_scale);
  }
}

// ---- rotary embedding + int8 cache append + attention partials in ONE launch (int8 cache) ---------------------------
// rope_append_i8_kernel -> attn_partial_kernel<true> without the kernel boundary, as attn_fused_kernel does it for the
// fp16 cache.  The scale of an int8 row spans all kv heads of the position, so each of the Hkv workgroups whose chunk
// holds the current position rotates the whole k row (Hkv * 64 pairs) and scans the whole v row to get the two scales
// (all of them write the same two values), then quantises and appends its own head's 128 + 128 values and patches
// them, with the new scales, into the registers of the wave that owns the position.  Dynamic LDS: Hkv * 128 floats.
__global__ void __launch_bounds__(256) attn_fused_i8_kernel(const _Float16 *__restrict__ qkv, int8_t *kc, float *ks, int8_t *vc,
                                                            float *vs, const int32_t *__restrict__ pos_ptr, int hq, int hkv,
                                                            int max_ctx, int max_chunks, float scale, float theta,
                                                            float *__restrict__ part, _Float16 *__restrict__ qrot) {
  constexpr int HD = 128;
  extern __shared__ float krow_lds[];  // owner only: the rotated k row of every kv head, f32
  __shared__ __attribute__((aligned(16))) _Float16 q_lds[4][HD];
  __shared__ __attribute__((aligned(16))) _Float16 knew[HD], vnew[HD];  // the appended int8 values, as fp16
  __shared__ float red[4], new_k_scale, new_v_scale;
  __shared__ __attribute__((aligned(16))) _Float16 p_lds[ATT_WAVES][4][32];
  __shared__ float w_m[ATT_WAVES][4], w_l[ATT_WAVES][4];
  __shared__ float w_o[ATT_WAVES][4][HD];
  // chunk index slowest: the workgroups of the last, partly filled chunk (a quarter of the loads or less) are the
  // ones that run while the grid drains
  const int kvh = blockIdx.x, b = blockIdx.y, chunk = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int group = hq / hkv;
  const int pos = *pos_ptr;
  const int n_ctx = pos + 1;
  const int live_chunks = (n_ctx + ATT_CHUNK - 1) / ATT_CHUNK;
  if (chunk >= live_chunks) return;  // uniform in the workgroup, before any barrier
  const int p0 = chunk * ATT_CHUNK + wave * ATT_POS_PER_WAVE;
  const int row_elems = (hq + 2 * hkv) * HD;
  const bool wave_live = p0 < n_ctx;
  const bool owner = (pos / ATT_CHUNK) == chunk;

  // ---- K / V bytes and scales of this wave's 32 positions: requested before anything else, converted further down ----
  const size_t k_off = (((size_t)b * hkv + kvh) * max_ctx + p0) * HD;
  const size_t v_off = ((((size_t)b * hkv + kvh) * (max_ctx / 8) + p0 / 8) * HD) * 8;
  int2_t kraw[2][4], vraw[8];
  float k_scale[2] = {1.0f, 1.0f}, v_scale[2] = {1.0f, 1.0f};  // of position p0 + 16 pb + r
  if (wave_live) {
#pragma unroll
    for (int pb = 0; pb < 2; pb++) {
      k_scale[pb] = ks[(size_t)b * max_ctx + p0 + pb * 16 + r];
      v_scale[pb] = vs[(size_t)b * max_ctx + p0 + pb * 16 + r];
#pragma unroll
      for (int j = 0; j < 4; j++)
        kraw[pb][j] = *reinterpret_cast<const int2_t *>(kc + k_off + (size_t)(pb * 16 + r) * HD + 32 * c + 8 * j);
    }
#pragma unroll
    for (int t = 0; t < 8; t++) vraw[t] = *reinterpret_cast<const int2_t *>(vc + v_off + ((size_t)c * HD + t * 16 + r) * 8);
  }

  // ---- rotary embedding of the query heads; the owners also rotate k, find the row scales and append ----
  {
    const int h = tid >> 6, i = tid & 63;
    const SinCos sc = rope_sincos(theta, i, HD, pos);
    const float sn = sc.sn, cs = sc.cs;
    if (h < group) {
      const int head = kvh * group + h;
      const _Float16 *src = qkv + (size_t)b * row_elems + (size_t)head * HD;
      const float x0 = (float)src[i], x1 = (float)src[i + HD / 2];
      _Float16 y0, y1;
      rope_pair(x0, x1, cs, sn, y0, y1);
      q_lds[h][i] = y0;
      q_lds[h][i + HD / 2] = y1;
      if (chunk == 0) {
        qrot[((size_t)b * hq + head) * HD + i] = y0;
        qrot[((size_t)b * hq + head) * HD + i + HD / 2] = y1;
      }
    }
    if (owner) {
      const _Float16 *row = qkv + (size_t)b * row_elems;
      float kmax = 0.0f, vmax = 0.0f;
      for (int slot = h; slot < hkv; slot += 4) {  // pair i of kv head `slot`: the angle is this thread's
        const _Float16 *src = row + (size_t)(hq + slot) * HD;
        const float x0 = (float)src[i], x1 = (float)src[i + HD / 2];
        float y0, y1;
        rope_pair_f32(x0, x1, cs, sn, y0, y1);
        krow_lds[slot * HD + i] = y0;
        krow_lds[slot * HD + i + HD / 2] = y1;
        kmax = fmaxf(kmax, fmaxf(fabsf(y0), fabsf(y1)));
      }
      for (int idx = tid; idx < hkv * HD; idx += 256) vmax = fmaxf(vmax, fabsf((float)row[(size_t)(hq + hkv) * HD + idx]));
      kmax = block_max_256(kmax, red);
      vmax = block_max_256(vmax, red);
      float ksc, kinv, vsc, vinv;
      kv_row_scale(kmax, &ksc, &kinv);
      kv_row_scale(vmax, &vsc, &vinv);
      if (tid == 0) {
        ks[(size_t)b * max_ctx + pos] = ksc;
        vs[(size_t)b * max_ctx + pos] = vsc;
        new_k_scale = ksc;
        new_v_scale = vsc;
      }
      if (tid < HD) {
        const int8_t q8 = kv_quant_one(krow_lds[kvh * HD + tid], kinv);
        kc[(((size_t)b * hkv + kvh) * max_ctx + pos) * HD + tid] = q8;
        knew[tid] = (_Float16)(float)q8;
      } else {
        const int dd = tid - HD;
        const int8_t q8 = kv_quant_one((float)row[(size_t)(hq + hkv + kvh) * HD + dd], vinv);
        vc[((((size_t)b * hkv + kvh) * (max_ctx / 8) + pos / 8) * HD + dd) * 8 + (pos & 7)] = q8;
        vnew[dd] = (_Float16)(float)q8;
      }
    }
  }
  __syncthreads();

  float m_h = -INFINITY, l_h = 0.0f;
  float o_acc[8];
#pragma unroll
  for (int t = 0; t < 8; t++) o_acc[t] = 0.0f;

  if (wave_live) {
    half8_t qa[4];
    {
      const int h = r >> 2;
      const bool valid = ((r & 3) == 0) && h < group;
      const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 4; j++) qa[j] = valid ? *reinterpret_cast<const half8_t *>(&q_lds[h & 3][32 * c + 8 * j]) : z;
    }
    // int8 values are exact in fp16: the K scale multiplies the finished score, the V scale the softmax weight
    // (V is converted after the scores, so that the bytes and the fp16 values of both are never live together)
    half8_t kf[2][4];
#pragma unroll
    for (int pb = 0; pb < 2; pb++)
#pragma unroll
      for (int j = 0; j < 4; j++) kf[pb][j] = i8x8_to_half8(kraw[pb][j]);
    // the row appended in this launch: the loads above read whatever the cache held before
    const int rel = pos - p0;
    const bool patch = owner && rel >= 0 && rel < ATT_POS_PER_WAVE;
    if (patch) {
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
        if (rel == pb * 16 + r) {
          k_scale[pb] = new_k_scale;
          v_scale[pb] = new_v_scale;
#pragma unroll
          for (int j = 0; j < 4; j++) kf[pb][j] = *reinterpret_cast<const half8_t *>(&knew[32 * c + 8 * j]);
        }
    }

    float s[2];
#pragma unroll
    for (int pb = 0; pb < 2; pb++) {
      float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 4; j++) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[j], kf[pb][j], d, 0, 0, 0);
      const int p = p0 + pb * 16 + r;
      s[pb] = (p < n_ctx) ? d[0] * scale * k_scale[pb] : -INFINITY;
    }
    const float mx = row_max16(fmaxf(s[0], s[1]));  // over the 16 lanes of a group: DPP moves, no LDS round trips
    const float e0 = (s[0] == -INFINITY) ? 0.0f : __expf(s[0] - mx);
    const float e1 = (s[1] == -INFINITY) ? 0.0f : __expf(s[1] - mx);
    const float sum = row_sum16(e0 + e1);
    m_h = mx;
    l_h = sum;
    float vS_inv = 1.0f;
    const float vS = v_scale_pow2(v_scale[0], v_scale[1], p0 + r < n_ctx, p0 + 16 + r < n_ctx, &vS_inv);
    if (c < 4) {  // the V scale of the position rides on its weight (a dead position has weight 0 whatever its scale)
      p_lds[wave][c][r] = e0 == 0.0f ? (_Float16)0.0f : (_Float16)(e0 * (v_scale[0] * vS_inv));
      p_lds[wave][c][16 + r] = e1 == 0.0f ? (_Float16)0.0f : (_Float16)(e1 * (v_scale[1] * vS_inv));
    }
    __builtin_amdgcn_wave_barrier();
    half8_t vf[8];
#pragma unroll
    for (int t = 0; t < 8; t++) vf[t] = i8x8_to_half8(vraw[t]);
    if (patch) {
      const int e_new = rel - 8 * c;
      if (e_new >= 0 && e_new < 8) {
#pragma unroll
        for (int t = 0; t < 8; t++) {
          const _Float16 nv = vnew[t * 16 + r];
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (e == e_new) vf[t][e] = nv;
        }
      }
    }
    half8_t pa = {0, 0, 0, 0, 0, 0, 0, 0};
    if ((r & 3) == 0 && (r >> 2) < group) pa = *reinterpret_cast<const half8_t *>(&p_lds[wave][r >> 2][8 * c]);
#pragma unroll
    for (int t = 0; t < 8; t++) {
      half8_t vv = vf[t];
      if (p0 + 8 * c >= n_ctx) vv = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      else if (p0 + 8 * c + 8 > n_ctx) {
#pragma unroll
        for (int e = 0; e < 8; e++)
          if (p0 + 8 * c + e >= n_ctx) vv[e] = (_Float16)0.0f;
      }
      float4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
      d = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vv, d, 0, 0, 0);
      o_acc[t] = d[0] * vS;
    }
  }

  // ---- merge the 4 waves, write this chunk's partial ----
  if (c < 4) {
    if (r == 0) {
      w_m[wave][c] = m_h;
      w_l[wave][c] = l_h;
    }
#pragma unroll
    for (int t = 0; t < 8; t++) w_o[wave][c][t * 16 + r] = o_acc[t];
  }
  __syncthreads();
  for (int idx = tid; idx < group * HD; idx += blockDim.x) {
    const int h = idx / HD, dd = idx % HD;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; w++) mx = fmaxf(mx, w_m[w][h]);
    float l = 0.0f, o = 0.0f;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; w++) {
      const float f = (w_m[w][h] == -INFINITY) ? 0.0f : __expf(w_m[w][h] - mx);
      l += w_l[w][h] * f;
      o += w_o[w][h][dd] * f;
    }
    const int head = kvh * group + h;
    float *dst = part + (((size_t)b * hq + head) * max_chunks + chunk) * (HD + 2);
    dst[2 + dd] = o;
    if (dd == 0) {
      dst[0] = mx;
      dst[1] = l;
    }
  }
}

// natural [batch][pos][kv_head][d] fp16 (host order) -> int8 cache rows; one workgroup per (position, batch row)
__global__ void __launch_bounds__(256) kv_relayout_i8_kernel(const _Float16 *__restrict__ k_nat, const _Float16 *__restrict__ v_nat,
                                                             int npos, int hkv, int max_ctx, int8_t *__restrict__ kc,
                                                             float *__restrict__ ks, int8_t *__restrict__ vc,
                                                             float *__restrict__ vs) {
  constexpr int HD = 128;
  __shared__ float red[4];
  const int pos = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int kv_dim = hkv * HD;
  const _Float16 *kr = k_nat + ((size_t)b * npos + pos) * kv_dim, *vr = v_nat + ((size_t)b * npos + pos) * kv_dim;
  float kmax = 0.0f, vmax = 0.0f;
  for (int idx = tid; idx < kv_dim; idx += 256) {
    kmax = fmaxf(kmax, fabsf((float)kr[idx]));
    vmax = fmaxf(vmax, fabsf((float)vr[idx]));
  }
  kmax = block_max_256(kmax, red);
  vmax = block_max_256(vmax, red);
  float k_scale, k_inv, v_scale, v_inv;
  kv_row_scale(kmax, &k_scale, &k_inv);
  kv_row_scale(vmax, &v_scale, &v_inv);
  if (tid == 0) {
    ks[(size_t)b * max_ctx + pos] = k_scale;
    vs[(size_t)b * max_ctx + pos] = v_scale;
  }
  for (int idx = tid; idx < kv_dim; idx += 256) {
    const int kvh = idx / HD, i = idx % HD;
    kc[(((size_t)b * hkv + kvh) * max_ctx + pos) * HD + i] = kv_quant_one((float)kr[idx], k_inv);
    vc[((((size_t)b * hkv + kvh) * (max_ctx / 8) + pos / 8) * HD + i) * 8 + (pos & 7)] = kv_quant_one((float)vr[idx], v_inv);
  }
}

// benchmark fill of an int8 cache: uniform bytes in [-127, 127] and one constant scale, so values span about +-3.5
__global__ void kv_random_fill_i8_kernel(int8_t *__restrict__ buf, size_t n, uint64_t seed) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    buf[i] = (int8_t)((int)(z % 255u) - 127);
  }
}
__global__ void fill_const_f32_kernel(float *p, size_t n, float v) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

// ---- launchers -------------------------------------------------------------------------------------------
int32_t launch_embed(const int32_t *tokens, const _Float16 *table, int batch, int d, int vocab, float *h,
                     hipStream_t s) {
  hipLaunchKernelGGL(embed_kernel, dim3(batch), dim3(256), 0, s, tokens, table, d, vocab, h);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_embed_norm(const int32_t *tokens, const _Float16 *table, int batch, int d, int vocab, float eps, float *h,
                          const float *gamma, _Float16 *xg, float *ss_out, int ss_stride, float *pre, hipStream_t s) {
  if (d > 4096 || d % 8 != 0) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "embedding with a folded norm: rows of at most 4096 values, a multiple of 8");
  hipLaunchKernelGGL(embed_norm_kernel, dim3(batch), dim3(256), 0, s, tokens, table, d, vocab, eps, h, gamma, xg, ss_out, ss_stride,
                     pre);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_rmsnorm(const float *h, const float *gamma, int batch, int d, float eps, _Float16 *out,
                       hipStream_t s) {
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(batch), dim3(256), 0, s, h, gamma, d, eps, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_rope_append(_Float16 *qkv, const int32_t *pos_ptr, int batch, int hq, int hkv, int hd, float theta,
                           int max_ctx, _Float16 *kc, _Float16 *vc, hipStream_t s) {
  hipLaunchKernelGGL(rope_append_kernel, dim3(hq + 2 * hkv, batch), dim3(64), 0, s, qkv, pos_ptr, hq, hkv, hd,
                     theta, max_ctx, kc, vc);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_kv_relayout(const _Float16 *k_nat, const _Float16 *v_nat, int batch, int npos, int hkv, int hd,
                           int max_ctx, _Float16 *kc, _Float16 *vc, hipStream_t s) {
  size_t total = (size_t)batch * npos * hkv * hd;
  size_t blocks = ceil_div(total, (size_t)256);
  if (blocks > 65535) blocks = 65535;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(kv_relayout_kernel, dim3((unsigned)blocks), dim3(256), 0, s, k_nat, v_nat, batch, npos, hkv,
                     hd, max_ctx, kc, vc);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_attention(const _Float16 *qkv, const _Float16 *kc, const _Float16 *vc, const int32_t *pos_ptr,
                         int batch, int hq, int hkv, int hd, int max_ctx, float *part, _Float16 *out,
                         hipStream_t s) {
  if (hd != 128) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel is built for head_dim 128, got %d", hd);
  if (hq % hkv != 0 || hq / hkv > 4)
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel handles 1..4 query heads per kv head");
  const int max_chunks = max_ctx / ATT_CHUNK;
  const float scale = 1.0f / sqrtf((float)hd);
  hipLaunchKernelGGL(attn_partial_kernel<false>, dim3(max_chunks, hkv, batch), dim3(256), 0, s, qkv, kc, vc, nullptr, nullptr,
                     pos_ptr, hq, hkv, max_ctx, max_chunks, scale, part);
  YSCV_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(attn_combine_kernel, dim3(hq, batch), dim3(128), 0, s, part, pos_ptr, hq, max_chunks, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_attention_fused(const _Float16 *qkv, _Float16 *kc, _Float16 *vc, const int32_t *pos_ptr, int batch, int hq,
                               int hkv, int hd, float theta, int max_ctx, float *part, _Float16 *qrot, _Float16 *out,
                               hipStream_t s) {
  if (hd != 128) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel is built for head_dim 128, got %d", hd);
  if (hq % hkv != 0 || hq / hkv > 4)
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel handles 1..4 query heads per kv head");
  const int max_chunks = max_ctx / ATT_CHUNK;
  const float scale = 1.0f / sqrtf((float)hd);
  hipLaunchKernelGGL(attn_fused_kernel, dim3(hkv, batch, max_chunks), dim3(256), 0, s, qkv, kc, vc, pos_ptr, hq, hkv, max_ctx,
                     max_chunks, scale, theta, part, qrot);
  YSCV_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(attn_combine_kernel, dim3(hq, batch), dim3(128), 0, s, part, pos_ptr, hq, max_chunks, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_attention_i8(const _Float16 *qkv, const int8_t *kc, const float *ks, const int8_t *vc, const float *vs,
                            const int32_t *pos_ptr, int batch, int hq, int hkv, int hd, int max_ctx, float *part,
                            _Float16 *out, hipStream_t s) {
  if (hd != 128) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel is built for head_dim 128, got %d", hd);
  if (hq % hkv != 0 || hq / hkv > 4)
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel handles 1..4 query heads per kv head");
  const int max_chunks = max_ctx / ATT_CHUNK;
  const float scale = 1.0f / sqrtf((float)hd);
  hipLaunchKernelGGL(attn_partial_kernel<true>, dim3(max_chunks, hkv, batch), dim3(256), 0, s, qkv, kc, vc, ks, vs, pos_ptr, hq,
                     hkv, max_ctx, max_chunks, scale, part);
  YSCV_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(attn_combine_kernel, dim3(hq, batch), dim3(128), 0, s, part, pos_ptr, hq, max_chunks, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_attention_fused_i8(const _Float16 *qkv, int8_t *kc, float *ks, int8_t *vc, float *vs, const int32_t *pos_ptr,
                                  int batch, int hq, int hkv, int hd, float theta, int max_ctx, float *part, _Float16 *qrot,
                                  _Float16 *out, hipStream_t s) {
  if (hd != 128) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel is built for head_dim 128, got %d", hd);
  if (hq % hkv != 0 || hq / hkv > 4)
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "attention kernel handles 1..4 query heads per kv head");
  const size_t lds = (size_t)hkv * hd * sizeof(float);
  if (lds > 32 * 1024) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "int8 cache append: too many kv heads (%d)", hkv);
  const int max_chunks = max_ctx / ATT_CHUNK;
  const float scale = 1.0f / sqrtf((float)hd);
  hipLaunchKernelGGL(attn_fused_i8_kernel, dim3(hkv, batch, max_chunks), dim3(256), lds, s, qkv, kc, ks, vc, vs, pos_ptr, hq, hkv,
                     max_ctx, max_chunks, scale, theta, part, qrot);
  YSCV_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(attn_combine_kernel, dim3(hq, batch), dim3(128), 0, s, part, pos_ptr, hq, max_chunks, out);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_rope_append_i8(_Float16 *qkv, const int32_t *pos_ptr, int batch, int hq, int hkv, int hd, float theta,
                              int max_ctx, int8_t *kc, float *ks, int8_t *vc, float *vs, hipStream_t s) {
  if (hd != 128) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "int8 cache append is built for head_dim 128, got %d", hd);
  const size_t lds = (size_t)2 * hkv * hd * sizeof(float);
  if (lds > 48 * 1024) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "int8 cache append: too many kv heads (%d)", hkv);
  hipLaunchKernelGGL(rope_append_i8_kernel, dim3(batch), dim3(256), lds, s, qkv, pos_ptr, hq, hkv, theta, max_ctx, kc, ks, vc, vs);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_prefill_rope_append_i8(_Float16 *qkv, int rows, int start_pos, int hq, int hkv, int hd, float theta, int max_ctx,
                                      int8_t *kc, float *ks, int8_t *vc, float *vs, int t_ctx, _Float16 *tk, _Float16 *tv,
                                      hipStream_t s) {
  if (hd != 128) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "int8 cache append is built for head_dim 128, got %d", hd);
  const size_t lds = (size_t)2 * hkv * hd * sizeof(float);
  if (lds > 48 * 1024) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "int8 cache append: too many kv heads (%d)", hkv);
  if (t_ctx % 8 != 0 || t_ctx < start_pos + rows) return set_error(YSCV_HIP_ERR_INVALID_ARG, "scratch K / V: %d positions", t_ctx);
  if (start_pos > 0) {
    hipLaunchKernelGGL(kv_dequant_i8_kernel, dim3(start_pos), dim3(256), 0, s, kc, ks, vc, vs, hkv, max_ctx, t_ctx, tk, tv);
    YSCV_HIP_TRY(hipGetLastError());
  }
  hipLaunchKernelGGL(prefill_rope_append_i8_kernel, dim3(rows), dim3(256), lds, s, qkv, start_pos, hq, hkv, theta, max_ctx, kc, ks,
                     vc, vs, t_ctx, tk, tv);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_kv_relayout_i8(const _Float16 *k_nat, const _Float16 *v_nat, int batch, int npos, int hkv, int hd, int max_ctx,
                              int8_t *kc, float *ks, int8_t *vc, float *vs, hipStream_t s) {
  if (hd != 128) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "int8 cache is built for head_dim 128, got %d", hd);
  hipLaunchKernelGGL(kv_relayout_i8_kernel, dim3(npos, batch), dim3(256), 0, s, k_nat, v_nat, npos, hkv, max_ctx, kc, ks, vc, vs);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_kv_random_fill_i8(int8_t *buf, size_t n, float *scales, size_t n_scales, float scale, uint64_t seed, hipStream_t s) {
  size_t blocks = ceil_div(n, (size_t)256);
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(kv_random_fill_i8_kernel, dim3((unsigned)blocks), dim3(256), 0, s, buf, n, seed);
  YSCV_HIP_TRY(hipGetLastError());
  size_t sb = ceil_div(n_scales, (size_t)256);
  hipLaunchKernelGGL(fill_const_f32_kernel, dim3((unsigned)(sb > 65535 ? 65535 : sb)), dim3(256), 0, s, scales, n_scales, scale);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_argmax(const float *logits, int batch, int vocab, int32_t *tokens, int32_t *history,
                      int32_t *step_ptr, int max_steps, hipStream_t s) {
  hipLaunchKernelGGL(argmax_kernel, dim3(batch), dim3(1024), 0, s, logits, vocab, tokens, history, step_ptr, batch,
                     max_steps);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_advance(int32_t *pos_ptr, int32_t *step_ptr, hipStream_t s) {
  hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(64), 0, s, pos_ptr, step_ptr);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

int32_t launch_kv_random_fill(_Float16 *buf, size_t n, uint64_t seed, hipStream_t s) {
  size_t blocks = ceil_div(n, (size_t)256);
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(kv_random_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, s, buf, n, seed);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

}  // namespace yscv
