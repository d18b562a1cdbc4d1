// Internal interface between the C ABI (api.hip) and the kernel files.
#pragma once

#include "common.hpp"

// Device-resident packed-int4 weight (see int4_common.hpp for the tiled layout).
struct yscv_hip_int4_weight {
  size_t n = 0, k = 0, g = 0;
  int scale_dtype = YSCV_HIP_F32;  // storage type of the scales on the device
  bool has_zp = false;             // false: every zero point is 8
  bool tiled = false;              // fast layout built (g in {32,64} or g % 128 == 0)
  int gm = 0;                      // group mode of the tiled layout
  size_t nt = 0, kt = 0;           // tile counts: ceil(n/16), ceil(k/128)
  size_t ktp = 0;                  // stored 128-k tiles per 16-row block: kt rounded up to 4 (zero tiles)
  size_t chunks = 0;               // scale chunks per n-tile
  uint8_t *tiles = nullptr;        // [nt][ktp][1 KiB]
  void *tscales = nullptr;         // [nt][chunks][16][spt]
  uint8_t *tzps = nullptr;         // same shape, one byte each; null when !has_zp
  // generic layout, kept only when the tiled one cannot be built
  uint8_t *raw = nullptr;    // [n][k/2], unsigned nibbles, natural order
  void *rscales = nullptr;   // [n][k/g]
  uint8_t *rzps = nullptr;   // [n][k/g] bytes; null when !has_zp
  size_t device_bytes = 0;
};

// Device-resident int8 B matrix: transposed [n][k] fragments for the MFMA kernel + column sums.
struct yscv_hip_i8_weight {
  size_t k = 0, n = 0;
  size_t kp = 0, np = 0;        // padded extents (k to 64, n to 16)
  int8_t *frag = nullptr;       // [np/16][kp/64][64 lanes][16 B]
  int32_t *col_sum = nullptr;   // [np], sum over k of b[k][j]
  size_t device_bytes = 0;
};

namespace yscv {

// ---- int4 ------------------------------------------------------------------------
// raw_in: device copy of the caller's [n][k/2] bytes in its own nibble format.
int32_t launch_int4_retile(const uint8_t *raw_in, int nibble_format, size_t n, size_t k,
                           size_t nt, size_t kt, uint8_t *tiles, hipStream_t s);
// scales_in [n][k/g] (f32 or f16) -> [nt][chunks][16][spt], same element type; zps likewise from
// one byte per group.  Padded entries get scale 0 / zp 8.
int32_t launch_int4_retile_scales(const void *scales_in, int scale_dtype, const uint8_t *zps_in,
                                  size_t n, size_t k, size_t g, int gm, size_t nt, size_t chunks,
                                  void *tscales, uint8_t *tzps, hipStream_t s);
// unpack packed uint4 zero points [n][ceil(G/2)] -> one byte per group [n][G]
int32_t launch_unpack_zps(const uint8_t *zps_packed, size_t n, size_t groups, uint8_t *out,
                          hipStream_t s);
// signed nibbles -> unsigned (byte ^ 0x88), natural order (generic layout)
int32_t launch_xor88(uint8_t *buf, size_t bytes, hipStream_t s);

// x [m][k] (f32/f16/bf16) -> fp16 hi (and lo when split == 2) [m][k_pad], plus the
// power-of-two factor each row was divided by.
int32_t launch_x_prep(const void *x, int x_dtype, size_t m, size_t k, size_t k_pad, int split,
                      _Float16 *xh, _Float16 *xl, float *row_scale, hipStream_t s);

// epilogues of the skinny kernel
enum : int { EPI_STORE = 0, EPI_ADD_F32 = 1, EPI_SWIGLU = 2 };

// RMSNorm folded into the projections on either side of it (decode loop).  The kernel that updates the residual
// stream h (EPI_ADD_F32) also writes what the norm's consumer needs: xg = fp16(h_new * gamma * pre[row]) and, per row,
// partial sums of h_new^2 over fixed column blocks.  pre[row] is a power of two near 1 / (4 rms) of the row as the
// norm BEFORE this update saw it (the kernel that consumed that norm leaves it behind; the embedding lookup works
// it out from its own row): an unnormalised row would otherwise leave fp16's range at either end, and a power of two
// leaves the rounding what it is.  A row may grow 2^18 / (its largest |value| / rms * gamma) fold within one update
// before an element saturates at fp16's maximum, and shrink 2^12 fold before its typical element loses precision.
// The projection that consumes xg works out inv = 1 / (pre * sqrt(sum / d + eps)) per row from the partials and
// applies it to its f32 sums: the same product as RMSNorm followed by the projection, with the fp16 rounding taken
// before the row factor instead of after it.
struct NormFold {
  // producer side (with EPI_ADD_F32): all null when the call does not feed a norm
  const float *gamma_next = nullptr;  // [n]
  const float *pre = nullptr;         // [m] power of two per row
  _Float16 *xg = nullptr;             // [m][n]
  float *ss_out = nullptr;            // [m][ss_out_stride]; the call reports how many partials per row it wrote
  int ss_out_stride = 0;
  int *ss_out_count = nullptr;        // host
  // consumer side: null when the activations are already normalised
  const float *ss_in = nullptr;       // [m][ss_in_stride]
  const float *pre_in = nullptr;      // [m] what the rows of xg were multiplied by
  float *pre_next = nullptr;          // [m] or null: receives the power of two for the update that follows this norm
  int ss_in_count = 0, ss_in_stride = 0;
  float inv_d = 0.0f, eps = 0.0f;
};

struct SkinnyPlan {
  int tpw;     // 128-k tiles per wave
  int waves;   // wavefronts per workgroup (= k-slices per workgroup)
  int ksg;     // grid-level k split (partials reduced by a second kernel when > 1)
  int grid_x;  // workgroups along n
  size_t partial_bytes;
};
SkinnyPlan plan_int4_skinny(const yscv_hip_int4_weight *w, size_t m, int split, int num_cus);
// xraw != null: raw activations with row stride k_pad, f32 when split == 2 and bf16 when split == 1; the kernel
// normalises (and for f32 splits) them itself and xh, xl, row_scale are not used
int32_t launch_int4_skinny(const yscv_hip_int4_weight *w, const SkinnyPlan &plan, const _Float16 *xh,
                           const _Float16 *xl, const void *xraw, const float *row_scale, size_t k_pad, int split,
                           void *y, int y_dtype, size_t m, float *partial, int epi, hipStream_t s,
                           const NormFold *nf = nullptr);
int32_t launch_int4_generic(const yscv_hip_int4_weight *w, const void *x, int x_dtype, void *y,
                            int y_dtype, size_t m, hipStream_t s);
int32_t launch_int4_gemm(const yscv_hip_int4_weight *w, const _Float16 *xh, const _Float16 *xl,
                         const float *row_scale, size_t k_pad, int split, void *y, int y_dtype,
                         size_t m, hipStream_t s, int epi = EPI_STORE, float *partial = nullptr, size_t partial_bytes = 0);

// LDS-ring GEMM for fp16-prepared activations (split == 1)
bool int4_gemm_ring_eligible(const yscv_hip_int4_weight *w, const _Float16 *xh, const void *y, int y_dtype, int split, size_t m,
                             size_t k_pad);
// epi: EPI_STORE; EPI_ADD_F32 (y f32 [m][n], y += product); EPI_SWIGLU (weight rows 2i / 2i+1 = gate_i / up_i,
// y [m][n / 2] = silu(gate) * up)
// partial: optional scratch of int4_gemm_ring_partial_bytes() bytes (16-byte aligned).  With it, a shape whose tiles
// cover at most half the CUs is also cut along k (f32 partial products, added in a fixed order by a second kernel);
// without it the launch runs unsplit.
int32_t launch_int4_gemm_ring(const yscv_hip_int4_weight *w, const _Float16 *xh, const float *row_scale, size_t k_pad,
                              void *y, int y_dtype, size_t m, hipStream_t s, int epi = EPI_STORE, float *partial = nullptr,
                              size_t partial_bytes = 0);
size_t int4_gemm_ring_partial_bytes(const yscv_hip_int4_weight *w, size_t m, int num_cus);

// 17 .. 32 rows (int4_mid.hip): K split over the waves with all rows' activations in registers, the weights streamed
// once.  With K > 4096 K is also cut into parts over workgroups whose f32 partial sums need
// int4_mid_partial_bytes() of scratch; the kernel is used where that stays within kMidPartialCap.
constexpr size_t kMidPartialCap = (size_t)16 << 20;
size_t int4_mid_partial_bytes(const yscv_hip_int4_weight *w, size_t m);
bool int4_mid_eligible(const yscv_hip_int4_weight *w, const _Float16 *xh, const void *y, int y_dtype, int split, size_t m,
                       size_t k_pad, size_t max_partial_bytes);
int32_t launch_int4_mid(const yscv_hip_int4_weight *w, const _Float16 *xh, const float *row_scale, size_t k_pad, void *y,
                        int y_dtype, size_t m, hipStream_t s, int epi, float *partial, size_t partial_bytes);

// Whole int4 call (activation preparation + kernel) with caller-provided scratch; ws may be null.
int32_t int4_workspace_bytes(const yscv_hip_int4_weight *w, size_t m, int x_dtype, int force, size_t *bytes);
int32_t int4_run_ws(const yscv_hip_int4_weight *w, const void *x, int x_dtype, void *y, int y_dtype, size_t m,
                    int force, int epi, void *ws, size_t ws_bytes, hipStream_t s, const NormFold *nf = nullptr);

int32_t int4_create_from_device(const uint8_t *d_packed, const void *d_scales, int scale_dtype, int nibble_format,
                                size_t n, size_t k, size_t g, yscv_hip_int4_weight **out);

int32_t launch_pack_int4_symmetric(const float *w, size_t m_w, size_t k, size_t g, uint8_t *packed,
                                   float *scales, hipStream_t s);
int32_t launch_dequantize_int4(const uint8_t *packed, size_t n_bytes, float scale, int zp,
                               float *out, hipStream_t s);

// runtime counters: a call served by the tiled MFMA kernels / by the generic per-group kernel
void note_int4_fast();
void note_int4_fallback();

// ---- int8 --------------------------------------------------------------------------
int32_t launch_i8_pack_b(const int8_t *b_kn, size_t k, size_t n, size_t kp, size_t np,
                         int8_t *frag, int32_t *col_sum, hipStream_t s);
struct I8Epilogue {
  int mode;  // 0: int32 out, 1: requantize to bytes, 2: requantize, then (q - y_zp) * dq_scale as f32, 3: f32(int32) out,
             // 4: requantize, the quantised value kept as f32 (a NaN stays a NaN)
  const int32_t *corr;
  const float *composite_v;
  float composite;
  float y_zp;
  int round_mode;
  int lo, hi;
  float dq_scale;
  const float *a_zp_dev = nullptr;  // uint8 A only: its zero point as an f32 in device memory, used instead of a_zp
};
int32_t launch_i8_gemm(const void *a, int a_is_u8, int a_zp, const yscv_hip_i8_weight *b, size_t m,
                       void *out, const I8Epilogue &ep, hipStream_t s);

// ---- elementwise ---------------------------------------------------------------------
int32_t launch_quantize_linear_i8(const float *x, size_t len, float scale, float zp, int8_t *out,
                                  hipStream_t s);
int32_t launch_quantize_f32_to_int4(const float *x, size_t len, float scale, int zp, uint8_t *out, hipStream_t s);
int32_t launch_requant(const int32_t *acc, size_t len, size_t c, const int32_t *corr,
                       const float *composite_v, float composite, float y_zp, int round_mode,
                       int lo, int hi, int relu, void *out, hipStream_t s);
int32_t launch_dynamic_quantize_linear(const float *x, size_t len, uint8_t *y, float *scale_zp,
                                       hipStream_t s);

int32_t launch_kv_i8_quantize_rows(const float *src, size_t rows, size_t kv_dim, int8_t *data, float *scales, hipStream_t s);
int32_t launch_kv_i8_dequantize_rows(const int8_t *data, const float *scales, size_t rows, size_t kv_dim, float *out,
                                     hipStream_t s);

}  // namespace yscv
