// Launchers of the decode-step glue kernels (decoder_kernels.hip), used by decoder.hip.
#pragma once

#include "common.hpp"

namespace yscv {

int32_t launch_embed(const int32_t *tokens, const _Float16 *table, int batch, int d, int vocab, float *h,
                     hipStream_t s);
// embedding lookup + the first norm in its folded form (NormFold in kernels.hpp): one partial sum of squares and the
// power-of-two scale of xg per row
int32_t launch_embed_norm(const int32_t *tokens, const _Float16 *table, int batch, int d, int vocab, float eps, float *h,
                          const float *gamma, _Float16 *xg, float *ss_out, int ss_stride, float *pre, hipStream_t s);
int32_t launch_rmsnorm(const float *h, const float *gamma, int batch, int d, float eps, _Float16 *out,
                       hipStream_t s);
int32_t launch_rope_append(_Float16 *qkv, const int32_t *pos_ptr, int batch, int hq, int hkv, int hd, float theta,
                           int max_ctx, _Float16 *kc, _Float16 *vc, hipStream_t s);
int32_t launch_kv_relayout(const _Float16 *k_nat, const _Float16 *v_nat, int batch, int npos, int hkv, int hd,
                           int max_ctx, _Float16 *kc, _Float16 *vc, hipStream_t s);
int32_t launch_attention(const _Float16 *qkv, const _Float16 *kc, const _Float16 *vc, const int32_t *pos_ptr,
                         int batch, int hq, int hkv, int hd, int max_ctx, float *part, _Float16 *out,
                         hipStream_t s);
// rope_append fused into the attention partials, then the merge (fp16 cache): `qrot` receives the rotated query heads
// [batch][hq * 128] (diagnostics; qkv itself keeps the unrotated q)
int32_t launch_attention_fused(const _Float16 *qkv, _Float16 *kc, _Float16 *vc, const int32_t *pos_ptr, int batch, int hq,
                               int hkv, int hd, float theta, int max_ctx, float *part, _Float16 *qrot, _Float16 *out,
                               hipStream_t s);
// int8 cache (KvCache with KvDtype::I8): K int8 [batch][kv_head][max_ctx][128], V int8 [batch][kv_head][max_ctx/8][128][8],
// one f32 scale per (batch row, position) for each of them
int32_t launch_rope_append_i8(_Float16 *qkv, const int32_t *pos_ptr, int batch, int hq, int hkv, int hd, float theta,
                              int max_ctx, int8_t *kc, float *ks, int8_t *vc, float *vs, hipStream_t s);
// prompt pass: positions start_pos .. start_pos + rows - 1 of batch row 0 rotated, quantised and appended; tk / tv
// (fp16, laid out like the fp16 cache with t_ctx positions) receive what the int8 cache returns for positions
// 0 .. start_pos + rows - 1
int32_t launch_prefill_rope_append_i8(_Float16 *qkv, int rows, int start_pos, int hq, int hkv, int hd, float theta, int max_ctx,
                                      int8_t *kc, float *ks, int8_t *vc, float *vs, int t_ctx, _Float16 *tk, _Float16 *tv,
                                      hipStream_t s);
int32_t launch_kv_relayout_i8(const _Float16 *k_nat, const _Float16 *v_nat, int batch, int npos, int hkv, int hd, int max_ctx,
                              int8_t *kc, float *ks, int8_t *vc, float *vs, hipStream_t s);
int32_t launch_attention_i8(const _Float16 *qkv, const int8_t *kc, const float *ks, const int8_t *vc, const float *vs,
                            const int32_t *pos_ptr, int batch, int hq, int hkv, int hd, int max_ctx, float *part,
                            _Float16 *out, hipStream_t s);
// rope_append_i8 fused into the attention partials, then the merge (int8 cache); `qrot` as in launch_attention_fused
int32_t launch_attention_fused_i8(const _Float16 *qkv, int8_t *kc, float *ks, int8_t *vc, float *vs, const int32_t *pos_ptr,
                                  int batch, int hq, int hkv, int hd, float theta, int max_ctx, float *part, _Float16 *qrot,
                                  _Float16 *out, hipStream_t s);
int32_t launch_kv_random_fill_i8(int8_t *buf, size_t n, float *scales, size_t n_scales, float scale, uint64_t seed, hipStream_t s);
int32_t launch_argmax(const float *logits, int batch, int vocab, int32_t *tokens, int32_t *history,
                      int32_t *step_ptr, int max_steps, hipStream_t s);
int32_t launch_advance(int32_t *pos_ptr, int32_t *step_ptr, hipStream_t s);
int32_t launch_kv_random_fill(_Float16 *buf, size_t n, uint64_t seed, hipStream_t s);

// glue_ops.hip: the general attention kernel over the fp16 cache (any head width that is a multiple of 32 up to 128,
// any number of query heads per kv head).  pos_ptr != null: `rows` batch rows at the position *pos_ptr (decode);
// pos_ptr == null: `rows` consecutive positions start_pos .. of batch row 0, causal (prompt pass).
// With `qrot` (decode mode only) the rotary embedding and the cache append of the new position happen inside the
// kernel: qkv holds q, k, v unrotated, kc / vc receive the new row (they are written), qrot the rotated query heads
// [rows][hq * hd]; without it qkv holds the rotated q and the cache already has the row.
int32_t launch_gqa_cache(const _Float16 *qkv, const _Float16 *kc, const _Float16 *vc, const int32_t *pos_ptr, int rows,
                         int start_pos, int hq, int hkv, int hd, int max_ctx, _Float16 *out, hipStream_t s,
                         float rope_theta = 0.0f, _Float16 *qrot = nullptr);
int32_t launch_prefill_rope_append(_Float16 *qkv, int rows, int start_pos, int hq, int hkv, int hd, float theta, int max_ctx,
                                   _Float16 *kc, _Float16 *vc, hipStream_t s);
int32_t launch_bias_add_f16(_Float16 *x, const _Float16 *bias, size_t rows, size_t n, hipStream_t s);

}  // namespace yscv
