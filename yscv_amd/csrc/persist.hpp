// Interface of the persistent (single-launch) batch-1 decode path: weight stream layout,
// exchange buffers and the launcher used by decoder.hip.
//
// Weight stream
// -------------
// The persistent kernel runs G workgroups, one per CU, each with PS_WAVES compute wavefronts.  For a projection
// W[n][k] (k a multiple of 1024) compute wave v of every workgroup owns the k range [v*k/4, (v+1)*k/4), and
// workgroup w owns the 8-row blocks w, w+G, w+2G, ...  A tile is 8 rows x 256 k = 1 KiB: lane
// L = 16*c + r of a wavefront holds four 32-bit words, word j = the eight weights
//     W[8*blk + (r & 7)][k0 + 32*(j + 4*(r >> 3)) + 8*c + 0..7]
// in the permuted nibble order of int4_common.hpp.  Two consecutive tiles (512 k, one A fragment)
// plus their scales form a record of 2304 bytes: [tile0 1024][tile1 1024][scales 256]; the last
// record of an odd tile count is [tile 1024][scales 256] = 1280 bytes.  The scale block holds, for
// tile t and lane-row r, four fp16 values at byte t*128 + r*8: the scales of row (r & 7), groups
// (k0 + 256*t)/32 + j + 4*(r >> 3), j = 0..3.
// Every wave has one contiguous stream holding its records in the order the kernel consumes them:
// layer 0 {qkv, o, gate/up, down}, layer 1 ..., lm_head; the streams of the compute waves of workgroup w
// sit back to back at wg_off[w].
#pragma once

#include <hip/hip_runtime.h>

#include "common.hpp"

namespace yscv {

constexpr int PS_WAVES = 4;   // compute waves per workgroup = k slices of every projection
constexpr int PS_REC_FULL = 2304;
constexpr int PS_REC_SINGLE = 1280;
constexpr int PERSIST_TRACE_SLOTS = 24;  // timestamps per (workgroup, layer) in builds with YSCV_PERSIST_TRACE
enum : int { PK_QKV = 0, PK_O = 1, PK_GU = 2, PK_DOWN = 3, PK_LM = 4, PK_COUNT = 5 };

struct PersistPhase {
  int n;       // output rows
  int k;       // input channels
  int ks;      // k per wave = k / PS_WAVES
  int tiles;   // 256-k tiles per wave and block = ks / 256
  int pairs;   // records per wave and block = ceil(tiles / 2)
  int frags;   // 512-k A fragments per wave = pairs
  int nb;      // 8-row blocks = n / 8
  int blk_bytes;  // stream bytes per wave and block
};

struct PersistModel {
  int n_layers, d_model, n_heads, n_kv_heads, d_ff, vocab, max_ctx;
  float theta, eps;
  int G;  // workgroups
  PersistPhase ph[PK_COUNT];
  // device data
  const uint8_t *stream;
  const uint64_t *wg_off;       // [G] byte offset of workgroup w's streams
  const uint32_t *wave_bytes;   // [G] stream bytes of one wave of workgroup w
  const float *gammas;          // [(2 * n_layers + 1)][d_model]: attn_l, ffn_l interleaved, final last
  const _Float16 *emb;          // [vocab][d_model]
  _Float16 *const *kc;          // [n_layers] K cache [batch][kv_head][max_ctx][128]
  _Float16 *const *vc;          // [n_layers] V cache [batch][kv_head][max_ctx/8][128][8]
  // exchange buffers (8-byte entries {payload, tag})
  unsigned long long *xn;       // input of qkv / lm_head: d_model values as fp16 pairs + [G] sum-of-squares entries
  unsigned long long *qkv;      // (n_heads + 2 n_kv_heads) * 64 fp16-pair entries, natural order
  unsigned long long *part;     // [n_heads][max_ctx/128][132] f32 entries: max, sum, o[128]
  unsigned long long *ao;       // attention output, fragment order for k = n_heads*128
  unsigned long long *xn2;      // input of gate/up + [G] sum-of-squares entries
  unsigned long long *act;      // input of down, fragment order for k = d_ff
  unsigned long long *arg;      // [G][2] per-workgroup best logit {value, index}
  // outputs / state
  float *logits;                // [vocab]
  int32_t *tokens;              // [1] current token (in: first token; out: last pick)
  int32_t *history;             // [max_steps]
  uint32_t *abort_flag;         // set when a bounded wait gave up
  unsigned long long *dbg_t;    // null, or [G][n_layers][PERSIST_TRACE_SLOTS] stage timestamps (builds with YSCV_PERSIST_TRACE)
};

// entries an exchange vector of k values occupies (padded to whole 512-k fragments per wave)
__host__ __device__ inline size_t persist_vec_entries(int k) {
  const int ks = k / PS_WAVES;
  const int frags = (ks + 511) / 512;
  return (size_t)PS_WAVES * frags * 256;
}

// true when the shape can run on the persistent path
bool persist_supported(const yscv_hip_decoder_config &c, int num_cus, const char **why);
void persist_fill_phases(const yscv_hip_decoder_config &c, int G, PersistModel *m);
// stream bytes of one wave of workgroup w, and the offset of (layer, kind) inside it
size_t persist_wave_bytes(const PersistModel &m, int w);
size_t persist_seq_offset(const PersistModel &m, int w, int layer, int kind);

// Pack one projection (device inputs: packed [n][k/2] unsigned nibbles in natural order, fp16 scales
// [n][k/32]) into the streams.  For PK_QKV the rows of the q and k heads are re-ordered so that the
// rotary pairs (i, i + 64) sit next to each other.
int32_t launch_persist_pack(const PersistModel &m, int layer, int kind, const uint8_t *packed_dev,
                            const _Float16 *scales_dev, uint8_t *stream, hipStream_t s);

// Run n_steps decode steps in one cooperative launch.  pos0 = cached positions before the first step,
// step0 = index of the first step in the token history, epoch0 = tag epoch of the first step.
int32_t launch_persist_decode(const PersistModel &m, int n_steps, int pos0, int step0, int max_steps,
                              uint32_t epoch0, hipStream_t s);

}  // namespace yscv
