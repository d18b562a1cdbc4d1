// Llama-style decoder resident on the GPU: the decode loop of the llm-bench harness
// (apps/llm-bench/src/main.rs:403-561: feed the last token plus the KV cache, take the greedy
// pick, repeat) with every projection running through the skinny int4 kernel.
// One decode step is a fixed sequence of kernel launches that reads the position from device
// memory, so the step is captured once into a HIP graph and replayed for every token.
#include <algorithm>
#include <cmath>
#include <vector>

#include "decoder.hpp"
#include "int4_common.hpp"
#include "kernels.hpp"
#include "persist.hpp"

namespace yscv {

// ---- random-initialised tiled weights (benchmark setup) -------------------------------------------
// Uniform nibbles and scales ~U(0.005, 0.02) written straight into the tiled layout: for random data
// the tiling is just another arrangement of the same distribution, so no host round trip is needed.
// eight nibbles per word, each uniform over lo .. hi (0 .. 15: the random bits as they come)
__global__ void random_tiles_kernel(uint32_t *__restrict__ words, size_t n_words, uint64_t seed, int lo, int hi) {
  const uint32_t span = (uint32_t)(hi - lo + 1);
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n_words; i += (size_t)gridDim.x * blockDim.x) {
    uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    uint32_t w = (uint32_t)z;
    if (span != 16) {
      w = 0;
      for (int e = 0; e < 8; e++) w |= ((uint32_t)lo + (uint32_t)((z >> (8 * e)) & 0xFFu) * span / 256u) << (4 * e);
    }
    words[i] = w;
  }
}
__global__ void random_scales_kernel(_Float16 *__restrict__ sc, size_t n, uint64_t seed, float lo, float hi) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    const float u = (float)((z >> 40) & 0xFFFFFF) * (1.0f / 16777216.0f);
    sc[i] = (_Float16)(lo + (hi - lo) * u);
  }
}
__global__ void fill_f32_kernel(float *p, size_t n, float v) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
__global__ void set_counters_kernel(int32_t *pos, int32_t *step, int32_t p, int32_t s) {
  if (threadIdx.x == 0) {
    *pos = p;
    *step = s;
  }
}
__global__ void fill_i32_kernel(int32_t *p, size_t n, int32_t v) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

static unsigned grid_for(size_t n) {
  size_t b = ceil_div(n, (size_t)256);
  return (unsigned)(b > 65535 ? 65535 : (b < 1 ? 1 : b));
}

// Random raw weight on the device: [n][k/2] uniform nibble bytes and fp16 scales ~U(0.005, 0.02) in natural
// order, so that every layout built from it (tiled, persistent stream) holds the same logical matrix.
static int32_t random_raw_weight(size_t n, size_t k, size_t g, uint64_t seed, int lo, int hi, uint8_t *raw,
                                 _Float16 *scales) {
  const size_t words = n * k / 8, sc = n * (k / g);
  hipLaunchKernelGGL(random_tiles_kernel, dim3(grid_for(words)), dim3(256), 0, nullptr, reinterpret_cast<uint32_t *>(raw),
                     words, seed, lo, hi);
  hipLaunchKernelGGL(random_scales_kernel, dim3(grid_for(sc)), dim3(256), 0, nullptr, scales, sc, seed ^ 0x5ca1e5ull, 0.005f,
                     0.02f);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

static void destroy_int4(yscv_hip_int4_weight *w) {
  if (!w) return;
  (void)hipFree(w->tiles);
  (void)hipFree(w->tscales);
  (void)hipFree(w->tzps);
  (void)hipFree(w->raw);
  (void)hipFree(w->rscales);
  (void)hipFree(w->rzps);
  delete w;
}

}  // namespace yscv

using namespace yscv;

struct HostLinear {
  std::vector<uint8_t> packed;
  std::vector<uint16_t> scales;
  size_t n = 0, k = 0;
};

struct yscv_hip_decoder {
  yscv_hip_decoder_config cfg{};
  struct Layer {
    yscv_hip_int4_weight *wqkv = nullptr, *wo = nullptr, *wgu = nullptr, *wdown = nullptr;
    float *attn_norm = nullptr, *ffn_norm = nullptr;
    _Float16 *kc = nullptr, *vc = nullptr;   // fp16 cache
    int8_t *kc8 = nullptr, *vc8 = nullptr;   // int8 cache (kv_dtype I8) ...
    float *ks = nullptr, *vs = nullptr;      // ... with one scale per (batch row, position)
    _Float16 *qkv_bias = nullptr;            // null, or [(hq + 2 hkv) hd] added to the q / k / v projection
    HostLinear stage[7];  // q k v o gate up down, kept until finalize
  };
  std::vector<Layer> layers;
  yscv_hip_int4_weight *lm_head = nullptr;
  float *final_norm = nullptr;
  _Float16 *emb = nullptr;
  // activations
  float *h = nullptr, *logits = nullptr, *attn_part = nullptr;
  _Float16 *xn = nullptr, *qkv = nullptr, *ao = nullptr, *act = nullptr;
  _Float16 *qrot = nullptr;       // rotated query heads of the last fused attention launch (diagnostics)
  bool fused_attn = true;         // rope + append inside the attention kernel
  bool generic_attn = false;      // head width other than 128 or more than 4 query heads per kv head: the general kernel
  bool has_bias = false;          // a layer has a q / k / v bias (the single-launch kernel has none)
  // RMSNorm folded into the projections around it (NormFold, kernels.hpp): two buffers of partial sums of squares,
  // written and read in turn, each with the power of two per row that xn's rows were multiplied by
  bool fold_norm = false;         // decided in finish_setup from the shapes
  bool fold_norm_wanted = true;   // test aid: yscv_hip_decoder_debug_set_folded_norm
  float *ss[2] = {nullptr, nullptr};
  float *pre[2] = {nullptr, nullptr};
  int ss_stride = 0;
  int last_ss = 0, last_ss_count = 0;  // what the final norm's consumer read in the last enqueued step
  void *ws = nullptr;
  size_t ws_bytes = 0;
  int32_t *tokens = nullptr, *history = nullptr, *pos = nullptr, *step = nullptr;
  int batch = 0;
  int kv_dtype = YSCV_HIP_KV_F16;
  bool finalized = false;
  hipGraph_t graph = nullptr;
  hipGraphExec_t graph_exec = nullptr;
  int graph_batch = 0;
  size_t weight_bytes = 0;
  // persistent single-launch path (batch 1)
  bool persist_ok = false;     // the shape is supported and the buffers exist
  int last_path = -1;          // path of the last yscv_hip_decoder_run: 0 launches, 1 graph replays, 2 single launch
  int prefill_rows = 4096;     // prompt rows per pass of yscv_hip_decoder_prefill: bounds its activation scratch
  PersistModel pm{};
  uint8_t *p_stream = nullptr;
  uint64_t *p_wg_off = nullptr;
  uint32_t *p_wave_bytes = nullptr;
  float *p_gammas = nullptr;
  _Float16 **p_kc = nullptr, **p_vc = nullptr;
  unsigned long long *p_exch = nullptr;
  uint32_t *p_abort = nullptr;
  size_t p_stream_bytes = 0;
  size_t p_exch_entries = 0;
  uint32_t epoch = 1;          // tag epoch of the next persistent step; tags are 24 bits wide: see yscv_hip_decoder_run
  unsigned long long *p_trace = nullptr;  // stage timestamps (builds with YSCV_PERSIST_TRACE only)
};

// A captured step holds the addresses of the weights and of the workspace as they were at capture time: whatever
// frees or replaces one of them drops the graph, and the next graph run captures again.
static void drop_graph(yscv_hip_decoder *d) {
  if (d->graph_exec) (void)hipGraphExecDestroy(d->graph_exec);
  if (d->graph) (void)hipGraphDestroy(d->graph);
  d->graph_exec = nullptr;
  d->graph = nullptr;
  d->graph_batch = 0;
}

static void decoder_free(yscv_hip_decoder *d) {
  if (!d) return;
  drop_graph(d);
  for (auto &L : d->layers) {
    destroy_int4(L.wqkv);
    destroy_int4(L.wo);
    destroy_int4(L.wgu);
    destroy_int4(L.wdown);
    (void)hipFree(L.attn_norm);
    (void)hipFree(L.ffn_norm);
    (void)hipFree(L.kc);
    (void)hipFree(L.vc);
    (void)hipFree(L.kc8);
    (void)hipFree(L.vc8);
    (void)hipFree(L.ks);
    (void)hipFree(L.vs);
    (void)hipFree(L.qkv_bias);
  }
  destroy_int4(d->lm_head);
  (void)hipFree(d->final_norm);
  (void)hipFree(d->emb);
  (void)hipFree(d->h);
  (void)hipFree(d->logits);
  (void)hipFree(d->attn_part);
  (void)hipFree(d->qrot);
  (void)hipFree(d->ss[0]);
  (void)hipFree(d->ss[1]);
  (void)hipFree(d->pre[0]);
  (void)hipFree(d->pre[1]);
  (void)hipFree(d->xn);
  (void)hipFree(d->qkv);
  (void)hipFree(d->ao);
  (void)hipFree(d->act);
  (void)hipFree(d->ws);
  (void)hipFree(d->tokens);
  (void)hipFree(d->history);
  (void)hipFree(d->pos);
  (void)hipFree(d->step);
  (void)hipFree(d->p_stream);
  (void)hipFree(d->p_wg_off);
  (void)hipFree(d->p_wave_bytes);
  (void)hipFree(d->p_gammas);
  (void)hipFree(d->p_kc);
  (void)hipFree(d->p_vc);
  (void)hipFree(d->p_exch);
  (void)hipFree(d->p_abort);
  (void)hipFree(d->p_trace);
  delete d;
}

#define DEC_HIP(expr)                                                                                \
  do {                                                                                               \
    hipError_t _e = (expr);                                                                          \
    if (_e != hipSuccess)                                                                            \
      return set_error(_e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE, "%s failed: %s", #expr, \
                       hipGetErrorString(_e));                                                       \
  } while (0)

static size_t kv_elems(const yscv_hip_decoder_config &c) {
  return (size_t)c.max_batch * c.n_kv_heads * c.max_ctx * c.head_dim;
}

// Allocate the persistent path's stream and exchange buffers when the shape allows it.
static int32_t persist_setup(yscv_hip_decoder *d) {
  const Context *ctx = nullptr;
  YSCV_TRY(ensure_context(&ctx));
  const auto &c = d->cfg;
  const char *why = "";
  if (d->kv_dtype != YSCV_HIP_KV_F16) return YSCV_HIP_OK;  // the single-launch kernel reads an fp16 cache only
  if (!persist_supported(c, ctx->num_cus, &why)) return YSCV_HIP_OK;  // the multi-kernel path remains
  PersistModel &m = d->pm;
  persist_fill_phases(c, ctx->num_cus, &m);
  const int G = m.G;
  std::vector<uint64_t> off(G);
  std::vector<uint32_t> wb(G);
  size_t total = 0;
  for (int w = 0; w < G; w++) {
    const size_t b = persist_wave_bytes(m, w);
    YSCV_REQUIRE(b < (1ull << 32), "weight stream of one wave exceeds 4 GiB");
    off[w] = total;
    wb[w] = (uint32_t)b;
    total += b * PS_WAVES;
  }
  d->p_stream_bytes = total;
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_stream), total + 4096));  // slack: the prefetcher reads a dword lane pattern
  DEC_HIP(hipMemset(d->p_stream, 0, total + 4096));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_wg_off), G * 8));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_wave_bytes), G * 4));
  DEC_HIP(hipMemcpy(d->p_wg_off, off.data(), G * 8, hipMemcpyHostToDevice));
  DEC_HIP(hipMemcpy(d->p_wave_bytes, wb.data(), G * 4, hipMemcpyHostToDevice));
  const size_t D = c.d_model;
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_gammas), (2 * (size_t)c.n_layers + 1) * D * 4));
  std::vector<_Float16 *> kc(c.n_layers), vc(c.n_layers);
  for (int l = 0; l < c.n_layers; l++) {
    kc[l] = d->layers[l].kc;
    vc[l] = d->layers[l].vc;
  }
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_kc), c.n_layers * sizeof(void *)));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_vc), c.n_layers * sizeof(void *)));
  DEC_HIP(hipMemcpy(d->p_kc, kc.data(), c.n_layers * sizeof(void *), hipMemcpyHostToDevice));
  DEC_HIP(hipMemcpy(d->p_vc, vc.data(), c.n_layers * sizeof(void *), hipMemcpyHostToDevice));
  // exchange buffers, one allocation: xn | xn2 | qkv | ao | act | part | arg
  const size_t e_xn = persist_vec_entries(c.d_model) + G;
  const size_t e_qkv = (size_t)(c.n_heads + 2 * c.n_kv_heads) * 64;
  const size_t e_ao = persist_vec_entries(c.n_heads * 128);
  const size_t e_act = persist_vec_entries(c.d_ff);
  const size_t e_part = (size_t)c.n_heads * (c.max_ctx / 128) * 132;
  const size_t e_arg = 2 * (size_t)G;
  auto up = [](size_t e) { return (e + 31) & ~(size_t)31; };  // keep every buffer 256-byte aligned
  const size_t total_e = 2 * up(e_xn) + up(e_qkv) + up(e_ao) + up(e_act) + up(e_part) + up(e_arg);
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_exch), total_e * 8));
  DEC_HIP(hipMemset(d->p_exch, 0, total_e * 8));
  d->p_exch_entries = total_e;
  unsigned long long *p = d->p_exch;
  m.xn = p;   p += up(e_xn);
  m.xn2 = p;  p += up(e_xn);
  m.qkv = p;  p += up(e_qkv);
  m.ao = p;   p += up(e_ao);
  m.act = p;  p += up(e_act);
  m.part = p; p += up(e_part);
  m.arg = p;
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_abort), 4));
  DEC_HIP(hipMemset(d->p_abort, 0, 4));
  m.stream = d->p_stream;
  m.wg_off = d->p_wg_off;
  m.wave_bytes = d->p_wave_bytes;
  m.gammas = d->p_gammas;
  m.emb = d->emb;
  m.kc = d->p_kc;
  m.vc = d->p_vc;
  m.logits = d->logits;
  m.tokens = d->tokens;
  m.history = d->history;
  m.abort_flag = d->p_abort;
  m.dbg_t = nullptr;
#if defined(YSCV_PERSIST_TRACE) && YSCV_PERSIST_TRACE
  // performance builds only: [G][n_layers][PERSIST_TRACE_SLOTS] stage timestamps, read back by yscv_hip_debug_persist_trace
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->p_trace), (size_t)G * c.n_layers * PERSIST_TRACE_SLOTS * 8));
  DEC_HIP(hipMemset(d->p_trace, 0, (size_t)G * c.n_layers * PERSIST_TRACE_SLOTS * 8));
  m.dbg_t = d->p_trace;
#endif
  d->persist_ok = true;
  return YSCV_HIP_OK;
}

// pack one projection given on the host (fused, natural row order) into the persistent streams
static int32_t persist_pack_host(yscv_hip_decoder *d, int layer, int kind, const uint8_t *packed, const uint16_t *scales,
                                 size_t n, size_t k) {
  if (!d->persist_ok) return YSCV_HIP_OK;
  DevBuf dp, ds;
  YSCV_TRY(dp.alloc(n * k / 2));
  YSCV_TRY(ds.alloc(n * (k / 32) * 2));
  DEC_HIP(hipMemcpy(dp.p, packed, n * k / 2, hipMemcpyHostToDevice));
  DEC_HIP(hipMemcpy(ds.p, scales, n * (k / 32) * 2, hipMemcpyHostToDevice));
  YSCV_TRY(launch_persist_pack(d->pm, layer, kind, dp.as<uint8_t>(), ds.as<_Float16>(), d->p_stream, nullptr));
  DEC_HIP(hipDeviceSynchronize());
  return YSCV_HIP_OK;
}

static int32_t make_fused(yscv_hip_decoder *d, int layer, int pkind, const HostLinear *parts, int count, bool interleave,
                          size_t g, yscv_hip_int4_weight **out) {
  const size_t k = parts[0].k;
  size_t n_total = 0;
  for (int i = 0; i < count; i++) {
    YSCV_REQUIRE(parts[i].n > 0 && parts[i].k == k, "projection missing or with a different K");
    n_total += parts[i].n;
  }
  const size_t row_b = k / 2, row_s = k / g;
  std::vector<uint8_t> packed(n_total * row_b);
  std::vector<uint16_t> scales(n_total * row_s);
  if (interleave) {
    YSCV_REQUIRE(count == 2 && parts[0].n == parts[1].n, "interleaving needs two equal projections");
    for (size_t r = 0; r < parts[0].n; r++)
      for (int p = 0; p < 2; p++) {
        memcpy(&packed[(2 * r + p) * row_b], &parts[p].packed[r * row_b], row_b);
        memcpy(&scales[(2 * r + p) * row_s], &parts[p].scales[r * row_s], row_s * 2);
      }
  } else {
    size_t r0 = 0;
    for (int i = 0; i < count; i++) {
      memcpy(&packed[r0 * row_b], parts[i].packed.data(), parts[i].n * row_b);
      memcpy(&scales[r0 * row_s], parts[i].scales.data(), parts[i].n * row_s * 2);
      r0 += parts[i].n;
    }
  }
  YSCV_TRY(persist_pack_host(d, layer, pkind, packed.data(), scales.data(), n_total, k));
  return yscv_hip_int4_weight_create(packed.data(), scales.data(), YSCV_HIP_F16, nullptr, YSCV_HIP_NIBBLE_UNSIGNED,
                                     n_total, k, g, out);
}

static int32_t alloc_runtime(yscv_hip_decoder *d) {
  const auto &c = d->cfg;
  const size_t B = c.max_batch, D = c.d_model;
  const size_t qkv_n = (size_t)(c.n_heads + 2 * c.n_kv_heads) * c.head_dim;
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->h), B * D * 4));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->logits), B * c.vocab * 4));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->xn), B * D * 2));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->qkv), B * qkv_n * 2));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->ao), B * (size_t)c.n_heads * c.head_dim * 2));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->act), B * (size_t)c.d_ff * 2));
  const size_t chunks = c.max_ctx / 128;
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->attn_part), B * c.n_heads * chunks * (c.head_dim + 2) * 4));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->qrot), B * (size_t)c.n_heads * c.head_dim * 2));
  DEC_HIP(hipMemset(d->qrot, 0, B * (size_t)c.n_heads * c.head_dim * 2));
  d->ss_stride = c.d_model / 16;
  for (int i = 0; i < 2; i++) {
    DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->ss[i]), B * (size_t)d->ss_stride * 4));
    DEC_HIP(hipMemset(d->ss[i], 0, B * (size_t)d->ss_stride * 4));
    const std::vector<float> ones(B, 1.0f);
    DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->pre[i]), B * 4));
    DEC_HIP(hipMemcpy(d->pre[i], ones.data(), B * 4, hipMemcpyHostToDevice));
  }
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->tokens), B * 4));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->history), B * (size_t)c.max_steps * 4));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->pos), 4));
  DEC_HIP(hipMalloc(reinterpret_cast<void **>(&d->step), 4));
  DEC_HIP(hipMemset(d->tokens, 0, B * 4));
  DEC_HIP(hipMemset(d->history, 0, B * (size_t)c.max_steps * 4));
  DEC_HIP(hipMemset(d->pos, 0, 4));
  DEC_HIP(hipMemset(d->step, 0, 4));
  return YSCV_HIP_OK;
}

static int32_t finish_setup(yscv_hip_decoder *d) {
  drop_graph(d);
  // workspace: the largest any projection needs at the maximum batch
  size_t need = 0;
  auto upd = [&](const yscv_hip_int4_weight *w) -> int32_t {
    size_t b = 0;
    YSCV_TRY(int4_workspace_bytes(w, d->cfg.max_batch, YSCV_HIP_F16, 1, &b));
    if (b > need) need = b;
    return YSCV_HIP_OK;
  };
  d->weight_bytes = 0;
  for (auto &L : d->layers) {
    for (auto *w : {L.wqkv, L.wo, L.wgu, L.wdown}) {
      YSCV_REQUIRE(w != nullptr, "a projection was never set");
      YSCV_TRY(upd(w));
      d->weight_bytes += w->device_bytes;
    }
  }
  YSCV_REQUIRE(d->lm_head != nullptr, "lm_head was never set");
  YSCV_TRY(upd(d->lm_head));
  d->weight_bytes += d->lm_head->device_bytes;
  if (need > d->ws_bytes) {
    (void)hipFree(d->ws);
    d->ws = nullptr;
    DEC_HIP(hipMalloc(&d->ws, need));
    d->ws_bytes = need;
  }
  if (d->persist_ok) {
    const size_t D = d->cfg.d_model;
    for (size_t l = 0; l < d->layers.size(); l++) {
      DEC_HIP(hipMemcpy(d->p_gammas + (2 * l) * D, d->layers[l].attn_norm, D * 4, hipMemcpyDeviceToDevice));
      DEC_HIP(hipMemcpy(d->p_gammas + (2 * l + 1) * D, d->layers[l].ffn_norm, D * 4, hipMemcpyDeviceToDevice));
    }
    DEC_HIP(hipMemcpy(d->p_gammas + 2 * d->layers.size() * D, d->final_norm, D * 4, hipMemcpyDeviceToDevice));
  }
  // the norms fold into the projections when the second pass of a K-split update can take whole 256-column pieces
  // and the projections that consume a norm are not K-split themselves
  {
    const Context *ctx = nullptr;
    YSCV_TRY(ensure_context(&ctx));
    // (a consuming projection adds up at most 256 partial sums per row, four rows per wave of 512 k)
    bool ok = d->cfg.d_model % 256 == 0 && d->cfg.d_model <= 4096 && d->fold_norm_wanted;
    auto consumes = [&](const yscv_hip_int4_weight *w) {
      if (!w->tiled) return false;
      const SkinnyPlan plan = plan_int4_skinny(w, d->cfg.max_batch, 1, ctx->num_cus);
      return plan.ksg == 1 && d->cfg.max_batch <= 4 * plan.waves;
    };
    for (auto &L : d->layers)
      for (auto *w : {L.wqkv, L.wgu}) ok = ok && consumes(w);
    ok = ok && consumes(d->lm_head);
    for (auto &L : d->layers) ok = ok && L.wo->tiled && L.wdown->tiled;
    // every projection takes its fp16 activations as they are (no padded copy with a row scale of its own)
    auto direct = [](const yscv_hip_int4_weight *w) { return w->ktp * 128 == w->k; };
    for (auto &L : d->layers)
      for (auto *w : {L.wqkv, L.wo, L.wgu, L.wdown}) ok = ok && direct(w);
    ok = ok && direct(d->lm_head);
    d->fold_norm = ok;
  }
  d->finalized = true;
  return YSCV_HIP_OK;
}

// every launch of one decode step, in order, on stream s
static int32_t enqueue_step(yscv_hip_decoder *d, int batch, hipStream_t s) {
  const auto &c = d->cfg;
  const int D = c.d_model;
  const bool fold = d->fold_norm;
  // folded norms: `cur` is the buffer of partial sums the next consumer reads, `cnt` how many partials a row has there
  int cur = 0, cnt = 0;
  // `feeds_update`: a residual update follows this norm's projection and takes its row scales from it
  auto consumer = [&](NormFold &nf, bool feeds_update) {
    nf.ss_in = d->ss[cur];
    nf.pre_in = d->pre[cur];
    nf.pre_next = feeds_update ? d->pre[cur ^ 1] : nullptr;
    nf.ss_in_count = cnt;
    nf.ss_in_stride = d->ss_stride;
    nf.inv_d = 1.0f / (float)D;
    nf.eps = c.rms_eps;
  };
  auto producer = [&](NormFold &nf, const float *gamma, int *count_out) {
    nf.gamma_next = gamma;
    nf.pre = d->pre[cur ^ 1];
    nf.xg = d->xn;
    nf.ss_out = d->ss[cur ^ 1];
    nf.ss_out_stride = d->ss_stride;
    nf.ss_out_count = count_out;
  };
  if (fold) {
    YSCV_TRY(launch_embed_norm(d->tokens, d->emb, batch, D, c.vocab, c.rms_eps, d->h, d->layers[0].attn_norm, d->xn, d->ss[0],
                               d->ss_stride, d->pre[0], s));
    cur = 0;
    cnt = 1;
  } else {
    YSCV_TRY(launch_embed(d->tokens, d->emb, batch, D, c.vocab, d->h, s));
  }
  for (size_t li = 0; li < d->layers.size(); li++) {
    auto &L = d->layers[li];
    if (fold) {
      NormFold nf;
      consumer(nf, true);
      YSCV_TRY(int4_run_ws(L.wqkv, d->xn, YSCV_HIP_F16, d->qkv, YSCV_HIP_F16, batch, 1, EPI_STORE, d->ws, d->ws_bytes, s, &nf));
    } else {
      YSCV_TRY(launch_rmsnorm(d->h, L.attn_norm, batch, D, c.rms_eps, d->xn, s));
      YSCV_TRY(int4_run_ws(L.wqkv, d->xn, YSCV_HIP_F16, d->qkv, YSCV_HIP_F16, batch, 1, EPI_STORE, d->ws, d->ws_bytes, s));
    }
    const int qkv_n = (c.n_heads + 2 * c.n_kv_heads) * c.head_dim;
    if (L.qkv_bias) YSCV_TRY(launch_bias_add_f16(d->qkv, L.qkv_bias, (size_t)batch, (size_t)qkv_n, s));
    if (d->generic_attn && d->fused_attn) {
      YSCV_TRY(launch_gqa_cache(d->qkv, L.kc, L.vc, d->pos, batch, 0, c.n_heads, c.n_kv_heads, c.head_dim, c.max_ctx, d->ao, s,
                                c.rope_theta, d->qrot));
    } else if (d->generic_attn) {
      YSCV_TRY(launch_rope_append(d->qkv, d->pos, batch, c.n_heads, c.n_kv_heads, c.head_dim, c.rope_theta, c.max_ctx,
                                  L.kc, L.vc, s));
      YSCV_TRY(launch_gqa_cache(d->qkv, L.kc, L.vc, d->pos, batch, 0, c.n_heads, c.n_kv_heads, c.head_dim, c.max_ctx, d->ao, s));
    } else if (d->kv_dtype == YSCV_HIP_KV_I8 && d->fused_attn) {
      YSCV_TRY(launch_attention_fused_i8(d->qkv, L.kc8, L.ks, L.vc8, L.vs, d->pos, batch, c.n_heads, c.n_kv_heads, c.head_dim,
                                         c.rope_theta, c.max_ctx, d->attn_part, d->qrot, d->ao, s));
    } else if (d->kv_dtype == YSCV_HIP_KV_I8) {
      YSCV_TRY(launch_rope_append_i8(d->qkv, d->pos, batch, c.n_heads, c.n_kv_heads, c.head_dim, c.rope_theta, c.max_ctx,
                                     L.kc8, L.ks, L.vc8, L.vs, s));
      YSCV_TRY(launch_attention_i8(d->qkv, L.kc8, L.ks, L.vc8, L.vs, d->pos, batch, c.n_heads, c.n_kv_heads, c.head_dim,
                                   c.max_ctx, d->attn_part, d->ao, s));
    } else if (d->fused_attn) {
      YSCV_TRY(launch_attention_fused(d->qkv, L.kc, L.vc, d->pos, batch, c.n_heads, c.n_kv_heads, c.head_dim, c.rope_theta,
                                      c.max_ctx, d->attn_part, d->qrot, d->ao, s));
    } else {
      YSCV_TRY(launch_rope_append(d->qkv, d->pos, batch, c.n_heads, c.n_kv_heads, c.head_dim, c.rope_theta, c.max_ctx,
                                  L.kc, L.vc, s));
      YSCV_TRY(launch_attention(d->qkv, L.kc, L.vc, d->pos, batch, c.n_heads, c.n_kv_heads, c.head_dim, c.max_ctx,
                                d->attn_part, d->ao, s));
    }
    if (fold) {
      // o: h += W ao, and the ffn norm's inputs; gate/up reads them; down: h += W act, and the next norm's inputs
      NormFold po, cg, pd;
      int n_o = 0, n_d = 0;
      producer(po, L.ffn_norm, &n_o);
      YSCV_TRY(int4_run_ws(L.wo, d->ao, YSCV_HIP_F16, d->h, YSCV_HIP_F32, batch, 1, EPI_ADD_F32, d->ws, d->ws_bytes, s, &po));
      cur ^= 1;
      cnt = n_o;
      consumer(cg, true);
      YSCV_TRY(int4_run_ws(L.wgu, d->xn, YSCV_HIP_F16, d->act, YSCV_HIP_F16, batch, 1, EPI_SWIGLU, d->ws, d->ws_bytes, s, &cg));
      producer(pd, li + 1 < d->layers.size() ? d->layers[li + 1].attn_norm : d->final_norm, &n_d);
      YSCV_TRY(int4_run_ws(L.wdown, d->act, YSCV_HIP_F16, d->h, YSCV_HIP_F32, batch, 1, EPI_ADD_F32, d->ws, d->ws_bytes, s, &pd));
      cur ^= 1;
      cnt = n_d;
    } else {
      YSCV_TRY(int4_run_ws(L.wo, d->ao, YSCV_HIP_F16, d->h, YSCV_HIP_F32, batch, 1, EPI_ADD_F32, d->ws, d->ws_bytes, s));
      YSCV_TRY(launch_rmsnorm(d->h, L.ffn_norm, batch, D, c.rms_eps, d->xn, s));
      YSCV_TRY(int4_run_ws(L.wgu, d->xn, YSCV_HIP_F16, d->act, YSCV_HIP_F16, batch, 1, EPI_SWIGLU, d->ws, d->ws_bytes, s));
      YSCV_TRY(int4_run_ws(L.wdown, d->act, YSCV_HIP_F16, d->h, YSCV_HIP_F32, batch, 1, EPI_ADD_F32, d->ws, d->ws_bytes, s));
    }
  }
  if (fold) {
    NormFold nf;
    consumer(nf, false);
    d->last_ss = cur;
    d->last_ss_count = cnt;
    YSCV_TRY(int4_run_ws(d->lm_head, d->xn, YSCV_HIP_F16, d->logits, YSCV_HIP_F32, batch, 1, EPI_STORE, d->ws, d->ws_bytes, s, &nf));
  } else {
    YSCV_TRY(launch_rmsnorm(d->h, d->final_norm, batch, D, c.rms_eps, d->xn, s));
    YSCV_TRY(int4_run_ws(d->lm_head, d->xn, YSCV_HIP_F16, d->logits, YSCV_HIP_F32, batch, 1, EPI_STORE, d->ws, d->ws_bytes, s));
  }
  YSCV_TRY(launch_argmax(d->logits, batch, c.vocab, d->tokens, d->history, d->step, c.max_steps, s));
  YSCV_TRY(launch_advance(d->pos, d->step, s));
  return YSCV_HIP_OK;
}

static int32_t check_persist_abort(yscv_hip_decoder *d) {
  if (!d->persist_ok) return YSCV_HIP_OK;
  uint32_t flag = 0;
  DEC_HIP(hipMemcpy(&flag, d->p_abort, 4, hipMemcpyDeviceToHost));
  if (flag) {
    DEC_HIP(hipMemset(d->p_abort, 0, 4));
    return set_error(YSCV_HIP_ERR_DEVICE, "the single-launch decode kernel gave up waiting for a stage (bounded wait expired)");
  }
  return YSCV_HIP_OK;
}

extern "C" {

int32_t yscv_hip_decoder_create(const yscv_hip_decoder_config *cfg, yscv_hip_decoder **out) {
  return yscv_hip_decoder_create_kv(cfg, YSCV_HIP_KV_F16, out);
}

int32_t yscv_hip_decoder_create_kv(const yscv_hip_decoder_config *cfg, int32_t kv_dtype, yscv_hip_decoder **out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(cfg && out, "null argument");
  YSCV_REQUIRE(kv_dtype == YSCV_HIP_KV_F16 || kv_dtype == YSCV_HIP_KV_I8, "unknown KV cache dtype %d", kv_dtype);
  *out = nullptr;
  const auto &c = *cfg;
  YSCV_REQUIRE(c.n_layers > 0 && c.d_model > 0 && c.n_heads > 0 && c.n_kv_heads > 0 && c.d_ff > 0 && c.vocab > 0,
               "non-positive model dimension");
  YSCV_REQUIRE(c.head_dim == 32 || c.head_dim == 64 || c.head_dim == 96 || c.head_dim == 128,
               "head_dim must be 32, 64, 96 or 128 (got %d)", c.head_dim);
  YSCV_REQUIRE(c.n_heads % c.n_kv_heads == 0, "the kv heads must divide the query heads (%d over %d)", c.n_heads, c.n_kv_heads);
  const bool generic_attn = c.head_dim != 128 || c.n_heads / c.n_kv_heads > 4;
  if (generic_attn && kv_dtype == YSCV_HIP_KV_I8)
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "the int8 cache exists for head_dim 128 with 1..4 query heads per kv head");
  YSCV_REQUIRE(c.d_model % 128 == 0 && c.d_ff % 128 == 0 && (c.n_heads * c.head_dim) % 128 == 0,
               "d_model, d_ff and n_heads*head_dim must be multiples of 128");
  YSCV_REQUIRE(c.max_batch >= 1 && c.max_batch <= 16, "max_batch must be 1..16 (skinny kernel)");
  YSCV_REQUIRE(c.max_ctx >= 128 && c.max_ctx % 128 == 0, "max_ctx must be a positive multiple of 128");
  YSCV_REQUIRE(c.max_steps >= 1, "max_steps must be positive");
  YSCV_REQUIRE(c.group_size == 32 || c.group_size == 64 || c.group_size % 128 == 0, "unsupported group size");
  YSCV_REQUIRE(c.rms_eps > 0.0f, "rms_eps must be finite and > 0 (ops/norm.rs:1471)");
  auto *d = new yscv_hip_decoder();
  d->cfg = c;
  d->kv_dtype = kv_dtype;
  d->generic_attn = generic_attn;
  d->layers.resize(c.n_layers);
  int32_t st = alloc_runtime(d);
  const size_t D = c.d_model;
  for (auto &L : d->layers) {
    if (st != YSCV_HIP_OK) break;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&L.attn_norm), D * 4);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&L.ffn_norm), D * 4);
    if (kv_dtype == YSCV_HIP_KV_I8) {
      const size_t rows = (size_t)c.max_batch * c.max_ctx;
      if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&L.kc8), kv_elems(c));
      if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&L.vc8), kv_elems(c));
      if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&L.ks), rows * 4);
      if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&L.vs), rows * 4);
      if (e == hipSuccess) e = hipMemset(L.kc8, 0, kv_elems(c));
      if (e == hipSuccess) e = hipMemset(L.vc8, 0, kv_elems(c));
      if (e == hipSuccess) e = hipMemset(L.ks, 0, rows * 4);
      if (e == hipSuccess) e = hipMemset(L.vs, 0, rows * 4);
    } else {
      if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&L.kc), kv_elems(c) * 2);
      if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&L.vc), kv_elems(c) * 2);
      if (e == hipSuccess) e = hipMemset(L.kc, 0, kv_elems(c) * 2);
      if (e == hipSuccess) e = hipMemset(L.vc, 0, kv_elems(c) * 2);
    }
    if (e != hipSuccess)
      st = set_error(e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE, "layer allocation failed: %s",
                     hipGetErrorString(e));
    else {
      hipLaunchKernelGGL(fill_f32_kernel, dim3(grid_for(D)), dim3(256), 0, nullptr, L.attn_norm, D, 1.0f);
      hipLaunchKernelGGL(fill_f32_kernel, dim3(grid_for(D)), dim3(256), 0, nullptr, L.ffn_norm, D, 1.0f);
    }
  }
  if (st == YSCV_HIP_OK) {
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&d->final_norm), D * 4);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&d->emb), (size_t)c.vocab * D * 2);
    if (e != hipSuccess)
      st = set_error(e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE, "allocation failed: %s",
                     hipGetErrorString(e));
    else
      hipLaunchKernelGGL(fill_f32_kernel, dim3(grid_for(D)), dim3(256), 0, nullptr, d->final_norm, D, 1.0f);
  }
  if (st == YSCV_HIP_OK) {
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) st = set_error(YSCV_HIP_ERR_DEVICE, "setup failed: %s", hipGetErrorString(e));
  }
  if (st == YSCV_HIP_OK && c.max_batch >= 1) st = persist_setup(d);
  if (st != YSCV_HIP_OK) {
    decoder_free(d);
    return st;
  }
  *out = d;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_destroy(yscv_hip_decoder *d) {
  decoder_free(d);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_set_linear(yscv_hip_decoder *d, int32_t layer, int32_t kind, const uint8_t *packed,
                                    const uint16_t *scales_f16, size_t n, size_t k) {
  YSCV_REQUIRE(d && packed && scales_f16, "null argument");
  YSCV_REQUIRE(kind >= 0 && kind <= YSCV_HIP_DEC_LM_HEAD, "unknown projection kind %d", kind);
  const auto &c = d->cfg;
  const size_t g = c.group_size;
  YSCV_REQUIRE(k % g == 0, "group size does not divide k");
  const size_t hq = (size_t)c.n_heads * c.head_dim, hkv = (size_t)c.n_kv_heads * c.head_dim;
  const size_t exp_n[8] = {hq, hkv, hkv, (size_t)c.d_model, (size_t)c.d_ff, (size_t)c.d_ff, (size_t)c.d_model, (size_t)c.vocab};
  const size_t exp_k[8] = {(size_t)c.d_model, (size_t)c.d_model, (size_t)c.d_model, hq, (size_t)c.d_model,
                           (size_t)c.d_model, (size_t)c.d_ff, (size_t)c.d_model};
  YSCV_REQUIRE(n == exp_n[kind] && k == exp_k[kind], "projection %d must be [%zu][%zu], got [%zu][%zu]", kind,
               exp_n[kind], exp_k[kind], n, k);
  d->finalized = false;
  drop_graph(d);
  if (kind == YSCV_HIP_DEC_LM_HEAD) {
    destroy_int4(d->lm_head);
    d->lm_head = nullptr;
    YSCV_TRY(persist_pack_host(d, 0, PK_LM, packed, scales_f16, n, k));
    return yscv_hip_int4_weight_create(packed, scales_f16, YSCV_HIP_F16, nullptr, YSCV_HIP_NIBBLE_UNSIGNED, n, k, g,
                                       &d->lm_head);
  }
  YSCV_REQUIRE(layer >= 0 && layer < c.n_layers, "layer %d out of range", layer);
  HostLinear &hl = d->layers[layer].stage[kind];
  hl.n = n;
  hl.k = k;
  hl.packed.assign(packed, packed + n * k / 2);
  hl.scales.assign(scales_f16, scales_f16 + n * (k / g));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_set_norm(yscv_hip_decoder *d, int32_t layer, int32_t kind, const float *gamma) {
  YSCV_REQUIRE(d && gamma, "null argument");
  float *dst = nullptr;
  if (kind == YSCV_HIP_DEC_FINAL_NORM) {
    dst = d->final_norm;
  } else {
    YSCV_REQUIRE(layer >= 0 && layer < d->cfg.n_layers, "layer %d out of range", layer);
    YSCV_REQUIRE(kind == YSCV_HIP_DEC_ATTN_NORM || kind == YSCV_HIP_DEC_FFN_NORM, "unknown norm kind %d", kind);
    dst = kind == YSCV_HIP_DEC_ATTN_NORM ? d->layers[layer].attn_norm : d->layers[layer].ffn_norm;
  }
  DEC_HIP(hipMemcpy(dst, gamma, (size_t)d->cfg.d_model * 4, hipMemcpyHostToDevice));
  d->finalized = false;  // the persistent path keeps its own contiguous copy, refreshed by finalize
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_set_embedding(yscv_hip_decoder *d, const uint16_t *table_f16) {
  YSCV_REQUIRE(d && table_f16, "null argument");
  DEC_HIP(hipMemcpy(d->emb, table_f16, (size_t)d->cfg.vocab * d->cfg.d_model * 2, hipMemcpyHostToDevice));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_finalize(yscv_hip_decoder *d) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  const size_t g = d->cfg.group_size;
  for (int li = 0; li < (int)d->layers.size(); li++) {
    auto &L = d->layers[li];
    if (L.stage[0].n) {  // q, k, v staged -> fused [q; k; v]
      destroy_int4(L.wqkv);
      L.wqkv = nullptr;
      YSCV_TRY(make_fused(d, li, PK_QKV, &L.stage[0], 3, false, g, &L.wqkv));
      for (int i = 0; i < 3; i++) L.stage[i] = HostLinear();
    }
    if (L.stage[3].n) {
      destroy_int4(L.wo);
      L.wo = nullptr;
      YSCV_TRY(make_fused(d, li, PK_O, &L.stage[3], 1, false, g, &L.wo));
      L.stage[3] = HostLinear();
    }
    if (L.stage[4].n) {  // gate, up staged -> rows interleaved gate_0, up_0, gate_1, ... for the SwiGLU epilogue
      destroy_int4(L.wgu);
      L.wgu = nullptr;
      YSCV_TRY(make_fused(d, li, PK_GU, &L.stage[4], 2, true, g, &L.wgu));
      L.stage[4] = HostLinear();
      L.stage[5] = HostLinear();
    }
    if (L.stage[6].n) {
      destroy_int4(L.wdown);
      L.wdown = nullptr;
      YSCV_TRY(make_fused(d, li, PK_DOWN, &L.stage[6], 1, false, g, &L.wdown));
      L.stage[6] = HostLinear();
    }
  }
  return finish_setup(d);
}

int32_t yscv_hip_decoder_init_random(yscv_hip_decoder *d, uint64_t seed) {
  return yscv_hip_decoder_init_random_range(d, seed, 0, 15);
}

int32_t yscv_hip_decoder_init_random_range(yscv_hip_decoder *d, uint64_t seed, int32_t nibble_lo, int32_t nibble_hi) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  YSCV_REQUIRE(nibble_lo >= 0 && nibble_lo <= nibble_hi && nibble_hi <= 15, "nibble range must lie in 0..15");
  const auto &c = d->cfg;
  const size_t g = c.group_size, D = c.d_model;
  const size_t qkv_n = (size_t)(c.n_heads + 2 * c.n_kv_heads) * c.head_dim;
  uint64_t sd = seed * 0x100000001B3ull + 1;
  d->finalized = false;
  drop_graph(d);
  // one raw buffer, sized for the largest projection, reused for every weight
  const size_t max_elems = std::max(std::max(qkv_n, 2 * (size_t)c.d_ff) * D, std::max((size_t)c.vocab * D, D * (size_t)c.d_ff));
  DevBuf raw, rsc;
  YSCV_TRY(raw.alloc(max_elems / 2));
  YSCV_TRY(rsc.alloc(max_elems / g * 2));
  auto make = [&](int layer, int pkind, size_t n, size_t k, yscv_hip_int4_weight **out) -> int32_t {
    YSCV_REQUIRE(g == 32 || g == 64 || g % 128 == 0, "random weights need a tiled group size");
    YSCV_TRY(random_raw_weight(n, k, g, sd++, nibble_lo, nibble_hi, raw.as<uint8_t>(), rsc.as<_Float16>()));
    YSCV_TRY(int4_create_from_device(raw.as<uint8_t>(), rsc.p, YSCV_HIP_F16, YSCV_HIP_NIBBLE_UNSIGNED, n, k, g, out));
    if (d->persist_ok) YSCV_TRY(launch_persist_pack(d->pm, layer, pkind, raw.as<uint8_t>(), rsc.as<_Float16>(), d->p_stream, nullptr));
    DEC_HIP(hipDeviceSynchronize());  // the raw buffer is reused by the next weight
    return YSCV_HIP_OK;
  };
  for (int li = 0; li < (int)d->layers.size(); li++) {
    auto &L = d->layers[li];
    destroy_int4(L.wqkv);
    destroy_int4(L.wo);
    destroy_int4(L.wgu);
    destroy_int4(L.wdown);
    L.wqkv = L.wo = L.wgu = L.wdown = nullptr;
    YSCV_TRY(make(li, PK_QKV, qkv_n, D, &L.wqkv));
    YSCV_TRY(make(li, PK_O, D, (size_t)c.n_heads * c.head_dim, &L.wo));
    YSCV_TRY(make(li, PK_GU, 2 * (size_t)c.d_ff, D, &L.wgu));
    YSCV_TRY(make(li, PK_DOWN, D, (size_t)c.d_ff, &L.wdown));
  }
  destroy_int4(d->lm_head);
  d->lm_head = nullptr;
  YSCV_TRY(make(0, PK_LM, (size_t)c.vocab, D, &d->lm_head));
  YSCV_TRY(launch_kv_random_fill(d->emb, (size_t)c.vocab * D, sd++, nullptr));
  DEC_HIP(hipDeviceSynchronize());
  return finish_setup(d);
}

int32_t yscv_hip_decoder_fill_kv_random(yscv_hip_decoder *d, uint64_t seed) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  uint64_t sd = seed * 0x9E3779B1ull + 7;
  const size_t rows = (size_t)d->cfg.max_batch * d->cfg.max_ctx;
  for (auto &L : d->layers) {
    if (d->kv_dtype == YSCV_HIP_KV_I8) {  // bytes uniform in [-127, 127], scale 3.5 / 127: values span about +-3.5
      YSCV_TRY(launch_kv_random_fill_i8(L.kc8, kv_elems(d->cfg), L.ks, rows, 3.5f / 127.0f, sd++, nullptr));
      YSCV_TRY(launch_kv_random_fill_i8(L.vc8, kv_elems(d->cfg), L.vs, rows, 3.5f / 127.0f, sd++, nullptr));
    } else {
      YSCV_TRY(launch_kv_random_fill(L.kc, kv_elems(d->cfg), sd++, nullptr));
      YSCV_TRY(launch_kv_random_fill(L.vc, kv_elems(d->cfg), sd++, nullptr));
    }
  }
  DEC_HIP(hipDeviceSynchronize());
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_set_kv(yscv_hip_decoder *d, int32_t layer, const uint16_t *k_f16, const uint16_t *v_f16,
                                int32_t batch, int32_t n_positions) {
  YSCV_REQUIRE(d && k_f16 && v_f16, "null argument");
  const auto &c = d->cfg;
  YSCV_REQUIRE(layer >= 0 && layer < c.n_layers, "layer %d out of range", layer);
  YSCV_REQUIRE(batch >= 1 && batch <= c.max_batch && n_positions >= 0 && n_positions <= c.max_ctx, "bad batch / positions");
  if (n_positions == 0) return YSCV_HIP_OK;
  const size_t elems = (size_t)batch * n_positions * c.n_kv_heads * c.head_dim;
  DevBuf dk, dv;
  YSCV_TRY(dk.alloc(elems * 2));
  YSCV_TRY(dv.alloc(elems * 2));
  DEC_HIP(hipMemcpy(dk.p, k_f16, elems * 2, hipMemcpyHostToDevice));
  DEC_HIP(hipMemcpy(dv.p, v_f16, elems * 2, hipMemcpyHostToDevice));
  auto &L = d->layers[layer];
  if (d->kv_dtype == YSCV_HIP_KV_I8)
    YSCV_TRY(launch_kv_relayout_i8(dk.as<_Float16>(), dv.as<_Float16>(), batch, n_positions, c.n_kv_heads, c.head_dim,
                                   c.max_ctx, L.kc8, L.ks, L.vc8, L.vs, nullptr));
  else
    YSCV_TRY(launch_kv_relayout(dk.as<_Float16>(), dv.as<_Float16>(), batch, n_positions, c.n_kv_heads, c.head_dim,
                                c.max_ctx, L.kc, L.vc, nullptr));
  DEC_HIP(hipDeviceSynchronize());
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_get_kv(yscv_hip_decoder *d, int32_t layer, uint16_t *k_f16, uint16_t *v_f16, int32_t batch,
                                int32_t first_pos, int32_t n_positions) {
  YSCV_REQUIRE(d && k_f16 && v_f16, "null argument");
  const auto &c = d->cfg;
  YSCV_REQUIRE(layer >= 0 && layer < c.n_layers, "layer %d out of range", layer);
  YSCV_REQUIRE(batch >= 1 && batch <= c.max_batch && first_pos >= 0 && n_positions >= 0 &&
                   first_pos + n_positions <= c.max_ctx,
               "bad batch / position range");
  if (n_positions == 0) return YSCV_HIP_OK;
  DEC_HIP(hipDeviceSynchronize());
  const int hd = c.head_dim, hkv = c.n_kv_heads;
  const int s0 = first_pos / 8, s1 = (first_pos + n_positions + 7) / 8;  // 8-position slabs of the V layout
  const auto &L = d->layers[layer];
  if (d->kv_dtype == YSCV_HIP_KV_I8) {  // q * scale of its row (dequantise_to_vec, kv_cache.rs:64-79), narrowed to fp16
    std::vector<int8_t> k8((size_t)n_positions * hd), v8((size_t)(s1 - s0) * hd * 8);
    std::vector<float> ksc(n_positions), vsc(n_positions);
    for (int b = 0; b < batch; b++) {
      DEC_HIP(hipMemcpy(ksc.data(), L.ks + (size_t)b * c.max_ctx + first_pos, (size_t)n_positions * 4, hipMemcpyDeviceToHost));
      DEC_HIP(hipMemcpy(vsc.data(), L.vs + (size_t)b * c.max_ctx + first_pos, (size_t)n_positions * 4, hipMemcpyDeviceToHost));
      for (int h = 0; h < hkv; h++) {
        const size_t row = (size_t)b * hkv + h;
        DEC_HIP(hipMemcpy(k8.data(), L.kc8 + (row * c.max_ctx + first_pos) * hd, k8.size(), hipMemcpyDeviceToHost));
        DEC_HIP(hipMemcpy(v8.data(), L.vc8 + ((row * (c.max_ctx / 8) + s0) * hd) * 8, v8.size(), hipMemcpyDeviceToHost));
        for (int p = 0; p < n_positions; p++) {
          _Float16 *kd = reinterpret_cast<_Float16 *>(k_f16) + (((size_t)b * n_positions + p) * hkv + h) * hd;
          _Float16 *vd = reinterpret_cast<_Float16 *>(v_f16) + (((size_t)b * n_positions + p) * hkv + h) * hd;
          const int ap = first_pos + p;
          for (int i = 0; i < hd; i++) {
            kd[i] = (_Float16)((float)k8[(size_t)p * hd + i] * ksc[p]);
            vd[i] = (_Float16)((float)v8[((size_t)(ap / 8 - s0) * hd + i) * 8 + (ap & 7)] * vsc[p]);
          }
        }
      }
    }
    return YSCV_HIP_OK;
  }
  std::vector<uint16_t> kt((size_t)n_positions * hd), vt((size_t)(s1 - s0) * hd * 8);
  for (int b = 0; b < batch; b++)
    for (int h = 0; h < hkv; h++) {
      const size_t row = (size_t)b * hkv + h;
      DEC_HIP(hipMemcpy(kt.data(), L.kc + (row * c.max_ctx + first_pos) * hd, kt.size() * 2, hipMemcpyDeviceToHost));
      DEC_HIP(hipMemcpy(vt.data(), L.vc + ((row * (c.max_ctx / 8) + s0) * hd) * 8, vt.size() * 2, hipMemcpyDeviceToHost));
      for (int p = 0; p < n_positions; p++) {
        uint16_t *kd = k_f16 + (((size_t)b * n_positions + p) * hkv + h) * hd;
        uint16_t *vd = v_f16 + (((size_t)b * n_positions + p) * hkv + h) * hd;
        memcpy(kd, &kt[(size_t)p * hd], (size_t)hd * 2);
        const int ap = first_pos + p;
        for (int i = 0; i < hd; i++) vd[i] = vt[((size_t)(ap / 8 - s0) * hd + i) * 8 + (ap & 7)];
      }
    }
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_reset(yscv_hip_decoder *d, int32_t batch, int32_t start_pos, const int32_t *tokens_host) {
  YSCV_REQUIRE(d && tokens_host, "null argument");
  const auto &c = d->cfg;
  YSCV_REQUIRE(batch >= 1 && batch <= c.max_batch, "batch %d out of range 1..%d", batch, c.max_batch);
  YSCV_REQUIRE(start_pos >= 0 && start_pos < c.max_ctx, "start position %d out of range", start_pos);
  d->batch = batch;
  DEC_HIP(hipMemcpy(d->tokens, tokens_host, (size_t)batch * 4, hipMemcpyHostToDevice));
  DEC_HIP(hipMemcpy(d->pos, &start_pos, 4, hipMemcpyHostToDevice));
  const int32_t zero = 0;
  DEC_HIP(hipMemcpy(d->step, &zero, 4, hipMemcpyHostToDevice));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_run(yscv_hip_decoder *d, int32_t n_steps, int32_t use_graph, void *stream) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  YSCV_REQUIRE(d->finalized, "decoder weights are not finalized");
  YSCV_REQUIRE(d->batch >= 1, "call yscv_hip_decoder_reset first");
  YSCV_REQUIRE(n_steps >= 0, "negative step count");
  hipStream_t s = as_stream(stream);
  // host-side bound check: the cache must hold every position this run appends
  int32_t pos = 0, step = 0;
  DEC_HIP(hipStreamSynchronize(s));
  DEC_HIP(hipMemcpy(&pos, d->pos, 4, hipMemcpyDeviceToHost));
  DEC_HIP(hipMemcpy(&step, d->step, 4, hipMemcpyDeviceToHost));
  YSCV_REQUIRE(pos + n_steps <= d->cfg.max_ctx, "KV cache overflow: position %d + %d steps > max_ctx %d", pos, n_steps,
               d->cfg.max_ctx);
  YSCV_REQUIRE(step + n_steps <= d->cfg.max_steps, "token history overflow: %d + %d > max_steps %d", step, n_steps,
               d->cfg.max_steps);
  if (use_graph == YSCV_HIP_DECODE_AUTO)  // the fastest path this decoder has for its batch
    use_graph = (d->batch == 1 && d->persist_ok && !d->has_bias && d->kv_dtype == YSCV_HIP_KV_F16) ? 2 : 1;
  d->last_path = use_graph == 2 ? 2 : (use_graph ? 1 : 0);
  if (use_graph == 2) {
    if (d->kv_dtype != YSCV_HIP_KV_F16)
      return set_error(YSCV_HIP_ERR_UNSUPPORTED, "the single-launch decode path reads an fp16 KV cache only");
    if (!d->persist_ok)
      return set_error(YSCV_HIP_ERR_UNSUPPORTED, "the single-launch decode path does not support this model shape");
    if (d->has_bias) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "the single-launch decode path has no q / k / v bias");
    if (d->batch != 1) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "the single-launch decode path runs batch 1 only");
    if (n_steps == 0) return YSCV_HIP_OK;
    // A tag is ((epoch + step) * (layers + 2) + 1 + layer) modulo 2^24.  Before the tag space wraps, the exchange
    // buffers are cleared and the epoch starts again, so an entry left from half a million steps ago can never be taken
    // for a fresh one.
    const uint64_t per_step = (uint64_t)d->cfg.n_layers + 2;
    YSCV_REQUIRE((uint64_t)n_steps * per_step < (1u << 23), "too many steps for one launch of the single-launch path");
    if (((uint64_t)d->epoch + (uint64_t)n_steps + 1) * per_step + 2 >= (1u << 24)) {
      hipLaunchKernelGGL(fill_i32_kernel, dim3(grid_for(d->p_exch_entries * 2)), dim3(256), 0, s,
                         reinterpret_cast<int32_t *>(d->p_exch), d->p_exch_entries * 2, 0);
      DEC_HIP(hipGetLastError());
      d->epoch = 1;
    }
    YSCV_TRY(launch_persist_decode(d->pm, n_steps, pos, step, d->cfg.max_steps, d->epoch, s));
    d->epoch += (uint32_t)n_steps;
    // position and step counters live on the device for the multi-kernel path: keep them in step
    hipLaunchKernelGGL(set_counters_kernel, dim3(1), dim3(64), 0, s, d->pos, d->step, pos + n_steps, step + n_steps);
    DEC_HIP(hipGetLastError());
    return YSCV_HIP_OK;
  }
  if (!use_graph) {
    for (int i = 0; i < n_steps; i++) YSCV_TRY(enqueue_step(d, d->batch, s));
    return YSCV_HIP_OK;
  }
  if (!d->graph_exec || d->graph_batch != d->batch) {
    drop_graph(d);
    hipStream_t cs = nullptr;
    DEC_HIP(hipStreamCreateWithFlags(&cs, hipStreamNonBlocking));
    hipError_t e = hipStreamBeginCapture(cs, hipStreamCaptureModeThreadLocal);
    int32_t st = YSCV_HIP_OK;
    if (e == hipSuccess) {
      st = enqueue_step(d, d->batch, cs);
      hipError_t e2 = hipStreamEndCapture(cs, &d->graph);
      if (st == YSCV_HIP_OK && e2 != hipSuccess) e = e2;
    }
    if (st == YSCV_HIP_OK && e == hipSuccess) e = hipGraphInstantiate(&d->graph_exec, d->graph, nullptr, nullptr, 0);
    (void)hipStreamDestroy(cs);
    if (st != YSCV_HIP_OK) return st;
    if (e != hipSuccess) return set_error(YSCV_HIP_ERR_DEVICE, "graph capture failed: %s", hipGetErrorString(e));
    d->graph_batch = d->batch;
  }
  for (int i = 0; i < n_steps; i++) DEC_HIP(hipGraphLaunch(d->graph_exec, s));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_run_projections(yscv_hip_decoder *d, int32_t n_steps, void *stream) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  YSCV_REQUIRE(d->finalized, "decoder weights are not finalized");
  YSCV_REQUIRE(d->batch >= 1, "call yscv_hip_decoder_reset first");
  hipStream_t s = as_stream(stream);
  const int batch = d->batch;
  const auto &c = d->cfg;
  for (int i = 0; i < n_steps; i++) {
    // the same calls as in a real step, folded norms included (their partial sums are whatever the buffers hold)
    int cur = 0, cnt = 1;
    auto consumer = [&](NormFold &nf, bool feeds_update) {
      nf.ss_in = d->ss[cur];
      nf.pre_in = d->pre[cur];
      nf.pre_next = feeds_update ? d->pre[cur ^ 1] : nullptr;
      nf.ss_in_count = cnt;
      nf.ss_in_stride = d->ss_stride;
      nf.inv_d = 1.0f / (float)c.d_model;
      nf.eps = c.rms_eps;
    };
    auto producer = [&](NormFold &nf, const float *gamma, int *count_out) {
      nf.gamma_next = gamma;
      nf.pre = d->pre[cur ^ 1];
      nf.xg = d->xn;
      nf.ss_out = d->ss[cur ^ 1];
      nf.ss_out_stride = d->ss_stride;
      nf.ss_out_count = count_out;
    };
    for (size_t li = 0; li < d->layers.size(); li++) {
      auto &L = d->layers[li];
      NormFold cq, po, cg, pd;
      int n_o = 0, n_d = 0;
      if (d->fold_norm) consumer(cq, true);
      YSCV_TRY(int4_run_ws(L.wqkv, d->xn, YSCV_HIP_F16, d->qkv, YSCV_HIP_F16, batch, 1, EPI_STORE, d->ws, d->ws_bytes, s,
                           d->fold_norm ? &cq : nullptr));
      if (d->fold_norm) producer(po, L.ffn_norm, &n_o);
      YSCV_TRY(int4_run_ws(L.wo, d->ao, YSCV_HIP_F16, d->h, YSCV_HIP_F32, batch, 1, EPI_ADD_F32, d->ws, d->ws_bytes, s,
                           d->fold_norm ? &po : nullptr));
      if (d->fold_norm) {
        cur ^= 1;
        cnt = n_o;
        consumer(cg, true);
      }
      YSCV_TRY(int4_run_ws(L.wgu, d->xn, YSCV_HIP_F16, d->act, YSCV_HIP_F16, batch, 1, EPI_SWIGLU, d->ws, d->ws_bytes, s,
                           d->fold_norm ? &cg : nullptr));
      if (d->fold_norm) producer(pd, li + 1 < d->layers.size() ? d->layers[li + 1].attn_norm : d->final_norm, &n_d);
      YSCV_TRY(int4_run_ws(L.wdown, d->act, YSCV_HIP_F16, d->h, YSCV_HIP_F32, batch, 1, EPI_ADD_F32, d->ws, d->ws_bytes, s,
                           d->fold_norm ? &pd : nullptr));
      if (d->fold_norm) {
        cur ^= 1;
        cnt = n_d;
      }
    }
    NormFold cl;
    if (d->fold_norm) consumer(cl, false);
    YSCV_TRY(int4_run_ws(d->lm_head, d->xn, YSCV_HIP_F16, d->logits, YSCV_HIP_F32, batch, 1, EPI_STORE, d->ws, d->ws_bytes, s,
                         d->fold_norm ? &cl : nullptr));
  }
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_read_tokens(yscv_hip_decoder *d, int32_t first_step, int32_t n_steps, int32_t *out_host) {
  YSCV_REQUIRE(d && out_host, "null argument");
  YSCV_REQUIRE(first_step >= 0 && n_steps >= 0 && first_step + n_steps <= d->cfg.max_steps, "step range out of bounds");
  DEC_HIP(hipDeviceSynchronize());
  YSCV_TRY(check_persist_abort(d));
  DEC_HIP(hipMemcpy(out_host, d->history + (size_t)first_step * d->batch, (size_t)n_steps * d->batch * 4,
                    hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_read_logits(yscv_hip_decoder *d, float *out_host) {
  YSCV_REQUIRE(d && out_host, "null argument");
  DEC_HIP(hipDeviceSynchronize());
  YSCV_TRY(check_persist_abort(d));
  DEC_HIP(hipMemcpy(out_host, d->logits, (size_t)d->batch * d->cfg.vocab * 4, hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_read_activation(yscv_hip_decoder *d, int32_t which, float *out_host, size_t capacity) {
  YSCV_REQUIRE(d && out_host, "null argument");
  YSCV_REQUIRE(d->batch >= 1, "call yscv_hip_decoder_reset first");
  const auto &c = d->cfg;
  const size_t B = (size_t)d->batch;
  const size_t qkv_n = (size_t)(c.n_heads + 2 * c.n_kv_heads) * c.head_dim;
  const void *src = nullptr;
  size_t elems = 0;
  bool half = true;
  switch (which) {
    case YSCV_HIP_DEC_ACT_RESIDUAL: src = d->h; elems = B * c.d_model; half = false; break;
    case YSCV_HIP_DEC_ACT_NORMED: src = d->xn; elems = B * c.d_model; break;
    case YSCV_HIP_DEC_ACT_QKV: src = d->qkv; elems = B * qkv_n; break;
    case YSCV_HIP_DEC_ACT_ATTN_OUT: src = d->ao; elems = B * (size_t)c.n_heads * c.head_dim; break;
    case YSCV_HIP_DEC_ACT_FFN: src = d->act; elems = B * (size_t)c.d_ff; break;
    default: return set_error(YSCV_HIP_ERR_INVALID_ARG, "unknown activation buffer %d", which);
  }
  YSCV_REQUIRE(capacity >= elems, "output holds %zu values, the buffer has %zu", capacity, elems);
  DEC_HIP(hipDeviceSynchronize());
  if (!half) {
    DEC_HIP(hipMemcpy(out_host, src, elems * 4, hipMemcpyDeviceToHost));
    return YSCV_HIP_OK;
  }
  std::vector<_Float16> tmp(elems);
  DEC_HIP(hipMemcpy(tmp.data(), src, elems * 2, hipMemcpyDeviceToHost));
  if (which == YSCV_HIP_DEC_ACT_QKV && d->fused_attn) {
    // the fused attention kernel rotates q on the fly and leaves the buffer unrotated: report the rotated copy
    const size_t qn = (size_t)c.n_heads * c.head_dim;
    for (size_t b = 0; b < B; b++)
      DEC_HIP(hipMemcpy(tmp.data() + b * qkv_n, d->qrot + b * qn, qn * 2, hipMemcpyDeviceToHost));
  }
  for (size_t i = 0; i < elems; i++) out_host[i] = (float)tmp[i];
  if (which == YSCV_HIP_DEC_ACT_NORMED && d->fold_norm && d->last_ss_count > 0) {
    // folded norm: the buffer holds fp16(h * gamma * pre[row]); what the consumer multiplied by its weights is that
    // times the row factor it worked out from the partial sums of squares and pre[row]
    std::vector<float> ss((size_t)B * d->ss_stride), pre(B);
    DEC_HIP(hipMemcpy(ss.data(), d->ss[d->last_ss], ss.size() * 4, hipMemcpyDeviceToHost));
    DEC_HIP(hipMemcpy(pre.data(), d->pre[d->last_ss], B * 4, hipMemcpyDeviceToHost));
    for (size_t b = 0; b < B; b++) {
      float t = 0.0f;
      for (int j = 0; j < d->last_ss_count; j++) t += ss[b * d->ss_stride + j];
      const float f = 1.0f / (pre[b] * std::sqrt(t / (float)c.d_model + c.rms_eps));
      for (size_t i = 0; i < (size_t)c.d_model; i++) out_host[b * c.d_model + i] *= f;
    }
  }
  return YSCV_HIP_OK;
}

#if defined(YSCV_PERSIST_TRACE) && YSCV_PERSIST_TRACE
// Performance builds only (not declared in the public header): the stage timestamps of the last single-launch run,
// [workgroups][layers][PERSIST_TRACE_SLOTS] ticks of the 100 MHz wall clock.
__attribute__((visibility("default"))) int32_t yscv_hip_debug_persist_trace(yscv_hip_decoder *d, unsigned long long *out, size_t capacity,
                                                                           int32_t *workgroups, int32_t *slots) {
  YSCV_REQUIRE(d && out && d->p_trace, "no trace buffer");
  const size_t n = (size_t)d->pm.G * d->cfg.n_layers * PERSIST_TRACE_SLOTS;
  YSCV_REQUIRE(capacity >= n, "trace needs %zu entries", n);
  DEC_HIP(hipDeviceSynchronize());
  DEC_HIP(hipMemcpy(out, d->p_trace, n * 8, hipMemcpyDeviceToHost));
  *workgroups = d->pm.G;
  *slots = PERSIST_TRACE_SLOTS;
  return YSCV_HIP_OK;
}
#endif

int32_t yscv_hip_decoder_debug_set_tag_epoch(yscv_hip_decoder *d, uint32_t epoch) {
  YSCV_REQUIRE(d != nullptr && epoch >= 1, "null decoder or epoch 0");
  d->epoch = epoch;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_debug_set_fused_attention(yscv_hip_decoder *d, int32_t on) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  drop_graph(d);  // a captured step holds the launches of the other variant
  d->fused_attn = on != 0;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_debug_set_folded_norm(yscv_hip_decoder *d, int32_t on) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  drop_graph(d);
  d->fold_norm_wanted = on != 0;
  if (d->finalized) YSCV_TRY(finish_setup(d));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_set_qkv_bias(yscv_hip_decoder *d, int32_t layer, const uint16_t *bias_f16) {
  YSCV_REQUIRE(d != nullptr, "null decoder");
  const auto &c = d->cfg;
  YSCV_REQUIRE(layer >= 0 && layer < c.n_layers, "layer %d out of range", layer);
  auto &L = d->layers[layer];
  drop_graph(d);
  const size_t n = (size_t)(c.n_heads + 2 * c.n_kv_heads) * c.head_dim;
  if (!bias_f16) {
    (void)hipFree(L.qkv_bias);
    L.qkv_bias = nullptr;
  } else {
    if (!L.qkv_bias) DEC_HIP(hipMalloc(reinterpret_cast<void **>(&L.qkv_bias), n * 2));
    DEC_HIP(hipMemcpy(L.qkv_bias, bias_f16, n * 2, hipMemcpyHostToDevice));
  }
  d->has_bias = false;
  for (auto &l : d->layers) d->has_bias = d->has_bias || l.qkv_bias != nullptr;
  return YSCV_HIP_OK;
}

// The prompt pass: every projection sees all rows at once (the MFMA GEMM above 16 rows), attention is causal over the
// cache, and only the last row goes through the final norm and the LM head.
static int32_t prefill_chunk(yscv_hip_decoder *d, const int32_t *tokens_dev, int rows, int start_pos, bool last, hipStream_t s) {
  const auto &c = d->cfg;
  const size_t R = (size_t)rows, D = c.d_model, hq = (size_t)c.n_heads * c.head_dim;
  const size_t qkv_n = (size_t)(c.n_heads + 2 * c.n_kv_heads) * c.head_dim, ff = c.d_ff;
  StreamBuf h, xn, qkv, ao, act;
  YSCV_TRY(h.alloc(R * D * 4, s));
  YSCV_TRY(xn.alloc(R * D * 2, s));
  YSCV_TRY(qkv.alloc(R * qkv_n * 2, s));
  YSCV_TRY(ao.alloc(R * hq * 2, s));
  YSCV_TRY(act.alloc(R * ff * 2, s));
  const bool i8 = d->kv_dtype == YSCV_HIP_KV_I8;
  const int t_ctx = (start_pos + rows + 31) / 32 * 32;
  StreamBuf tk, tv;
  if (i8) {
    YSCV_TRY(tk.alloc((size_t)c.n_kv_heads * t_ctx * c.head_dim * 2, s));
    YSCV_TRY(tv.alloc((size_t)c.n_kv_heads * t_ctx * c.head_dim * 2, s));
  }
  // one scratch for all projections of the pass (prepared activations are not needed: the rows are fp16 already; what
  // remains are the K-split partial sums of the short-prompt shapes)
  size_t ws_bytes = 0;
  for (const yscv_hip_int4_weight *w : {d->layers[0].wqkv, d->layers[0].wo, d->layers[0].wgu, d->layers[0].wdown}) {
    size_t b = 0;
    YSCV_TRY(int4_workspace_bytes(w, R, YSCV_HIP_F16, 0, &b));
    ws_bytes = b > ws_bytes ? b : ws_bytes;
  }
  StreamBuf pws;
  if (ws_bytes > 0) YSCV_TRY(pws.alloc(ws_bytes, s));
  YSCV_TRY(launch_embed(tokens_dev, d->emb, rows, (int)D, c.vocab, h.as<float>(), s));
  for (auto &L : d->layers) {
    YSCV_TRY(launch_rmsnorm(h.as<float>(), L.attn_norm, rows, (int)D, c.rms_eps, xn.as<_Float16>(), s));
    YSCV_TRY(int4_run_ws(L.wqkv, xn.p, YSCV_HIP_F16, qkv.p, YSCV_HIP_F16, R, 0, EPI_STORE, pws.p, ws_bytes, s));
    if (L.qkv_bias) YSCV_TRY(launch_bias_add_f16(qkv.as<_Float16>(), L.qkv_bias, R, qkv_n, s));
    if (i8) {
      // the quantised append, and attention over what the int8 cache returns for every position so far (fp16 scratch)
      YSCV_TRY(launch_prefill_rope_append_i8(qkv.as<_Float16>(), rows, start_pos, c.n_heads, c.n_kv_heads, c.head_dim, c.rope_theta,
                                             c.max_ctx, L.kc8, L.ks, L.vc8, L.vs, t_ctx, tk.as<_Float16>(), tv.as<_Float16>(), s));
      YSCV_TRY(launch_gqa_cache(qkv.as<_Float16>(), tk.as<_Float16>(), tv.as<_Float16>(), nullptr, rows, start_pos, c.n_heads,
                                c.n_kv_heads, c.head_dim, t_ctx, ao.as<_Float16>(), s));
    } else {
      YSCV_TRY(launch_prefill_rope_append(qkv.as<_Float16>(), rows, start_pos, c.n_heads, c.n_kv_heads, c.head_dim, c.rope_theta,
                                          c.max_ctx, L.kc, L.vc, s));
      YSCV_TRY(launch_gqa_cache(qkv.as<_Float16>(), L.kc, L.vc, nullptr, rows, start_pos, c.n_heads, c.n_kv_heads, c.head_dim,
                                c.max_ctx, ao.as<_Float16>(), s));
    }
    // the residual update and SwiGLU ride on the projections' epilogues (both kernels have them: the skinny kernel up to
    // 16 rows, the LDS-ring GEMM above)
    YSCV_TRY(int4_run_ws(L.wo, ao.p, YSCV_HIP_F16, h.p, YSCV_HIP_F32, R, 0, EPI_ADD_F32, pws.p, ws_bytes, s));
    YSCV_TRY(launch_rmsnorm(h.as<float>(), L.ffn_norm, rows, (int)D, c.rms_eps, xn.as<_Float16>(), s));
    YSCV_TRY(int4_run_ws(L.wgu, xn.p, YSCV_HIP_F16, act.p, YSCV_HIP_F16, R, 0, EPI_SWIGLU, pws.p, ws_bytes, s));
    YSCV_TRY(int4_run_ws(L.wdown, act.p, YSCV_HIP_F16, h.p, YSCV_HIP_F32, R, 0, EPI_ADD_F32, pws.p, ws_bytes, s));
  }
  if (last) {
    YSCV_TRY(launch_rmsnorm(h.as<float>() + (R - 1) * D, d->final_norm, 1, (int)D, c.rms_eps, d->xn, s));
    YSCV_TRY(int4_run_ws(d->lm_head, d->xn, YSCV_HIP_F16, d->logits, YSCV_HIP_F32, 1, 1, EPI_STORE, d->ws, d->ws_bytes, s));
  }
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_prefill(yscv_hip_decoder *d, const int32_t *tokens_host, int32_t n_tokens, int32_t start_pos,
                                 void *stream) {
  YSCV_REQUIRE(d != nullptr && tokens_host != nullptr, "null argument");
  YSCV_REQUIRE(d->finalized, "decoder weights are not finalized");
  const auto &c = d->cfg;
  YSCV_REQUIRE(n_tokens >= 1 && start_pos >= 0, "prefill needs at least one token and a non-negative position");
  YSCV_REQUIRE((int64_t)start_pos + n_tokens <= c.max_ctx, "KV cache overflow: position %d + %d tokens > max_ctx %d", start_pos,
               n_tokens, c.max_ctx);
  for (int32_t i = 0; i < n_tokens; i++)
    YSCV_REQUIRE(tokens_host[i] >= 0 && tokens_host[i] < c.vocab, "token %d outside the vocabulary (%d)", tokens_host[i], c.vocab);
  hipStream_t s = as_stream(stream);
  d->batch = 1;
  StreamBuf toks;
  YSCV_TRY(toks.alloc((size_t)n_tokens * 4, s));
  DEC_HIP(hipMemcpyAsync(toks.p, tokens_host, (size_t)n_tokens * 4, hipMemcpyHostToDevice, s));
  DEC_HIP(hipStreamSynchronize(s));  // tokens_host is the caller's again
  const int chunk = d->prefill_rows;  // rows per pass: bounds the activation buffers
  for (int32_t r0 = 0; r0 < n_tokens; r0 += chunk) {
    const int rows = n_tokens - r0 < chunk ? n_tokens - r0 : chunk;
    YSCV_TRY(prefill_chunk(d, toks.as<int32_t>() + r0, rows, start_pos + r0, r0 + rows == n_tokens, s));
  }
  // as after reset(last token, start_pos + n - 1) + one decode step: the pick is the next input, position and step advance
  hipLaunchKernelGGL(set_counters_kernel, dim3(1), dim3(64), 0, s, d->pos, d->step, start_pos + n_tokens - 1, 0);
  DEC_HIP(hipGetLastError());
  YSCV_TRY(launch_argmax(d->logits, 1, c.vocab, d->tokens, d->history, d->step, c.max_steps, s));
  YSCV_TRY(launch_advance(d->pos, d->step, s));
  d->last_path = 1;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_set_prefill_rows(yscv_hip_decoder *d, int32_t rows) {
  YSCV_REQUIRE(d != nullptr, "null argument");
  YSCV_REQUIRE(rows >= 1 && rows <= 65536, "rows per prompt pass must be in 1 .. 65536, got %d", rows);
  d->prefill_rows = rows;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_last_path(const yscv_hip_decoder *d, int32_t *path) {
  YSCV_REQUIRE(d != nullptr && path != nullptr, "null argument");
  *path = d->last_path;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_vocab(const yscv_hip_decoder *d, size_t *vocab) {
  YSCV_REQUIRE(d && vocab, "null argument");
  *vocab = (size_t)d->cfg.vocab;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_weight_bytes(const yscv_hip_decoder *d, size_t *bytes) {
  YSCV_REQUIRE(d && bytes, "null argument");
  *bytes = d->weight_bytes;
  return YSCV_HIP_OK;
}

}  // extern "C"
