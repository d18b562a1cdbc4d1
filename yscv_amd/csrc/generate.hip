// Host-side sampling loop over the device-resident decoder: the counterpart of generate() / sample_token()
// (crates/yscv-onnx/src/generate.rs:58-208).  The reference re-runs its model on the whole sequence for every
// token; here every token is one decode step against the KV cache, the logits of that step come back to the host
// and the reference's sampler runs on them operation by operation (repetition penalty, temperature, top-k
// threshold, softmax, top-p cut, xorshift64 draw).  Greedy decoding (top_k = 1 with no ties) gives the tokens
// yscv_hip_decoder_run picks on the device.
#include <algorithm>
#include <cmath>
#include <numeric>
#include <vector>

#include "common.hpp"

using namespace yscv;

namespace {

// f32::max(a, b): a NaN operand is ignored
inline float rust_max(float a, float b) { return (b != b) ? a : ((a != a) ? b : (a > b ? a : b)); }

// indices sorted by descending value; incomparable (NaN) pairs count as equal (generate.rs:128-133, 160-165).
// The reference uses an unstable sort, so the order among equal values is unspecified there; a stable sort fixes it
// to ascending index here.
std::vector<size_t> sorted_desc(const float *v, size_t n) {
  std::vector<size_t> idx(n);
  std::iota(idx.begin(), idx.end(), (size_t)0);
  std::stable_sort(idx.begin(), idx.end(), [&](size_t a, size_t b) { return v[a] > v[b]; });
  return idx;
}

}  // namespace

extern "C" {

int32_t yscv_hip_sample_token(float *logits, size_t vocab_size, size_t top_k, float top_p, uint64_t *rng, uint32_t *token_out) {
  YSCV_REQUIRE(logits && rng && token_out, "null argument");
  YSCV_REQUIRE(vocab_size > 0, "empty vocabulary");
  // top-k: everything below the k-th largest logit is removed (generate.rs:125-141)
  if (top_k > 0 && top_k < vocab_size) {
    const std::vector<size_t> order = sorted_desc(logits, vocab_size);
    const float threshold = logits[order[top_k - 1]];
    for (size_t i = 0; i < vocab_size; i++)
      if (logits[i] < threshold) logits[i] = -INFINITY;
  }
  // softmax (generate.rs:143-155)
  float max_val = -INFINITY;
  for (size_t i = 0; i < vocab_size; i++) max_val = rust_max(max_val, logits[i]);
  float sum = 0.0f;
  for (size_t i = 0; i < vocab_size; i++) {
    logits[i] = expf(logits[i] - max_val);
    sum += logits[i];
  }
  if (sum > 0.0f) {
    const float inv = 1.0f / sum;
    for (size_t i = 0; i < vocab_size; i++) logits[i] *= inv;
  }
  // top-p: keep the most probable tokens until their cumulative probability exceeds p (generate.rs:157-186)
  if (top_p < 1.0f) {
    const std::vector<size_t> order = sorted_desc(logits, vocab_size);
    float cumsum = 0.0f;
    for (size_t pos = 0; pos < vocab_size; pos++) {
      cumsum += logits[order[pos]];
      if (cumsum > top_p) {
        for (size_t rest = pos + 1; rest < vocab_size; rest++) logits[order[rest]] = 0.0f;
        break;
      }
    }
    float new_sum = 0.0f;
    for (size_t i = 0; i < vocab_size; i++) new_sum += logits[i];
    if (new_sum > 0.0f) {
      const float inv = 1.0f / new_sum;
      for (size_t i = 0; i < vocab_size; i++) logits[i] *= inv;
    }
  }
  // xorshift64 draw (generate.rs:188-192); `u64 as f32` rounds to nearest, u64::MAX as f32 is 2^64
  uint64_t x = *rng;
  x ^= x << 13;
  x ^= x >> 7;
  x ^= x << 17;
  *rng = x;
  const float u = (float)x / 18446744073709551616.0f;
  float cumsum = 0.0f;
  for (size_t i = 0; i < vocab_size; i++) {
    cumsum += logits[i];
    if (cumsum > u) {
      *token_out = (uint32_t)i;
      return YSCV_HIP_OK;
    }
  }
  // fallback: the most probable token; Iterator::max_by keeps the last of equal maxima (generate.rs:202-207)
  size_t best = 0;
  for (size_t i = 1; i < vocab_size; i++)
    if (!(logits[best] > logits[i])) best = i;
  *token_out = (uint32_t)best;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_decoder_generate(yscv_hip_decoder *d, const uint32_t *input_ids, size_t n_input,
                                  const yscv_hip_generate_config *cfg, uint32_t *generated_out, size_t *n_generated) {
  YSCV_REQUIRE(d && input_ids && cfg && n_generated, "null argument");
  YSCV_REQUIRE(n_input > 0, "empty prompt");
  YSCV_REQUIRE(cfg->max_tokens == 0 || generated_out != nullptr, "null output buffer");
  *n_generated = 0;
  size_t vocab = 0;
  YSCV_TRY(yscv_hip_decoder_vocab(d, &vocab));
  std::vector<uint32_t> tokens(input_ids, input_ids + n_input);
  std::vector<float> logits(vocab);
  uint64_t rng_state = 0xdeadbeefULL;  // generate.rs:68
  // the prompt goes through the decoder in one pass (yscv_hip_decoder_prefill: every projection sees all positions at
  // once); the KV cache then holds positions 0 .. n_input-1 and the logits are those of the last prompt position
  {
    std::vector<int32_t> prompt(n_input);
    for (size_t p = 0; p < n_input; p++) {
      YSCV_REQUIRE(input_ids[p] < vocab, "prompt token %u outside the vocabulary (%zu)", input_ids[p], vocab);
      prompt[p] = (int32_t)input_ids[p];
    }
    YSCV_REQUIRE(n_input < ((size_t)1 << 31), "prompt too long");
    YSCV_TRY(yscv_hip_decoder_prefill(d, prompt.data(), (int32_t)n_input, 0, nullptr));
  }
  for (size_t g = 0; g < cfg->max_tokens; g++) {
    YSCV_TRY(yscv_hip_decoder_read_logits(d, logits.data()));
    if (cfg->repetition_penalty != 1.0f) {  // generate.rs:80-92
      for (uint32_t t : tokens) {
        if (t < logits.size()) {
          if (logits[t] > 0.0f) logits[t] /= cfg->repetition_penalty;
          else logits[t] *= cfg->repetition_penalty;
        }
      }
    }
    if (cfg->temperature != 1.0f && cfg->temperature > 0.0f) {  // generate.rs:95-100
      const float inv_temp = 1.0f / cfg->temperature;
      for (float &v : logits) v *= inv_temp;
    }
    uint32_t next = 0;
    YSCV_TRY(yscv_hip_sample_token(logits.data(), vocab, cfg->top_k, cfg->top_p, &rng_state, &next));
    if (cfg->has_eos && cfg->eos_token_id == next) break;
    generated_out[(*n_generated)++] = next;
    tokens.push_back(next);
    if (g + 1 == cfg->max_tokens) break;
    const int32_t tok = (int32_t)next;
    YSCV_TRY(yscv_hip_decoder_reset(d, 1, (int32_t)(tokens.size() - 1), &tok));
    YSCV_TRY(yscv_hip_decoder_run(d, 1, YSCV_HIP_DECODE_AUTO, nullptr));
  }
  return YSCV_HIP_OK;
}

}  // extern "C"
