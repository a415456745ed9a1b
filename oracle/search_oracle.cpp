// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// CPU restatement of the onnxruntime-genai per-step search & sampling path, used only as the
// checker by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py.  Nothing in the
// shipped library links, loads or calls this file.
//
// Every function cites the reference source it restates (paths relative to the reference tree).
// Differences from the reference, all deliberate:
//   * Random draws are explicit arguments.  A categorical draw takes the double `u` that libstdc++'s
//     std::discrete_distribution would obtain from generate_canonical<double,53>; an accept test
//     takes the float `u` of std::uniform_real_distribution<float>(0,1).
//   * Ties between equal scores are broken towards the lowest index everywhere (the reference leaves
//     the order of equal elements to std::partial_sort).  NaN scores order below every number.
//   * DeviceSpan/GeneratorParams plumbing is replaced by plain pointers and sizes.
//
// Pinning status (what independently checks each function is listed in tests/test_oracle_*.py):
//   argmax, penalties, mask, sampled categorical (top-k and nucleus), discrete draw, softmax family,
//   accept/correction math: pinned by the reference's own known-answer tests and, where it builds,
//   by oracle/_ref (the unmodified reference headers compiled from /root/reference).
//   the accept loops (sparse and dense): pinned as whole rounds on the reference's own functions driven by a
//   real std::mt19937 (oracle/_ref); the dense one through selections that list the whole vocabulary.
//   beam top-2B selection: pinned by brute force (full stable sort) on small inputs.
//   argmax, BeamSearch_Cpu::SelectTop, BeamSearchScorer::Process (candidates that are not EOS), Finalize,
//   GetBeamHypotheses and the beam sequence append: pinned by the reference's own golden generations
//   (ModelTests.GreedySearchGptFp32 / BeamSearchGptFp32, test/model_tests.cpp:57-130), replayed from
//   the logits of the tiny GPT-2 those tests load (tests/golden/gpt2_search_vectors.npz).
//   BeamSearchScorer's EOS branch (BeamHypotheses::Add / CanImprove, done batches, padding, the
//   done window's offset): no EOS is produced in those golden runs; pinned by hand-worked cases
//   with literal expected values derived from the reference source (tests/beam_scorer_cases.py,
//   tests/test_beam_scorer_handworked.py), each of sixteen one-line mistakes patched into this file
//   failing at least one of them.
//   KV gather: pinned by numpy.take.
//   Cast conversions (fp16/bf16 <-> fp32, int32 -> int64): pinned by known answers and, for
//   fp32 -> fp16, by agreement with IEEE round-to-nearest on every value that is not an exact tie
//   (the reference file, src/models/utils.cpp, does not build without ONNX Runtime headers).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <numeric>
#include <vector>

namespace {

constexpr float kLowest = std::numeric_limits<float>::lowest();

// Order-preserving integer image of a float: larger key <=> larger score.  -0 and +0 share a key
// (the reference compares floats, so they tie); NaN maps below everything.
inline uint32_t OrderKey(float f) {
  if (f != f) return 0u;
  if (f == 0.0f) f = 0.0f + 0.0f;  // canonical +0
  uint32_t b;
  std::memcpy(&b, &f, 4);
  if (b == 0x80000000u) b = 0;
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// "a ranks before b": score descending, then index ascending.
struct RankBefore {
  const float* s;
  bool operator()(int32_t a, int32_t b) const {
    const uint32_t ka = OrderKey(s[a]), kb = OrderKey(s[b]);
    return ka > kb || (ka == kb && a < b);
  }
};

// libstdc++ std::discrete_distribution<int>(probs)(urng) with the canonical draw made explicit
// (/usr/include/c++/11/bits/random.tcc: param_type::_M_initialize and operator()).
// Fewer than two weights: returns 0 and would consume no draw.
int DiscreteDraw(const float* w, int n, double u) {
  if (n < 2) return 0;
  std::vector<double> prob(w, w + n);
  const double sum = std::accumulate(prob.begin(), prob.end(), 0.0);
  for (auto& v : prob) v /= sum;
  std::vector<double> cp;
  cp.reserve(n);
  std::partial_sum(prob.begin(), prob.end(), std::back_inserter(cp));
  cp[n - 1] = 1.0;
  return static_cast<int>(std::lower_bound(cp.begin(), cp.end(), u) - cp.begin());
}

// src/sampling_distribution.h:139-206 FindNucleus.
int FindNucleus(const float* scores, int vocab_size, int32_t* indices, float p, float max_score,
                float inv_temp) {
  constexpr int kInitial = 16, kGrowth = 4;
  std::iota(indices, indices + vocab_size, 0);
  RankBefore before{scores};
  int sorted_count = 0;
  int k = std::min(kInitial, vocab_size);
  float prefix_exp_sum = 0.0f;
  int cutoff_index = 0;
  while (k <= vocab_size) {
    std::partial_sort(indices + sorted_count, indices + k, indices + vocab_size, before);
    cutoff_index = k;
    for (int i = sorted_count; i < k; ++i) {
      const float exp_i = std::exp((scores[indices[i]] - max_score) * inv_temp);
      prefix_exp_sum += exp_i;
      const float tail_bound = static_cast<float>(vocab_size - i - 1) * exp_i;
      if (prefix_exp_sum >= p * (prefix_exp_sum + tail_bound)) {
        cutoff_index = i + 1;
        break;
      }
    }
    sorted_count = k;
    if (cutoff_index < k || k == vocab_size) break;
    k = std::min(k * kGrowth, vocab_size);
  }
  if (vocab_size <= kInitial * kGrowth) {
    if (sorted_count < vocab_size)
      std::partial_sort(indices + sorted_count, indices + vocab_size, indices + vocab_size, before);
    float global_exp_sum = 0.0f;
    for (int i = 0; i < vocab_size; ++i)
      global_exp_sum += std::exp((scores[indices[i]] - max_score) * inv_temp);
    float cum = 0.0f;
    for (int i = 0; i < vocab_size; ++i) {
      cum += std::exp((scores[indices[i]] - max_score) * inv_temp);
      if (cum >= p * global_exp_sum) return i + 1;
    }
  }
  return cutoff_index;
}

}  // namespace

extern "C" {

// ---- a2: src/search.h:9-29 ArgMax (strict '>' keeps the first maximum; a NaN only wins at index 0).
int32_t orc_argmax(const float* v, int n) {
  int32_t best = 0;
  float best_score = v[0];
  for (int i = 1; i < n; ++i)
    if (v[i] > best_score) {
      best_score = v[i];
      best = i;
    }
  return best;
}

// ---- a3: src/sampling_distribution.h:26-35 ApplyMinLengthToLogits.
void orc_apply_min_length(float* logits, int vocab, int current_length, int min_length,
                          const int32_t* eos, int n_eos) {
  if (current_length >= min_length) return;
  for (int i = 0; i < n_eos; ++i)
    if (eos[i] >= 0 && eos[i] < vocab) logits[eos[i]] = kLowest;
}

// ---- a4: src/sampling_distribution.h:41-62 ApplyRepetitionPenaltyToLogits (once per distinct id).
void orc_apply_repetition_penalty(float* logits, int vocab, const int32_t* prefix, int n,
                                  float penalty) {
  if (penalty == 1.0f) return;
  std::vector<bool> visited(static_cast<size_t>(vocab), false);
  for (int i = 0; i < n; ++i) {
    const int32_t w = prefix[i];
    if (w >= 0 && w < vocab && !visited[w]) {
      visited[w] = true;
      const float score = logits[w];
      logits[w] = (score < 0 ? score * penalty : score / penalty);
    }
  }
}

// ---- a5: src/sampling_distribution.h:64-79 ApplyNoRepeatNgramToLogits.
void orc_apply_no_repeat_ngram(float* logits, int vocab, const int32_t* prefix, int n, int ngram) {
  if (ngram <= 0 || n < ngram) return;
  const int plen = ngram - 1;
  const int32_t* target = prefix + (n - plen);
  const int last_start = n - ngram;
  for (int start = 0; start <= last_start; ++start) {
    if (std::equal(target, target + plen, prefix + start)) {
      const int32_t banned = prefix[start + plen];
      if (banned >= 0 && banned < vocab) logits[banned] = kLowest;
    }
  }
}

// ---- a6: src/constrained_logits_processor.cpp:246-258 (bit set = token allowed; row stride
// (vocab-1)/32+1 words, :174-183).
void orc_apply_mask(float* logits, int rows, int vocab, const uint32_t* mask) {
  const size_t words = static_cast<size_t>((vocab - 1) / 32 + 1);
  for (int r = 0; r < rows; ++r) {
    float* row = logits + static_cast<size_t>(r) * vocab;
    const uint32_t* m = mask + r * words;
    for (int i = 0; i < vocab; ++i)
      row[i] = (m[i / 32] & (uint32_t{1} << (i % 32))) ? row[i] : kLowest;
  }
}

// ---- a7/a8: src/sampling_distribution.h:233-297 ComputeSampledCategorical.
// indices/probs need room for min(top_k, vocab) (top-k branch) or vocab (nucleus branch) entries;
// scratch needs vocab entries.  Returns the kept count.
int orc_sampled_categorical(const float* scores, int vocab, int top_k, float top_p,
                            float temperature, int32_t* scratch, int32_t* indices, float* out_probs) {
  const float inv_temp = 1.0f / temperature;
  const bool apply_topk = top_k > 1;
  const bool apply_topp = top_p > 0.0f && top_p < 1.0f;
  if (apply_topk) {
    const int m = std::min(top_k, vocab);
    std::iota(scratch, scratch + vocab, 0);
    std::partial_sort(scratch, scratch + m, scratch + vocab, RankBefore{scores});
    const float max_score = scores[scratch[0]];
    std::vector<float> probs(m);
    float sum = 0.0f;
    for (int j = 0; j < m; j++) {
      probs[j] = std::exp((scores[scratch[j]] - max_score) * inv_temp);
      sum += probs[j];
    }
    if (sum > 0.0f)
      for (auto& v : probs) v /= sum;
    int keep = m;
    if (apply_topp) {
      float cum = 0.0f;
      for (int j = 0; j < m; j++) {
        cum += probs[j];
        if (cum >= top_p) {
          keep = j + 1;
          break;
        }
      }
    }
    float keep_sum = 0.0f;
    for (int j = 0; j < keep; j++) keep_sum += probs[j];
    const float inv = keep_sum > 0.0f ? 1.0f / keep_sum : 0.0f;
    for (int j = 0; j < keep; j++) {
      indices[j] = scratch[j];
      out_probs[j] = probs[j] * inv;
    }
    return keep;
  }
  // std::max_element with operator<: the first maximum; NaNs never replace the running maximum.
  float max_score = scores[0];
  for (int i = 1; i < vocab; ++i)
    if (max_score < scores[i]) max_score = scores[i];
  const int cutoff = FindNucleus(scores, vocab, scratch, top_p, max_score, inv_temp);
  std::vector<float> probs(cutoff);
  float sum = 0.0f;
  for (int j = 0; j < cutoff; j++) {
    probs[j] = std::exp((scores[scratch[j]] - max_score) * inv_temp);
    sum += probs[j];
  }
  const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
  for (int j = 0; j < cutoff; j++) {
    indices[j] = scratch[j];
    out_probs[j] = probs[j] * inv;
  }
  return cutoff;
}

// ---- a9: src/sampling_distribution.h:218-227 SampleCategoricalToken with the draw made explicit.
int orc_discrete_draw(const float* weights, int n, double u) { return DiscreteDraw(weights, n, u); }

// One row of GreedySearch_Cpu::SampleTopK / SampleTopP / SampleTopKTopP (src/search.cpp:203-254):
// build the kept distribution, draw.  kept_* may be null.
int32_t orc_sample_row(const float* scores, int vocab, int top_k, float top_p, float temperature,
                       double u, int32_t* scratch, int32_t* kept_idx, float* kept_probs,
                       int* kept_count) {
  std::vector<int32_t> idx_local;
  std::vector<float> probs_local;
  const int cap = top_k > 1 ? std::min(top_k, vocab) : vocab;
  if (!kept_idx) {
    idx_local.resize(cap);
    kept_idx = idx_local.data();
  }
  if (!kept_probs) {
    probs_local.resize(cap);
    kept_probs = probs_local.data();
  }
  const int keep =
      orc_sampled_categorical(scores, vocab, top_k, top_p, temperature, scratch, kept_idx, kept_probs);
  if (kept_count) *kept_count = keep;
  return kept_idx[DiscreteDraw(kept_probs, keep, u)];
}

// Serial loop over rows, as GreedySearch_Cpu::SampleTop* does (src/search.cpp:207,224,243).
// k>1 && 0<p<1: top-k+top-p; k>1: top-k; else nucleus.
void orc_sample_batch(const float* logits, int rows, int vocab, int top_k, float top_p,
                      float temperature, const double* u, int32_t* tokens) {
  std::vector<int32_t> scratch(static_cast<size_t>(vocab));
  for (int r = 0; r < rows; ++r)
    tokens[r] = orc_sample_row(logits + static_cast<size_t>(r) * vocab, vocab, top_k, top_p,
                               temperature, u[r], scratch.data(), nullptr, nullptr, nullptr);
}

// GreedySearch_Cpu::SelectTop over rows (src/search.cpp:178-192) without the EOS bookkeeping.
void orc_argmax_batch(const float* logits, int rows, int vocab, int32_t* tokens) {
  for (int r = 0; r < rows; ++r) tokens[r] = orc_argmax(logits + static_cast<size_t>(r) * vocab, vocab);
}

// ---- a11: src/softmax.h:9-47 and src/softmax_cpu.cpp:5-31.
void orc_softmax(float* s, int n, float temperature) {
  float max_score = s[0];
  for (int i = 1; i < n; ++i)
    if (max_score < s[i]) max_score = s[i];
  const float inv_temp = 1.0f / temperature;
  float exp_sum = 0.0f;
  for (int i = 0; i < n; ++i) {
    s[i] = std::exp((s[i] - max_score) * inv_temp);
    exp_sum += s[i];
  }
  if (exp_sum > 0.0f) {
    const float inv_sum = 1.0f / exp_sum;
    for (int i = 0; i < n; ++i) s[i] *= inv_sum;
  }
}

void orc_log_softmax(float* s, int n, float temperature) {
  float max_score = s[0];
  for (int i = 1; i < n; ++i)
    if (max_score < s[i]) max_score = s[i];
  const float inv_temp = 1.0f / temperature;
  float exp_sum = 0.0f;
  for (int i = 0; i < n; ++i) {
    s[i] = (s[i] - max_score) * inv_temp;
    exp_sum += std::exp(s[i]);
  }
  const float log_sum_exp = std::log(exp_sum);
  for (int i = 0; i < n; ++i) s[i] -= log_sum_exp;
}

void orc_softmax_plain(float* v, int n) {
  float mx = *std::max_element(v, v + n);
  float sum = 0.0f;
  for (int i = 0; i < n; ++i) {
    v[i] = std::exp(v[i] - mx);
    sum += v[i];
  }
  if (sum > 0.0f) {
    const float inv = 1.0f / sum;
    for (int i = 0; i < n; ++i) v[i] *= inv;
  }
}

void orc_log_softmax_plain(float* v, int n) {
  float mx = *std::max_element(v, v + n);
  float sum = 0.0f;
  for (int i = 0; i < n; ++i) {
    v[i] -= mx;
    sum += std::exp(v[i]);
  }
  const float log_sum = std::log(sum);
  for (int i = 0; i < n; ++i) v[i] -= log_sum;
}

// src/models/utils.cpp:103-109 FastFloat16ToFloat32 (fp16 Inf/NaN become finite, as there).
float orc_fp16_to_fp32(uint16_t x) {
  const uint32_t e = (x & 0x7C00u) >> 10;
  const uint32_t m = (x & 0x03FFu) << 13;
  const float mf = static_cast<float>(m);
  uint32_t mbits;
  std::memcpy(&mbits, &mf, 4);
  const uint32_t v = mbits >> 23;
  const uint32_t bits = (static_cast<uint32_t>(x & 0x8000u) << 16) |
                        (e != 0) * ((e + 112) << 23 | m) |
                        ((e == 0) & (m != 0)) * ((v - 37) << 23 | ((m << (150 - v)) & 0x007FE000u));
  float out;
  std::memcpy(&out, &bits, 4);
  return out;
}

// src/models/utils.cpp:111-118 FastFloat32ToFloat16.
uint16_t orc_fp32_to_fp16(float v) {
  uint32_t bits;
  std::memcpy(&bits, &v, 4);
  const uint32_t b = bits + 0x00001000u;
  const uint32_t e = (b & 0x7F800000u) >> 23;
  const uint32_t m = b & 0x007FFFFFu;
  return static_cast<uint16_t>((b & 0x80000000u) >> 16 | (e > 112) * ((((e - 112) << 10) & 0x7C00u) | m >> 13) |
                               ((e < 113) & (e > 101)) * ((((0x007FF000u + m) >> (125 - e)) + 1) >> 1) |
                               (e > 143) * 0x7FFFu);
}

// src/models/utils.cpp:84-86 BFloat16ToFloat32 = TFloatToFloat32<8, 7> (:55-77).
float orc_bf16_to_fp32(uint16_t v) {
  const uint32_t sign = v >> 15, exponent = (v >> 7) & 0xFFu, fraction = v & 0x7Fu;
  if (exponent == 0) {
    if (fraction == 0) return sign ? -0.0f : 0.0f;
    return std::ldexp((sign ? -1.0f : 1.0f) * static_cast<float>(fraction) / 128.0f, 1 - 127);
  }
  if (exponent == 255) {
    if (fraction == 0) return sign ? -std::numeric_limits<float>::infinity() : std::numeric_limits<float>::infinity();
    return std::numeric_limits<float>::quiet_NaN();
  }
  return std::ldexp((sign ? -1.0f : 1.0f) * (1.0f + static_cast<float>(fraction) / 128.0f), static_cast<int>(exponent) - 127);
}

// src/models/utils.cpp:89-93 Float32ToBFloat16: the most significant 16 bits.
uint16_t orc_fp32_to_bf16(float v) {
  uint32_t bits;
  std::memcpy(&bits, &v, 4);
  return static_cast<uint16_t>(bits >> 16);
}

// DeviceInterface::Cast on the CPU (src/cpu/interface.cpp:74-106); kind as in the device kernel:
// 0 fp16->fp32, 1 bf16->fp32, 2 fp32->fp16, 3 fp32->bf16, 4 int32->int64.
void orc_cast(const void* in, void* out, size_t n, int kind) {
  for (size_t i = 0; i < n; ++i) {
    switch (kind) {
      case 0: static_cast<float*>(out)[i] = orc_fp16_to_fp32(static_cast<const uint16_t*>(in)[i]); break;
      case 1: static_cast<float*>(out)[i] = orc_bf16_to_fp32(static_cast<const uint16_t*>(in)[i]); break;
      case 2: static_cast<uint16_t*>(out)[i] = orc_fp32_to_fp16(static_cast<const float*>(in)[i]); break;
      case 3: static_cast<uint16_t*>(out)[i] = orc_fp32_to_bf16(static_cast<const float*>(in)[i]); break;
      default: static_cast<int64_t*>(out)[i] = static_cast<const int32_t*>(in)[i]; break;
    }
  }
}

void orc_fp16_to_fp32_array(const uint16_t* in, float* out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = orc_fp16_to_fp32(in[i]);
}

// ---- a12: src/search.cpp:101-164 BeamSearch_Cpu::SelectTop up to the scorer call.
// scores [batch*beams, vocab] is modified in place exactly as the reference does (log-softmax, then
// += beam score).  Outputs are [batch, 2*beams].
void orc_beam_select_top(float* scores, int batch, int beams, int vocab, const float* beam_scores,
                         float* out_scores, int32_t* out_tokens, int32_t* out_indices) {
  const int bb = batch * beams;
  for (int i = 0; i < bb; ++i) orc_log_softmax(scores + static_cast<size_t>(i) * vocab, vocab, 1.0f);
  size_t off = 0;
  for (int i = 0; i < bb; ++i)
    for (int k = 0; k < vocab; ++k, ++off) scores[off] += beam_scores[i];
  const int top_k = 2 * beams;
  const size_t total = static_cast<size_t>(beams) * vocab;
  std::vector<int32_t> idx(total);
  for (int b = 0; b < batch; ++b) {
    const float* sub = scores + b * total;
    std::iota(idx.begin(), idx.end(), 0);
    std::partial_sort(idx.begin(), idx.begin() + top_k, idx.end(), RankBefore{sub});
    for (int i = 0; i < top_k; ++i) {
      out_indices[b * top_k + i] = idx[i] / vocab;
      out_tokens[b * top_k + i] = idx[i] % vocab;
      out_scores[b * top_k + i] = sub[idx[i]];
    }
  }
}

// ---- a13: src/beam_search_scorer.{h,cpp}.
struct OrcHypothesis {
  std::vector<int32_t> tokens;
  float score;
};

struct OrcBeamHyps {  // BeamHypotheses, src/beam_search_scorer.cpp:12-44
  std::vector<OrcHypothesis> beams;  // sorted, best first; capacity num_beams
  int capacity{};
  float length_penalty{};
  bool done{};
  void Add(const int32_t* seq, int length, float sum_logprobs) {
    const float score = sum_logprobs / std::pow(static_cast<float>(length), length_penalty);
    size_t index = beams.size();
    if (static_cast<int>(index) == capacity) {
      if (score <= beams[--index].score) return;
    } else {
      beams.emplace_back();
    }
    for (; index > 0 && score > beams[index - 1].score; index--) beams[index] = beams[index - 1];
    beams[index] = OrcHypothesis{std::vector<int32_t>(seq, seq + length), score};
  }
  bool CanImprove(float best_sum_logprobs, int current_length) const {
    const float current = best_sum_logprobs / std::pow(static_cast<float>(current_length), length_penalty);
    return beams.back().score < current;
  }
};

struct OrcBeamScorer {
  int batch, beams, max_length, pad;
  std::vector<int32_t> eos;
  bool early_stopping;
  int not_done;
  std::vector<float> next_scores;
  std::vector<int32_t> next_tokens, next_indices;
  std::vector<OrcBeamHyps> hyps;
  bool IsEos(int32_t t) const { return std::find(eos.begin(), eos.end(), t) != eos.end(); }
};

void* orc_beam_scorer_create(int batch, int beams, int max_length, int pad, const int32_t* eos,
                             int n_eos, float length_penalty, int early_stopping) {
  auto* s = new OrcBeamScorer;
  s->batch = batch;
  s->beams = beams;
  s->max_length = max_length;
  s->pad = pad;
  s->eos.assign(eos, eos + n_eos);
  s->early_stopping = early_stopping != 0;
  s->not_done = batch;
  s->next_scores.assign(static_cast<size_t>(batch) * beams, 0.0f);  // :76-81
  for (int i = 0; i < batch; ++i)
    for (int j = 1; j < beams; ++j) s->next_scores[i * beams + j] = -1e9;
  s->next_tokens.assign(static_cast<size_t>(batch) * beams, 0);
  s->next_indices.assign(static_cast<size_t>(batch) * beams, 0);
  s->hyps.resize(batch);
  for (auto& h : s->hyps) {
    h.capacity = beams;
    h.length_penalty = length_penalty;
    h.done = false;
  }
  return s;
}

void orc_beam_scorer_destroy(void* h) { delete static_cast<OrcBeamScorer*>(h); }

// src/beam_search_scorer.cpp:84-171 Process.  sequences is [batch*beams, max_length] with
// sequence_length valid tokens per row; candidates are [batch, 2*beams].
void orc_beam_scorer_process(void* h, const int32_t* sequences, int sequence_length,
                             const float* cand_scores, const int32_t* cand_tokens,
                             const int32_t* cand_indices) {
  auto& s = *static_cast<OrcBeamScorer*>(h);
  const int nb = s.beams, top_k = 2 * nb;
  for (int batch = 0; batch < s.batch; ++batch) {
    auto& hyp = s.hyps[batch];
    if (hyp.done) {
      for (int j = 0; j < nb; ++j) {
        s.next_scores[batch * nb + j] = 0.0f;
        s.next_tokens[batch * nb + j] = s.pad;
        s.next_indices[batch * nb + j] = 0;
      }
      continue;
    }
    int beam_idx = 0;
    for (int j = 0; j < top_k; ++j) {
      const int32_t tok = cand_tokens[batch * top_k + j];
      const float score = cand_scores[batch * top_k + j];
      const int32_t bidx = cand_indices[batch * top_k + j];
      const int batch_beam_idx = batch * nb + bidx;
      if (s.IsEos(tok)) {
        if (j >= nb) continue;
        hyp.Add(sequences + static_cast<size_t>(batch_beam_idx) * s.max_length, sequence_length, score);
      } else {
        s.next_scores[batch * nb + beam_idx] = score;
        s.next_tokens[batch * nb + beam_idx] = tok;
        s.next_indices[batch * nb + beam_idx] = batch_beam_idx;
        ++beam_idx;
      }
      if (beam_idx == nb) break;
    }
    if (static_cast<int>(hyp.beams.size()) < nb) continue;
    if (!s.early_stopping) {
      // The window starts at batch*num_beams, not batch*2*num_beams (:161); reproduced as is.
      const float* w = cand_scores + batch * nb;
      const float best = *std::max_element(w, w + top_k);
      if (hyp.CanImprove(best, sequence_length)) continue;
    }
    hyp.done = true;
    s.not_done--;
  }
}

// src/beam_search_scorer.cpp:173-196 Finalize.
void orc_beam_scorer_finalize(void* h, const int32_t* sequences, int sequence_length) {
  auto& s = *static_cast<OrcBeamScorer*>(h);
  for (int b = 0; b < s.batch; ++b) {
    auto& hyp = s.hyps[b];
    if (hyp.done) continue;
    for (int j = 0; j < s.beams; ++j) {
      const int bbi = b * s.beams + j;
      hyp.Add(sequences + static_cast<size_t>(bbi) * s.max_length, sequence_length, s.next_scores[bbi]);
    }
  }
}

int orc_beam_scorer_is_done(void* h) { return static_cast<OrcBeamScorer*>(h)->not_done == 0; }
const float* orc_beam_scorer_next_scores(void* h) { return static_cast<OrcBeamScorer*>(h)->next_scores.data(); }
const int32_t* orc_beam_scorer_next_tokens(void* h) { return static_cast<OrcBeamScorer*>(h)->next_tokens.data(); }
const int32_t* orc_beam_scorer_next_indices(void* h) { return static_cast<OrcBeamScorer*>(h)->next_indices.data(); }
int orc_beam_scorer_batch_done(void* h, int batch) { return static_cast<OrcBeamScorer*>(h)->hyps[batch].done; }
int orc_beam_scorer_hyp_count(void* h, int batch) {
  return static_cast<int>(static_cast<OrcBeamScorer*>(h)->hyps[batch].beams.size());
}
// Copies hypothesis `index` of `batch` into out (capacity cap); returns its length, score in *score.
int orc_beam_scorer_hyp(void* h, int batch, int index, int32_t* out, int cap, float* score) {
  auto& hy = static_cast<OrcBeamScorer*>(h)->hyps[batch];
  if (index < 0 || index >= static_cast<int>(hy.beams.size())) return -1;
  const auto& t = hy.beams[index].tokens;
  const int n = std::min<int>(cap, static_cast<int>(t.size()));
  std::copy(t.begin(), t.begin() + n, out);
  if (score) *score = hy.beams[index].score;
  return static_cast<int>(t.size());
}

// ---- a14: src/search.cpp:354-381 BeamSearch_Cpu::AppendNextTokensToSequences (buffer swap left to
// the caller).
void orc_beam_append(const int32_t* seq, int32_t* seq_next, int batch_beam, int max_length,
                     int current_length, const int32_t* beam_indices, const int32_t* tokens) {
  for (int i = 0; i < batch_beam; ++i) {
    const int32_t* src = seq + static_cast<size_t>(beam_indices[i]) * max_length;
    int32_t* dst = seq_next + static_cast<size_t>(i) * max_length;
    std::copy(src, src + current_length, dst);
    dst[current_length] = tokens[i];
  }
}

// ---- a15: src/models/kv_cache.cpp:710-740 PickPastState: past[j] = present[beam_indices[j]].
void orc_kv_gather(const void* present, void* past, const int32_t* beam_indices, int rows,
                   size_t block_bytes) {
  for (int j = 0; j < rows; ++j)
    std::memcpy(static_cast<char*>(past) + j * block_bytes,
                static_cast<const char*>(present) + beam_indices[j] * block_bytes, block_bytes);
}

// ---- a16: src/speculative_sampling.h:140-146.
float orc_accept_prob(float p_target, float p_draft) {
  if (p_draft <= 0.0f) return 1.0f;
  return std::min(1.0f, p_target / p_draft);
}

// ---- a17: src/speculative_sampling.h:150-177 BuildCorrectionDistribution.
void orc_build_correction(const float* p_target, const float* p_draft, float* out, int n) {
  float sum = 0.0f;
  for (int i = 0; i < n; ++i) {
    const float diff = p_target[i] - p_draft[i];
    out[i] = diff > 0.0f ? diff : 0.0f;
    sum += out[i];
  }
  if (sum > 0.0f) {
    const float inv_sum = 1.0f / sum;
    for (int i = 0; i < n; ++i) out[i] *= inv_sum;
  } else {
    for (int i = 0; i < n; ++i) out[i] = p_target[i];
  }
}

// src/speculative_sampling.h:22-30.
float orc_sparse_prob(const int32_t* indices, const float* probs, int n, int32_t token) {
  for (int i = 0; i < n; ++i)
    if (indices[i] == token) return probs[i];
  return 0.0f;
}

// ---- a17: src/speculative_sampling.h:39-57 SampleCorrectionToken (sparse supports, explicit draw).
int32_t orc_sample_correction(const int32_t* t_idx, const float* t_probs, int nt, const int32_t* d_idx,
                              const float* d_probs, int nd, double u) {
  std::vector<float> residual(nt);
  float sum = 0.0f;
  for (int i = 0; i < nt; ++i) {
    const float diff = t_probs[i] - orc_sparse_prob(d_idx, d_probs, nd, t_idx[i]);
    residual[i] = diff > 0.0f ? diff : 0.0f;
    sum += residual[i];
  }
  if (sum > 0.0f) return t_idx[DiscreteDraw(residual.data(), nt, u)];
  return t_idx[DiscreteDraw(t_probs, nt, u)];
}

// ---- a16/a17: the accept loop of SpeculativeDecodingStrategy::RunRound
// (src/speculative_decoding_strategy.cpp:718-762) on dense distributions: p_target, p_draft are
// [batch, K+1, vocab]; row i of a batch judges draft token i, row K supplies the bonus token.
// accept_u is [batch, K] floats (one per accept test, consumed in order), sample_u is [batch] doubles
// (the single categorical draw a round makes: the correction on the first reject, else the bonus).
void orc_spec_verify_dense(const float* p_target, const float* p_draft, const int32_t* draft_tokens,
                           const float* accept_u, const double* sample_u, int batch, int K, int vocab,
                           int32_t* accepted_len, int32_t* final_token) {
  std::vector<float> residual(vocab);
  for (int b = 0; b < batch; ++b) {
    int n_direct = 0;
    int32_t tok = -1;
    for (int i = 0; i < K; ++i) {
      const float* pt = p_target + (static_cast<size_t>(b) * (K + 1) + i) * vocab;
      const float* pd = p_draft + (static_cast<size_t>(b) * (K + 1) + i) * vocab;
      const int32_t d = draft_tokens[b * K + i];
      if (accept_u[b * K + i] < orc_accept_prob(pt[d], pd[d])) {
        n_direct++;
        continue;
      }
      float sum = 0.0f;
      for (int v = 0; v < vocab; ++v) {
        const float diff = pt[v] - pd[v];
        residual[v] = diff > 0.0f ? diff : 0.0f;
        sum += residual[v];
      }
      tok = sum > 0.0f ? DiscreteDraw(residual.data(), vocab, sample_u[b])
                       : DiscreteDraw(pt, vocab, sample_u[b]);
      break;
    }
    if (n_direct == K) {
      const float* pt = p_target + (static_cast<size_t>(b) * (K + 1) + K) * vocab;
      tok = DiscreteDraw(pt, vocab, sample_u[b]);
    }
    accepted_len[b] = n_direct;
    final_token[b] = tok;
  }
}

// ---- a16/a17 on sparse selections, the production form of the accept loop
// (src/speculative_decoding_strategy.cpp:718-762): target row i (t_off[i]..t_off[i+1]) judges proposal
// token i, target row K supplies the bonus token; draft row i is the proposal's own distribution at
// position i.  accept_u[i] is the i-th uniform_real_distribution<float> draw; sample_u[e] is the
// categorical draw the engine would yield after e accept draws have been taken (the loop takes one per
// evaluated position, so the round's single categorical draw uses sample_u[evaluated]).  *engine_draws
// = 32-bit engine outputs the reference would have consumed: one per evaluated position plus two for
// the categorical draw unless its distribution has fewer than two entries.
void orc_spec_verify_sparse(const int32_t* proposal, int K, const int32_t* t_off, const int32_t* t_idx,
                            const float* t_probs, const int32_t* d_off, const int32_t* d_idx,
                            const float* d_probs, const float* accept_u, const double* sample_u,
                            int32_t* accepted_len, int32_t* final_token, int32_t* engine_draws) {
  int n_direct = 0, n_evaluated = 0, final_n = 0;
  int32_t tok = -1;
  for (int i = 0; i < K; ++i) {
    n_evaluated++;
    const int nt = t_off[i + 1] - t_off[i], nd = d_off[i + 1] - d_off[i];
    const float p_t = orc_sparse_prob(t_idx + t_off[i], t_probs + t_off[i], nt, proposal[i]);
    const float p_d = orc_sparse_prob(d_idx + d_off[i], d_probs + d_off[i], nd, proposal[i]);
    if (accept_u[i] < orc_accept_prob(p_t, p_d)) {
      n_direct++;
      continue;
    }
    tok = orc_sample_correction(t_idx + t_off[i], t_probs + t_off[i], nt, d_idx + d_off[i], d_probs + d_off[i], nd,
                                sample_u[n_evaluated]);
    final_n = nt;
    break;
  }
  if (n_direct == K) {
    const int nt = t_off[K + 1] - t_off[K];
    tok = t_idx[t_off[K] + DiscreteDraw(t_probs + t_off[K], nt, sample_u[n_evaluated])];
    final_n = nt;
  }
  *accepted_len = n_direct;
  *final_token = tok;
  *engine_draws = n_evaluated + (final_n >= 2 ? 2 : 0);
}

// ---- a18: src/speculative_sampling.h:59-79 ComputeTargetTokenSelection with
// LogitsPenaltyProcessor::Apply (src/sampling_distribution.h:100-110): copy, min-length,
// repetition, n-gram, then argmax (greedy) or the kept distribution.  Returns kept count (0 if greedy).
int orc_target_selection(const float* logits, int vocab, int current_length, const int32_t* prefix,
                         int n_prefix, int greedy, int top_k, float top_p, float temperature,
                         float repetition_penalty, int min_length, int ngram, const int32_t* eos,
                         int n_eos, int32_t* greedy_token, int32_t* indices, float* probs) {
  std::vector<float> buf(logits, logits + vocab);
  const bool active = repetition_penalty != 1.0f || min_length > 0 || ngram > 0;
  if (active) {
    orc_apply_min_length(buf.data(), vocab, current_length, min_length, eos, n_eos);
    orc_apply_repetition_penalty(buf.data(), vocab, prefix, n_prefix, repetition_penalty);
    orc_apply_no_repeat_ngram(buf.data(), vocab, prefix, n_prefix, ngram);
  }
  if (greedy) {
    // std::max_element: first maximum under operator<.
    int32_t best = 0;
    for (int i = 1; i < vocab; ++i)
      if (buf[best] < buf[i]) best = i;
    *greedy_token = best;
    return 0;
  }
  *greedy_token = -1;
  std::vector<int32_t> scratch(vocab);
  return orc_sampled_categorical(buf.data(), vocab, top_k, top_p, temperature, scratch.data(), indices, probs);
}

// src/speculative_sampling.h:96-127 VerifyDeterministicProposal with explicit draws: draws[i] is
// consumed by the i-th SampleTargetToken call whose distribution has at least two entries (a
// one-entry distribution consumes none).  sel_off/sel_idx/sel_probs hold n_prop+1 sparse rows
// (row 0 = first_target, row i = subsequent_targets[i-1]).  Returns accepted count; *n_draws_used
// reports how many draws were consumed.
int orc_verify_deterministic(const int32_t* proposal, int n_prop, const int32_t* sel_off,
                             const int32_t* sel_idx, const float* sel_probs, const double* draws,
                             int32_t* final_token, int* evaluated, int* used_bonus, int* n_draws_used) {
  int accepted = 0, used = 0;
  *evaluated = 0;
  *used_bonus = 0;
  auto sample = [&](int row) {
    const int n = sel_off[row + 1] - sel_off[row];
    const int pos = DiscreteDraw(sel_probs + sel_off[row], n, n >= 2 ? draws[used] : 0.0);
    if (n >= 2) used++;
    return sel_idx[sel_off[row] + pos];
  };
  for (int i = 0; i < n_prop; ++i) {
    (*evaluated)++;
    *final_token = sample(i);
    if (*final_token != proposal[i]) {
      *n_draws_used = used;
      return accepted;
    }
    accepted++;
  }
  *final_token = sample(n_prop);
  *used_bonus = 1;
  *n_draws_used = used;
  return accepted;
}

}  // extern "C"
