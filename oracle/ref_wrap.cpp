// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// C-callable wrapper over the UNMODIFIED reference headers, included from where they lie
// (-I/root/reference/src): sampling_distribution.h, speculative_sampling.h, softmax.h, span.h.
// These four are STL-only and compile stand-alone.  The result (oracle/_ref/libref_headers.so) is
// used to validate oracle/search_oracle.cpp and, optionally, as the "reference" CPU baseline.
// The remaining reference sources on the path (search.cpp, beam_search_scorer.cpp, sequences.cpp,
// softmax_cpu.cpp) include generators.h -> onnxruntime_c_api.h, which this image lacks, so they are
// unbuildable here and are not wrapped.
//
// Random draws: the reference only accepts std::mt19937&.  Each wrapper seeds an engine, reports the
// uniform the reference will consume (computed on a clone with the same arithmetic libstdc++ uses)
// and then calls the reference with the original engine.
#include <cstdint>
#include <random>
#include <vector>
#include "sampling_distribution.h"
#include "speculative_sampling.h"
#include "softmax.h"

using namespace Generators;

namespace {
// generate_canonical<double,53>(mt19937): two 32-bit draws, (x0 + x1*2^32) / 2^64, clamped below 1
// (/usr/include/c++/11/bits/random.tcc:3348-3380).
double CanonicalDouble(std::mt19937 rng) {
  const double x0 = static_cast<double>(rng());
  const double x1 = static_cast<double>(rng());
  double r = (x0 + x1 * 4294967296.0) / 18446744073709551616.0;
  if (r >= 1.0) r = std::nextafter(1.0, 0.0);
  return r;
}
// uniform_real_distribution<float>(0,1): one 32-bit draw, float(x)/2^32, clamped below 1.
float CanonicalFloat(std::mt19937 rng) {
  float r = static_cast<float>(rng()) / 4294967296.0f;
  if (r >= 1.0f) r = std::nextafter(1.0f, 0.0f);
  return r;
}
}  // namespace

extern "C" {

int ref_sampled_categorical(const float* scores, int vocab, int top_k, float top_p, float temperature,
                            int32_t* indices, float* probs) {
  SampledCategorical c;
  ComputeSampledCategorical({scores, static_cast<size_t>(vocab)}, top_k, top_p, temperature, c);
  std::copy(c.indices.begin(), c.indices.end(), indices);
  std::copy(c.probs.begin(), c.probs.end(), probs);
  return static_cast<int>(c.indices.size());
}

// SampleCategoricalToken with mt19937{seed}; *u_out = the canonical double it consumes (valid when
// n >= 2), *draws_out = number of 32-bit engine draws consumed.
int32_t ref_sample_categorical(const int32_t* indices, const float* probs, int n, uint32_t seed,
                               double* u_out, int* draws_out) {
  std::mt19937 rng{seed};
  *u_out = CanonicalDouble(rng);
  std::mt19937 before = rng;
  const int32_t tok = SampleCategoricalToken({indices, static_cast<size_t>(n)}, {probs, static_cast<size_t>(n)}, rng);
  int draws = 0;
  while (!(before == rng) && draws < 8) {
    before();
    draws++;
  }
  *draws_out = draws;
  return tok;
}

float ref_uniform_float(uint32_t seed) {
  std::mt19937 rng{seed};
  const float expect = CanonicalFloat(rng);
  std::uniform_real_distribution<float> uni(0.f, 1.f);
  const float got = uni(rng);
  return got == expect ? got : -1.0f;
}

void ref_softmax(float* s, int n, float temperature) { Softmax({s, static_cast<size_t>(n)}, temperature); }
void ref_log_softmax(float* s, int n, float temperature) { LogSoftMax({s, static_cast<size_t>(n)}, temperature); }

void ref_apply_min_length(float* logits, int vocab, int cur, int min_len, const int32_t* eos, int n_eos) {
  ApplyMinLengthToLogits({logits, static_cast<size_t>(vocab)}, cur, min_len, {eos, static_cast<size_t>(n_eos)});
}
void ref_apply_repetition_penalty(float* logits, int vocab, const int32_t* prefix, int n, float pen) {
  std::vector<bool> visited;
  ApplyRepetitionPenaltyToLogits({logits, static_cast<size_t>(vocab)}, {prefix, static_cast<size_t>(n)}, pen, visited);
}
void ref_apply_no_repeat_ngram(float* logits, int vocab, const int32_t* prefix, int n, int ngram) {
  ApplyNoRepeatNgramToLogits({logits, static_cast<size_t>(vocab)}, {prefix, static_cast<size_t>(n)}, ngram);
}

float ref_accept_prob(float pt, float pd) { return ComputeAcceptProb(pt, pd); }
void ref_build_correction(const float* pt, const float* pd, float* out, int n) {
  BuildCorrectionDistribution({pt, static_cast<size_t>(n)}, {pd, static_cast<size_t>(n)}, {out, static_cast<size_t>(n)});
}
int32_t ref_sample_correction(const int32_t* t_idx, const float* t_probs, int nt, const int32_t* d_idx,
                              const float* d_probs, int nd, uint32_t seed, double* u_out) {
  std::mt19937 rng{seed};
  *u_out = CanonicalDouble(rng);
  return SampleCorrectionToken({t_idx, static_cast<size_t>(nt)}, {t_probs, static_cast<size_t>(nt)},
                               {d_idx, static_cast<size_t>(nd)}, {d_probs, static_cast<size_t>(nd)}, rng);
}

int ref_target_selection(const float* logits, int vocab, int current_length, const int32_t* prefix,
                         int n_prefix, int greedy, int top_k, float top_p, float temperature,
                         float repetition_penalty, int min_length, int ngram, const int32_t* eos,
                         int n_eos, int32_t* greedy_token, int32_t* indices, float* probs) {
  LogitsPenaltyProcessor proc{vocab, repetition_penalty, min_length, ngram, {eos, static_cast<size_t>(n_eos)}};
  SampledCategorical sampled;
  TargetTokenSelection sel;
  ComputeTargetTokenSelection({logits, static_cast<size_t>(vocab)}, current_length,
                              {prefix, static_cast<size_t>(n_prefix)}, greedy != 0, top_k, top_p,
                              temperature, proc, sampled, sel);
  *greedy_token = sel.greedy_token;
  std::copy(sel.indices.begin(), sel.indices.end(), indices);
  std::copy(sel.probs.begin(), sel.probs.end(), probs);
  return static_cast<int>(sel.indices.size());
}

// VerifyDeterministicProposal with mt19937{seed}.  Selections as CSR rows (row 0 = first target).
// draws_out receives the canonical doubles consumed, in order (capacity n_prop+1).
int ref_verify_deterministic(const int32_t* proposal, int n_prop, const int32_t* sel_off,
                             const int32_t* sel_idx, const float* sel_probs, uint32_t seed,
                             int32_t* final_token, int* evaluated, int* used_bonus, double* draws_out,
                             int* n_draws) {
  std::vector<TargetTokenSelection> sels(n_prop + 1);
  for (int r = 0; r <= n_prop; ++r) {
    sels[r].indices.assign(sel_idx + sel_off[r], sel_idx + sel_off[r + 1]);
    sels[r].probs.assign(sel_probs + sel_off[r], sel_probs + sel_off[r + 1]);
  }
  std::mt19937 rng{seed};
  std::vector<std::mt19937> states;
  std::mt19937 prev = rng;
  auto result = VerifyDeterministicProposal({proposal, static_cast<size_t>(n_prop)}, sels[0],
                                            {sels.data() + 1, static_cast<size_t>(n_prop)}, rng, &states);
  int nd = 0;
  for (auto& st : states) {
    if (!(st == prev)) draws_out[nd++] = CanonicalDouble(prev);
    prev = st;
  }
  *n_draws = nd;
  *final_token = result.final_token;
  *evaluated = result.evaluated_count;
  *used_bonus = result.used_bonus ? 1 : 0;
  return result.accepted_count;
}

// The accept loop of SpeculativeDecodingStrategy::RunRound (src/speculative_decoding_strategy.cpp:718-762;
// the strategy itself needs models and ONNX Runtime, so the loop is driven here) with the reference's own
// ComputeAcceptProb, GetSparseTokenProbability, SampleCorrectionToken and SampleSparseToken and a real
// std::mt19937{seed}.  accept_u_out (capacity K) and sample_u_out (capacity K+1: the canonical double
// the engine would yield after e accept draws) report the uniforms in the oracle's explicit-draw form;
// *engine_draws = engine outputs consumed by the round.
void ref_spec_round_sparse(const int32_t* proposal, int K, const int32_t* t_off, const int32_t* t_idx,
                           const float* t_probs, const int32_t* d_off, const int32_t* d_idx,
                           const float* d_probs, uint32_t seed, float* accept_u_out, double* sample_u_out,
                           int32_t* accepted_len, int32_t* final_token, int32_t* engine_draws) {
  auto row = [](const int32_t* off, const int32_t* idx, const float* probs, int r) {
    TargetTokenSelection sel;
    sel.indices.assign(idx + off[r], idx + off[r + 1]);
    sel.probs.assign(probs + off[r], probs + off[r + 1]);
    return sel;
  };
  {
    std::mt19937 probe{seed};
    std::uniform_real_distribution<float> uni(0.f, 1.f);
    for (int e = 0; e <= K; ++e) {
      std::mt19937 at = probe;
      sample_u_out[e] = CanonicalDouble(at);
      if (e < K) accept_u_out[e] = uni(probe);
    }
  }
  std::mt19937 rng{seed};
  std::uniform_real_distribution<float> uni(0.f, 1.f);
  int n_direct = 0;
  int32_t tok = -1;
  for (int i = 0; i < K; i++) {
    const TargetTokenSelection target = row(t_off, t_idx, t_probs, i);
    const TargetTokenSelection draft = row(d_off, d_idx, d_probs, i);
    const float p_t = GetTargetTokenProbability(target, proposal[i]);
    const float p_d = GetTargetTokenProbability(draft, proposal[i]);
    if (uni(rng) < ComputeAcceptProb(p_t, p_d)) {
      n_direct++;
    } else {
      tok = SampleCorrectionToken(target.indices, target.probs, draft.indices, draft.probs, rng);
      break;
    }
  }
  if (n_direct == K) {
    const TargetTokenSelection bonus = row(t_off, t_idx, t_probs, K);
    tok = SampleSparseToken(bonus.indices, bonus.probs, rng);
  }
  int used = 0;
  for (std::mt19937 walk{seed}; !(walk == rng); walk.discard(1)) ++used;
  *accepted_len = n_direct;
  *final_token = tok;
  *engine_draws = used;
}

}  // extern "C"
