// MI355X search & sampling backend behind the reference's plug-in contract: a DeviceInterface whose
// CreateGreedy / CreateBeam / CreateBatchedSampler build Search and BatchedSampler objects that run on
// the HIP kernels of libmi355x_search (C ABI, include/mi355x_search.h).  The classes only marshal:
// no selection, softmax or scoring arithmetic happens on the host.
#pragma once
#ifdef MI355X_USE_REFERENCE_HEADERS
#include "generators.h"
#include "search.h"
#else
#include "hip_contract.h"
#endif
#include "mi355x_search.h"

namespace Generators {

DeviceInterface* GetHipInterface();  // process-wide instance (device 0)

// The random stream of a HipBatchedSampler request: Philox4x32 with 10 rounds, and the double in [0, 1) that
// draw number `counter` of the stream with seed `seed` feeds to the sampling kernel.
void Philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);
double PhiloxUniform(uint64_t seed, uint64_t counter);

// GreedySearch_Cpu's device counterpart (src/search.h:202-240, src/search.cpp:178-324).
// Token selection, the draws and the EOS / padding / append tail run on the GPU; a step synchronises once.
// Sampling matches the CPU class draw for draw: the host prepares the next canonical doubles of (a copy of) the
// caller's std::mt19937, the device hands them to the rows in the order std::discrete_distribution would have
// consumed them (a row with one kept token and a finished row take none) and reports how many were used, and the
// caller's engine is advanced by exactly that many, so both token and engine state equal the CPU path's.
struct GreedySearch_Hip : Search {
  explicit GreedySearch_Hip(const GeneratorParams& params);
  ~GreedySearch_Hip() override;

  DeviceSpan<int32_t> GetNextTokens() override { return next_tokens_; }
  DeviceSpan<int32_t> GetNextIndices() override { return {}; }
  DeviceSpan<int32_t> GetSequenceLengths() override { return sequence_lengths_; }
  DeviceSpan<float> GetLogits() const override;
  void SetLogits(DeviceSpan<float> logits) override;
  bool IsDone() const override { return done_; }
  // Batched sampling seam (src/search.h:40-67): the engine samples a shared buffer with the
  // BatchedSampler, binds one element of it here, and OnNextTokensSampled() launches the device tail
  // (EOS / pad / append) on that element; CompleteGeneration() synchronises and advances the length.
  // Token selection through SelectTop / Sample* always completes inline, which DeferCompletion(true)
  // permits.
  void DeferCompletion(bool defer) override { defer_completion_ = defer; }
  void CompleteGeneration() override;
  bool BindNextTokensSlot(DeviceSpan<int32_t> slot) override;
  bool SupportsBatchedSampling() const override { return params_->BatchBeamSize() == 1; }
  void OnNextTokensSampled() override;

  void SelectTop() override;
  void CommitToken(int32_t token) override;
  void SampleTopP(float p, float temperature, std::mt19937& rng) override { Sample(0, p, temperature, rng); }
  void SampleTopK(int k, float temperature, std::mt19937& rng) override { Sample(k, 0.0f, temperature, rng); }
  void SampleTopKTopP(int k, float p, float temperature, std::mt19937& rng) override { Sample(k, p, temperature, rng); }
  void ApplyMinLength(int min_length) override;
  void ApplyRepetitionPenalty(float penalty) override;
  void ApplyNoRepeatNgram(int ngram_size) override;
  void AppendTokens(DeviceSpan<int32_t>& next_tokens) override;
  void RewindTo(size_t index) override;

 protected:
  void SaveStateForTransactionImpl(bool checkpoint_local_state) override;
  void RestoreStateForTransactionImpl() override;

 private:
  void Sample(int k, float p, float temperature, std::mt19937& rng);
  mi355x_logits_xform* PendingXform();
  void Materialize() const;  // applies the deferred logits processing to the logits in place
  void ClearPending() const;
  void LaunchTail(int32_t* tokens);
  void FinishStep();
  void ResetDone();

  mi355x_search_ctx* ctx_{};
  DeviceSpan<int32_t> next_tokens_, sequence_lengths_;
  DeviceSpan<float> next_token_scores_;
  DeviceSpan<int32_t> kept_count_, kept_ids_;
  DeviceSpan<float> kept_probs_;
  DeviceSpan<double> uniforms_;
  DeviceSpan<int32_t> draws_used_;
  int kept_capacity_{};
  DeviceSpan<int32_t> state_, tx_state_;  // per-row EOS flags followed by the all-rows-finished flag
  std::vector<int32_t> eos_ids_;
  bool done_{};
  bool defer_completion_{}, external_pending_{};
  DeviceSpan<int32_t> bound_slot_;
  // deferred logits processing
  mutable bool pending_min_length_{};
  mutable float pending_penalty_{1.0f};
  mutable int pending_ngram_{};
  mutable mi355x_logits_xform xf_{};
  // transaction checkpoint
  std::vector<int32_t> tx_next_tokens_, tx_sequence_lengths_;
  bool tx_done_{};
};

// BeamSearch_Cpu's device counterpart (src/search.h:242-270, src/search.cpp:101-176,326-400): candidate
// selection, BeamSearchScorer and the beam-reordered sequence store all live on the GPU.
struct BeamSearch_Hip : Search {
  explicit BeamSearch_Hip(const GeneratorParams& params);
  ~BeamSearch_Hip() override;
  DeviceSpan<int32_t> GetNextTokens() override;
  DeviceSpan<int32_t> GetNextIndices() override;
  DeviceSpan<int32_t> GetSequenceLengths() override { return sequence_lengths_; }
  DeviceSpan<int32_t> GetSequence(size_t index) override;
  DeviceSpan<int32_t> GetSequence(size_t batch_id, size_t beam_id);
  DeviceSpan<float> GetLogits() const override { return next_token_scores_; }
  void SetLogits(DeviceSpan<float> logits) override { next_token_scores_ = logits; }
  bool IsDone() const override;
  void SelectTop() override;
  void ApplyMinLength(int min_length) override;
  void ApplyRepetitionPenalty(float penalty) override;
  void ApplyNoRepeatNgram(int ngram_size) override;
  void AppendTokens(DeviceSpan<int32_t>& next_tokens) override;

 private:
  mi355x_search_ctx* ctx_{};
  mi355x_beam_scorer* scorer_{};
  DeviceSpan<int32_t> sequence_lengths_;
  DeviceSpan<float> next_token_scores_;
  DeviceSpan<float> cand_scores_;
  DeviceSpan<int32_t> cand_tokens_, cand_indices_;
  std::vector<DeviceSpan<int32_t>> hypotheses_;
  int length_{};
};

}  // namespace Generators

extern "C" {
// The add-on entry points the reference's loader resolves (src/cuda/interface.cpp:698-715,
// src/generators.cpp:321-356).
uint32_t GetInterfaceVersion();
Generators::DeviceInterface* GetInterface(GenaiInterface* p_genai, const char* deviceType, const OrtApi* ort_api);
}
