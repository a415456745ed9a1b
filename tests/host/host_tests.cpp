// Host-layer tests for the MI355X add-on: they drive the backend through the same virtuals the
// reference's Generator / ScheduledRequests call, and mirror the reference's own tests for this seam
// (test/search_checkpoint_tests.cpp, test/cuda_batched_sampler_tests/cuda_batched_sampler_tests.cpp,
// test/sampling_tests.cpp:22-49).  Expected values come from the CPU oracle (liboracle, test
// infrastructure) combined with std::discrete_distribution / std::mt19937, i.e. from what
// GreedySearch_Cpu / BeamSearch_Cpu would produce on the same inputs.
//
// Usage: host_tests [filter-substring]; prints one line per test, exits non-zero on any failure.
#include "hip_backend.h"

#include <algorithm>
#include <array>
#include <cmath>
#include <cstdio>
#include <functional>
#include <limits>
#include <numeric>
#include <random>

using namespace Generators;

extern "C" {
int32_t orc_argmax(const float* v, int n);
void orc_apply_min_length(float* logits, int vocab, int current_length, int min_length, const int32_t* eos, int n_eos);
void orc_apply_repetition_penalty(float* logits, int vocab, const int32_t* prefix, int n, float penalty);
void orc_apply_no_repeat_ngram(float* logits, int vocab, const int32_t* prefix, int n, int ngram);
int orc_sampled_categorical(const float* scores, int vocab, int top_k, float top_p, float temperature, int32_t* scratch,
                            int32_t* indices, float* out_probs);
void orc_beam_select_top(float* scores, int batch, int beams, int vocab, const float* beam_scores, float* out_scores,
                         int32_t* out_tokens, int32_t* out_indices);
void* orc_beam_scorer_create(int batch, int beams, int max_length, int pad, const int32_t* eos, int n_eos,
                             float length_penalty, int early_stopping);
void orc_beam_scorer_destroy(void* h);
void orc_beam_scorer_process(void* h, const int32_t* sequences, int sequence_length, const float* cand_scores,
                             const int32_t* cand_tokens, const int32_t* cand_indices);
void orc_beam_scorer_finalize(void* h, const int32_t* sequences, int sequence_length);
int orc_beam_scorer_is_done(void* h);
const float* orc_beam_scorer_next_scores(void* h);
const int32_t* orc_beam_scorer_next_tokens(void* h);
const int32_t* orc_beam_scorer_next_indices(void* h);
int orc_beam_scorer_hyp(void* h, int batch, int index, int32_t* out, int cap, float* score);
void orc_beam_append(const int32_t* seq, int32_t* seq_next, int batch_beam, int max_length, int current_length,
                     const int32_t* beam_indices, const int32_t* tokens);
}

namespace {

int g_failures = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::printf("    FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);     \
      ++g_failures;                                                         \
    }                                                                       \
  } while (0)
#define EXPECT_EQ(a, b) EXPECT((a) == (b))
template <typename E, typename F>
bool Throws(F&& f) {
  try {
    f();
  } catch (const E&) {
    return true;
  } catch (...) {
    return false;
  }
  return false;
}

DeviceInterface* Device() { return GetInterface(nullptr, "AMDGPU", nullptr); }

template <typename T>
DeviceSpan<T> ToDevice(const std::vector<T>& v) {
  auto s = Device()->Allocate<T>(v.size());
  std::copy(v.begin(), v.end(), s.CpuSpan().begin());
  s.CopyCpuToDevice();
  return s;
}
template <typename T>
std::vector<T> ToHost(DeviceSpan<T> s) {
  auto h = s.CopyDeviceToCpu();
  return {h.begin(), h.end()};
}

std::vector<float> RandomLogits(std::mt19937& gen, size_t n, float sigma) {
  std::normal_distribution<float> dist(0.0f, sigma);
  std::vector<float> v(n);
  for (auto& x : v) x = dist(gen);
  return v;
}

// ---- a host model of GreedySearch_Cpu (src/search.cpp:178-296,407-430) built on the oracle ----------------
struct GreedyModel {
  GreedyModel(const Config& c) : config{c}, batch{c.search.batch_size}, vocab{c.model.vocab_size} {
    sequences.assign(static_cast<size_t>(batch) * c.search.max_length, 0);
    next_tokens.assign(batch, 0);
    eos_seen.assign(batch, 0);
    not_done = batch;
    eos.assign(c.model.eos_token_id.begin(), c.model.eos_token_id.end());
  }
  void Append() {
    for (int i = 0; i < batch; ++i) sequences[static_cast<size_t>(i) * config.search.max_length + length] = next_tokens[i];
    if (++length == config.search.max_length) done = true;
  }
  void AppendPrompt(const std::vector<int32_t>& tokens) {
    const int per_row = static_cast<int>(tokens.size()) / batch;
    for (int j = 0; j < per_row; ++j) {
      for (int i = 0; i < batch; ++i) next_tokens[i] = tokens[i * per_row + j];
      Append();
    }
    done = false;
    not_done = batch;
    std::fill(eos_seen.begin(), eos_seen.end(), 0);
  }
  void SetNext(int b, int32_t t) {
    next_tokens[b] = t;
    if (std::find(eos.begin(), eos.end(), t) != eos.end()) {
      eos_seen[b] = 1;
      if (--not_done == 0) done = true;
    }
  }
  void Process(std::vector<float>& logits, int min_length, float penalty, int ngram = 0) {
    for (int b = 0; b < batch; ++b) {
      float* row = logits.data() + static_cast<size_t>(b) * vocab;
      const int32_t* seq = sequences.data() + static_cast<size_t>(b) * config.search.max_length;
      orc_apply_min_length(row, vocab, length, min_length, eos.data(), static_cast<int>(eos.size()));
      if (penalty != 1.0f) orc_apply_repetition_penalty(row, vocab, seq, length, penalty);
      orc_apply_no_repeat_ngram(row, vocab, seq, length, ngram);
    }
  }
  void SelectTop(const std::vector<float>& logits) {
    for (int b = 0; b < batch; ++b) {
      if (eos_seen[b]) {
        next_tokens[b] = config.model.pad_token_id;
        continue;
      }
      SetNext(b, orc_argmax(logits.data() + static_cast<size_t>(b) * vocab, vocab));
    }
    if (!done) Append();
  }
  void Sample(const std::vector<float>& logits, int k, float p, float t, std::mt19937& rng) {
    std::vector<int32_t> scratch(vocab), ids(vocab);
    std::vector<float> probs(vocab);
    for (int b = 0; b < batch; ++b) {
      if (eos_seen[b]) {
        next_tokens[b] = config.model.pad_token_id;
        continue;
      }
      const int n = orc_sampled_categorical(logits.data() + static_cast<size_t>(b) * vocab, vocab, k, p, t, scratch.data(),
                                            ids.data(), probs.data());
      std::discrete_distribution<int> dist(probs.begin(), probs.begin() + n);
      SetNext(b, ids[dist(rng)]);
    }
    if (!done) Append();
  }
  const Config& config;
  int batch, vocab, length{}, not_done{};
  bool done{};
  std::vector<int32_t> sequences, next_tokens, eos;
  std::vector<uint8_t> eos_seen;
};

struct GreedyFixture {
  GreedyFixture(int batch, int vocab, int max_length, std::vector<int> eos, int pad = 0) {
    config.model.vocab_size = vocab;
    config.model.eos_token_id = std::move(eos);
    config.model.pad_token_id = pad;
    config.search.batch_size = batch;
    config.search.max_length = max_length;
    config.search.random_seed = 1234;
    params = std::make_shared<GeneratorParams>(config);
    params->p_device = Device();
    search = params->p_device->CreateGreedy(*params);
  }
  void SetLogits(const std::vector<float>& values) {
    logits = ToDevice(values);
    search->SetLogits(logits);
  }
  std::vector<int32_t> NextTokens() { return ToHost(search->GetNextTokens()); }
  Config config;
  std::shared_ptr<GeneratorParams> params;
  std::unique_ptr<Search> search;
  DeviceSpan<float> logits;
};

// ---- tests -------------------------------------------------------------------------------------------------
void InterfaceEntryPoints() {
  EXPECT_EQ(GetInterfaceVersion(), kDeviceInterfaceVersion);
  EXPECT(GetInterface(nullptr, "cuda", nullptr) == nullptr);
  auto* device = Device();
  EXPECT(device != nullptr);
  EXPECT(device == GetInterface(nullptr, "HIP", nullptr));
  EXPECT(device->GetType() == DeviceType::AMDGPU);
  EXPECT(device->GetCudaStream() != nullptr);
  size_t free_bytes = 0, total_bytes = 0;
  device->GetAvailableMemory(free_bytes, total_bytes);
  EXPECT(total_bytes > (size_t{64} << 30) && free_bytes <= total_bytes);
  EXPECT(Throws<std::runtime_error>([&] { device->GetAllocator(); }));
}

void DeviceBufferContract() {
  auto* device = Device();
  auto a = device->Allocate<int32_t>(8);
  std::iota(a.CpuSpan().begin(), a.CpuSpan().end(), 10);
  a.CopyCpuToDevice();
  auto b = device->Allocate<int32_t>(8);
  b.Zero();
  EXPECT_EQ(ToHost(b), std::vector<int32_t>(8, 0));
  b.subspan(2, 4).CopyFrom(a.subspan(1, 4));  // device -> device with offsets
  EXPECT_EQ(ToHost(b), (std::vector<int32_t>{0, 0, 11, 12, 13, 14, 0, 0}));
  auto wrapped = device->WrapMemory<int32_t>(a.Span().subspan(4, 4));  // non-owning view
  EXPECT_EQ(ToHost(wrapped), (std::vector<int32_t>{14, 15, 16, 17}));
  EXPECT(std::string(a.subspan(0, 1).Span().data() == a.Span().data() ? "same" : "diff") == "same");
  const std::array<int32_t, 8> src{7, 6, 5, 4, 3, 2, 1, 0};
  a.CopyFromCpu(src);
  EXPECT_EQ(ToHost(a), std::vector<int32_t>(src.begin(), src.end()));
}

// test/cuda_batched_sampler_tests/cuda_batched_sampler_tests.cpp:63-96
void LogitsMaskUsesPaddedRowStride() {
  constexpr int batch_size = 2, vocab_size = 33;
  auto logits = ToDevice(std::vector<float>(batch_size * vocab_size, 1.0f));
  auto mask = ToDevice(std::vector<uint32_t>{1u << 0, 1u << 0, 1u << 1, 1u << 0});
  Device()->LaunchAddLogitsMask(logits.Span().data(), batch_size, vocab_size, mask.Span().data());
  const auto result = ToHost(logits);
  for (int row = 0; row < batch_size; ++row)
    for (int token = 0; token < vocab_size; ++token) {
      const bool allowed = token == 32 || token == row;
      EXPECT_EQ(result[row * vocab_size + token], allowed ? 1.0f : std::numeric_limits<float>::lowest());
    }
}

uint16_t FloatToHalfBits(float f) {  // round-to-nearest-even, normal range only (test inputs are tame)
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  int32_t e = static_cast<int32_t>((x >> 23) & 0xff) - 127 + 15;
  uint32_t m = x & 0x7fffffu;
  if (e <= 0) return static_cast<uint16_t>(sign);
  uint32_t h = (static_cast<uint32_t>(e) << 10) | (m >> 13);
  const uint32_t rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) ++h;
  return static_cast<uint16_t>(sign | h);
}
float HalfBitsToFloat(uint16_t h) {
  const int e = (h >> 10) & 0x1f, m = h & 0x3ff;
  const float v = e == 0 ? std::ldexp(static_cast<float>(m), -24) : std::ldexp(static_cast<float>(m | 0x400), e - 25);
  return (h & 0x8000) ? -v : v;
}

// DeviceInterface::ArgMax / ArgMaxDevice / TopKScores (src/smartptrs.h:249-259)
void DeviceFastPaths() {
  constexpr int rows = 5, vocab = 3001, k = 8;
  std::mt19937 gen(7);
  auto values = RandomLogits(gen, rows * vocab, 2.0f);
  auto logits = ToDevice(values);
  std::vector<int32_t> tokens(rows);
  EXPECT(Device()->ArgMax(logits.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, rows, vocab, tokens.data()));
  for (int r = 0; r < rows; ++r) EXPECT_EQ(tokens[r], orc_argmax(values.data() + r * vocab, vocab));
  auto out = Device()->Allocate<int32_t>(rows);
  EXPECT(Device()->ArgMaxDevice(logits.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, rows, vocab, out));
  EXPECT_EQ(ToHost(out), tokens);
  EXPECT(!Device()->ArgMax(logits.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32, rows, vocab, tokens.data()));

  std::vector<uint16_t> halves(values.size());
  std::vector<float> widened(values.size());
  for (size_t i = 0; i < values.size(); ++i) widened[i] = HalfBitsToFloat(halves[i] = FloatToHalfBits(values[i]));
  auto half_logits = ToDevice(halves);
  std::vector<int32_t> top_tokens(rows * k);
  std::vector<float> top_scores(rows * k);
  EXPECT(Device()->TopKScores(half_logits.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16, rows, vocab, k,
                              top_tokens.data(), top_scores.data()));
  for (int r = 0; r < rows; ++r) {
    std::vector<int32_t> order(vocab);
    std::iota(order.begin(), order.end(), 0);
    const float* row = widened.data() + r * vocab;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return row[a] > row[b]; });
    for (int j = 0; j < k; ++j) {
      EXPECT_EQ(top_tokens[r * k + j], order[j]);
      EXPECT_EQ(top_scores[r * k + j], row[order[j]]);
    }
  }
  // k beyond 64 (an MTP / speculative caller with top_k 100, src/mtp_generator.cpp:386-397) stays on the device
  {
    constexpr int k2 = 100;
    std::vector<int32_t> tokens2(rows * k2);
    std::vector<float> scores2(rows * k2);
    EXPECT(Device()->TopKScores(half_logits.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16, rows, vocab, k2,
                                tokens2.data(), scores2.data()));
    for (int r = 0; r < rows; ++r) {
      std::vector<int32_t> order(vocab);
      std::iota(order.begin(), order.end(), 0);
      const float* row = widened.data() + r * vocab;
      std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return row[a] > row[b]; });
      for (int j = 0; j < k2; ++j) {
        EXPECT_EQ(tokens2[r * k2 + j], order[j]);
        EXPECT_EQ(scores2[r * k2 + j], row[order[j]]);
      }
    }
  }
  EXPECT(!Device()->TopKScores(half_logits.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16, rows, vocab, vocab + 1,
                               top_tokens.data(), top_scores.data()));
  // DeviceInterface::Cast: fp16 -> fp32 on the device equals the host-side widening used above
  auto widened_dev = Device()->Allocate<float>(values.size());
  EXPECT(Device()->Cast(half_logits.Span().data(), widened_dev.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16,
                        ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, values.size()));
  EXPECT(ToHost(widened_dev) == widened);
  EXPECT(!Device()->Cast(widened_dev.Span().data(), half_logits.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT,
                         ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32, values.size()));
  EXPECT(Throws<std::runtime_error>([&] {
    Device()->Cast(widened_dev.Span().data(), widened_dev.Span().data(), ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT,
                   ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, 1);
  }));
}

// test/sampling_tests.cpp:22-49: top_k = 1 sampling returns the argmax of every row
void SamplingTopKOneIsGreedy() {
  GreedyFixture f(4, 5, 10, {99});
  f.SetLogits({0.1f, 0.6f, 0.1f, 0.1f, 0.1f, 0.25f, 0.25f, 0.3f, 0.1f, 0.1f,
               0.1f, 0.1f, 0.1f, 0.6f, 0.1f, 0.1f, 0.1f, 0.1f, 0.1f, 0.6f});
  std::mt19937 rng(42);
  const auto before = rng;
  f.search->SampleTopK(1, 1.0f, rng);
  EXPECT_EQ(f.NextTokens(), (std::vector<int32_t>{1, 2, 3, 4}));
  EXPECT(rng == before);  // one-element distributions draw nothing (libstdc++ discrete_distribution)
}

// test/search_checkpoint_tests.cpp:50-82
void SamplingRollbackRestoresRandomState() {
  GreedyFixture f(2, 4, 8, {3});
  auto input = ToDevice(std::vector<int32_t>{1, 2});
  f.search->AppendTokens(input);
  f.SetLogits({1.0f, 1.0f, 1.0f, -100.0f, 1.0f, 1.0f, 1.0f, -100.0f});
  std::mt19937 rng(1234);
  f.search->SaveStateForTransaction();
  const auto transaction_rng = rng;
  std::vector<int32_t> first_tokens, retried_tokens;
  for (int i = 0; i < 4; ++i) {
    f.search->SampleTopK(3, 1.0f, rng);
    auto next = f.NextTokens();
    first_tokens.insert(first_tokens.end(), next.begin(), next.end());
  }
  EXPECT_EQ(f.search->GetSequenceLength(), 5);
  f.search->RestoreStateForTransaction();
  rng = transaction_rng;
  EXPECT_EQ(f.search->GetSequenceLength(), 1);
  EXPECT_EQ(f.NextTokens(), (std::vector<int32_t>{1, 2}));
  for (int i = 0; i < 4; ++i) {
    f.search->SampleTopK(3, 1.0f, rng);
    auto next = f.NextTokens();
    retried_tokens.insert(retried_tokens.end(), next.begin(), next.end());
  }
  EXPECT_EQ(retried_tokens, first_tokens);
  // and the draws are the CPU class's: three equal weights, one generate_canonical each
  std::mt19937 model_rng(1234);
  std::vector<int32_t> expected;
  for (int i = 0; i < 8; ++i) {
    const std::array<float, 3> w{1.0f, 1.0f, 1.0f};
    std::discrete_distribution<int> dist(w.begin(), w.end());
    expected.push_back(dist(model_rng));
  }
  EXPECT_EQ(first_tokens, expected);
  EXPECT(rng == model_rng);
}

// test/search_checkpoint_tests.cpp:84-127
void RollbackRestoresDoneEosAndLengthState() {
  GreedyFixture f(2, 4, 8, {3});
  auto input = ToDevice(std::vector<int32_t>{1, 2});
  f.search->AppendTokens(input);
  auto lengths = f.search->GetSequenceLengths();
  lengths.CpuSpan()[0] = 5;
  lengths.CpuSpan()[1] = 7;
  lengths.CopyCpuToDevice();
  f.search->SaveStateForTransaction();
  f.SetLogits({0, 10, 0, 0, 0, 0, 10, 0});
  f.search->SelectTop();
  EXPECT_EQ(f.search->GetSequenceLength(), 2);
  lengths.CpuSpan()[0] = 50;
  lengths.CpuSpan()[1] = 70;
  lengths.CopyCpuToDevice();
  f.SetLogits({0, 0, 0, 10, 0, 0, 0, 10});
  f.search->SelectTop();
  EXPECT(f.search->IsDone());
  f.search->RestoreStateForTransaction();
  EXPECT(!f.search->IsDone());
  EXPECT_EQ(f.search->GetSequenceLength(), 1);
  EXPECT_EQ(ToHost(f.search->GetSequence(0)), std::vector<int32_t>{1});
  EXPECT_EQ(ToHost(f.search->GetSequence(1)), std::vector<int32_t>{2});
  EXPECT_EQ(f.NextTokens(), (std::vector<int32_t>{1, 2}));
  EXPECT_EQ(ToHost(f.search->GetSequenceLengths()), (std::vector<int32_t>{5, 7}));
  f.SetLogits({0, 0, 0, 10, 0, 10, 0, 0});
  f.search->SelectTop();
  EXPECT(!f.search->IsDone());
  EXPECT_EQ(f.search->GetSequenceLength(), 2);
  EXPECT_EQ(f.NextTokens(), (std::vector<int32_t>{3, 1}));
  f.SetLogits({10, 0, 0, 0, 0, 0, 0, 10});
  f.search->SelectTop();
  EXPECT(f.search->IsDone());
  EXPECT_EQ(f.search->GetSequenceLength(), 2);
}

// test/search_checkpoint_tests.cpp:129-142
void EnforcesOneActiveCheckpoint() {
  GreedyFixture f(2, 4, 8, {3});
  f.search->SaveStateForTransaction();
  EXPECT(Throws<std::logic_error>([&] { f.search->SaveStateForTransaction(); }));
  f.search->CommitStateForTransaction();
  EXPECT(Throws<std::logic_error>([&] { f.search->CommitStateForTransaction(); }));
  EXPECT(Throws<std::logic_error>([&] { f.search->RestoreStateForTransaction(); }));
  f.search->SaveStateForTransaction();
  f.search->RestoreStateForTransaction();
  EXPECT(Throws<std::logic_error>([&] { f.search->RestoreStateForTransaction(); }));
  EXPECT(Throws<std::logic_error>([&] { f.search->CommitStateForTransaction(); }));
}

// test/search_checkpoint_tests.cpp:217-255
void BatchedSamplerRollbackRestoresRequestRandomStates() {
  auto sampler = Device()->CreateBatchedSampler(2, 4);
  EXPECT(sampler != nullptr && sampler->SupportsTransactions());
  auto first_state = sampler->CreateState(1234), second_state = sampler->CreateState(5678);
  std::array<BatchedSamplerState*, 2> states{first_state.get(), second_state.get()};
  std::array<BatchedSamplingParams, 2> sampling_params{BatchedSamplingParams{3, 1.0f, 1.0f}, BatchedSamplingParams{3, 1.0f, 1.0f}};
  auto scores = ToDevice(std::vector<float>{1, 1, 1, -100, 1, 1, 1, -100});
  std::array<DeviceSpan<float>, 2> rows{scores.subspan(0, 4), scores.subspan(4, 4)};
  sampler->SaveStateForTransaction(states);
  const auto first = ToHost(sampler->Sample(rows, sampling_params, states, 4));
  sampler->RestoreStateForTransaction();
  const auto retried = ToHost(sampler->Sample(rows, sampling_params, states, 4));
  EXPECT_EQ(retried, first);
  // without a restore the streams move on: eight more draws cannot all repeat the first pair
  bool moved = false;
  for (int i = 0; i < 8; ++i) moved = moved || ToHost(sampler->Sample(rows, sampling_params, states, 4)) != first;
  EXPECT(moved);
  auto other = Device()->CreateBatchedSampler(2, 4);
  EXPECT(sampler->OwnsState(*first_state) && !other->OwnsState(*first_state));
  EXPECT(Throws<std::runtime_error>([&] { other->Sample(rows, sampling_params, states, 4); }));
}

// test/search_checkpoint_tests.cpp:257-302
void ExternalSamplingRollbackRestoresSearchTailState() {
  GreedyFixture f(1, 4, 8, {3});
  auto input = ToDevice(std::vector<int32_t>{1});
  f.search->AppendTokens(input);
  auto lengths = f.search->GetSequenceLengths();
  lengths.CpuSpan()[0] = 5;
  lengths.CopyCpuToDevice();
  auto sampler = Device()->CreateBatchedSampler(1, 4);
  auto state = sampler->CreateState(1234);
  std::array<BatchedSamplerState*, 1> states{state.get()};
  std::array<BatchedSamplingParams, 1> sampling_params{BatchedSamplingParams{1, 0.0f, 1.0f}};
  auto scores = ToDevice(std::vector<float>{0, 0, 0, 10});
  std::array<DeviceSpan<float>, 1> rows{scores};
  EXPECT(f.search->SupportsBatchedSampling());
  f.search->SaveStateForExternalSamplingTransaction();
  sampler->SaveStateForTransaction(states);
  auto next_tokens = sampler->Sample(rows, sampling_params, states, 4);
  EXPECT(f.search->BindNextTokensSlot(next_tokens));
  f.search->OnNextTokensSampled();
  next_tokens.CopyDeviceToCpu();
  f.search->CompleteGeneration();
  EXPECT(f.search->IsDone());
  EXPECT_EQ(f.NextTokens(), std::vector<int32_t>{3});
  sampler->RestoreStateForTransaction();
  f.search->RestoreStateForTransaction();
  EXPECT(!f.search->IsDone());
  EXPECT_EQ(f.search->GetSequenceLength(), 1);
  EXPECT_EQ(ToHost(f.search->GetSequenceLengths())[0], 5);
  // a two-row search cannot bind a shared slot
  GreedyFixture two(2, 4, 8, {3});
  EXPECT(!two.search->SupportsBatchedSampling() && !two.search->BindNextTokensSlot(next_tokens));
}

// test/cuda_batched_sampler_tests/cuda_batched_sampler_tests.cpp:25-61
void BatchedSamplerHandlesHeterogeneousRows() {
  constexpr int vocab_size = 5;
  auto sampler = Device()->CreateBatchedSampler(3, vocab_size);
  const std::vector<std::vector<float>> logits{{0, 5, 1, 2, 3}, {0, 1, 6, 2, 3}, {0, 1, 2, 7, 3}};
  std::vector<DeviceSpan<float>> rows;
  for (auto& row : logits) rows.push_back(ToDevice(row));
  const std::array<BatchedSamplingParams, 3> params{{{1, 0.0f, 1.0f}, {2, 0.01f, 0.7f}, {-1, 0.01f, 1.3f}}};
  std::array<std::unique_ptr<BatchedSamplerState>, 3> owned;
  std::array<BatchedSamplerState*, 3> states;
  for (size_t i = 0; i < 3; ++i) states[i] = (owned[i] = sampler->CreateState(static_cast<int>(10 + i))).get();
  EXPECT_EQ(ToHost(sampler->Sample(rows, params, states, vocab_size)), (std::vector<int32_t>{1, 2, 3}));
}

// test/cuda_batched_sampler_tests/cuda_batched_sampler_tests.cpp:98-135
void BatchedSamplerPreservesRngAcrossBatchReorder() {
  constexpr int vocab_size = 8;
  auto sampler_ab = Device()->CreateBatchedSampler(2, vocab_size), sampler_ba = Device()->CreateBatchedSampler(2, vocab_size);
  const std::vector<float> logits{0.0f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.6f, 0.7f};
  std::array<DeviceSpan<float>, 2> rows{ToDevice(logits), ToDevice(logits)};
  const std::array<BatchedSamplingParams, 2> params{{{4, 1.0f, 1.0f}, {4, 1.0f, 1.0f}}};
  auto a_ab = sampler_ab->CreateState(11), b_ab = sampler_ab->CreateState(29);
  auto b_ba = sampler_ba->CreateState(29), a_ba = sampler_ba->CreateState(11);
  std::array<BatchedSamplerState*, 2> states_ab{a_ab.get(), b_ab.get()}, states_ba{b_ba.get(), a_ba.get()};
  std::array<DeviceSpan<float>, 2> rows_ba{rows[1], rows[0]};
  for (int step = 0; step < 8; ++step) {
    const auto ab = ToHost(sampler_ab->Sample(rows, params, states_ab, vocab_size));
    const auto ba = ToHost(sampler_ba->Sample(rows_ba, params, states_ba, vocab_size));
    EXPECT_EQ(ab[0], ba[1]);
    EXPECT_EQ(ab[1], ba[0]);
  }
}

// test/cuda_batched_sampler_tests/cuda_batched_sampler_tests.cpp:141-190
void BatchedSamplerKeepsRngRowsAlignedForContiguousBatch() {
  constexpr int batch_size = 20, vocab_size = 8;
  auto contiguous_sampler = Device()->CreateBatchedSampler(batch_size, vocab_size);
  auto separate_sampler = Device()->CreateBatchedSampler(batch_size, vocab_size);
  const std::vector<float> logits{0.0f, 0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.6f, 0.7f};
  std::vector<float> packed_values;
  for (int r = 0; r < batch_size; ++r) packed_values.insert(packed_values.end(), logits.begin(), logits.end());
  auto packed = ToDevice(packed_values);
  std::vector<DeviceSpan<float>> contiguous_rows, separate_rows;
  for (int r = 0; r < batch_size; ++r) {
    contiguous_rows.push_back(packed.subspan(static_cast<size_t>(r) * vocab_size, vocab_size));
    separate_rows.push_back(ToDevice(logits));
  }
  const std::vector<BatchedSamplingParams> params(batch_size, BatchedSamplingParams{4, 1.0f, 1.0f});
  std::vector<std::unique_ptr<BatchedSamplerState>> c_owned, s_owned;
  std::vector<BatchedSamplerState*> c_states, s_states;
  for (int r = 0; r < batch_size; ++r) {
    c_owned.push_back(contiguous_sampler->CreateState(1000 + 7 * r));
    s_owned.push_back(separate_sampler->CreateState(1000 + 7 * r));
    c_states.push_back(c_owned.back().get());
    s_states.push_back(s_owned.back().get());
  }
  bool saw_distinct = false;
  for (int step = 0; step < 4; ++step) {
    const auto c = ToHost(contiguous_sampler->Sample(contiguous_rows, params, c_states, vocab_size));
    const auto s = ToHost(separate_sampler->Sample(separate_rows, params, s_states, vocab_size));
    EXPECT_EQ(c, s);
    for (int r = 0; r < batch_size; ++r) saw_distinct = saw_distinct || c[r] != c[0];
  }
  EXPECT(saw_distinct);
}

// test/cuda_batched_sampler_tests/cuda_batched_sampler_tests.cpp:192-228
void BatchedSamplerLargeVocabulary() {
  constexpr int batch_size = 3, vocab_size = 100001, top_k = 25;
  auto sampler = Device()->CreateBatchedSampler(batch_size, vocab_size);
  std::array<DeviceSpan<float>, batch_size> rows;
  for (int r = 0; r < batch_size; ++r) {
    std::vector<float> logits(vocab_size, 0.0f);
    logits[r + 1] = 100.0f;
    rows[r] = ToDevice(logits);
  }
  const std::array<BatchedSamplingParams, batch_size> params{{{top_k, 0.01f, 1.0f}, {top_k, 0.02f, 1.0f}, {top_k, 0.02f, 1.0f}}};
  std::array<std::unique_ptr<BatchedSamplerState>, batch_size> owned;
  std::array<BatchedSamplerState*, batch_size> states;
  for (int r = 0; r < batch_size; ++r) states[r] = (owned[r] = sampler->CreateState(r)).get();
  EXPECT_EQ(ToHost(sampler->Sample(rows, params, states, vocab_size)), (std::vector<int32_t>{1, 2, 3}));
}

// Known-answer vectors of Philox4x32-10 from Random123's kat_vectors (counter words, key words -> output
// words): all zero, all ones, and the digits of pi.  PhiloxUniform must be the first two output words of
// counter (draw, 0, 0, 0) under key (seed lo, seed hi), top 53 bits, scaled to [0, 1).
void PhiloxKnownAnswers() {
  struct Kat {
    uint32_t c[4], k[2], want[4];
  };
  const Kat kats[] = {
      {{0u, 0u, 0u, 0u}, {0u, 0u}, {0x6627e8d5u, 0xe169c58du, 0xbc57ac4cu, 0x9b00dbd8u}},
      {{0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu}, {0xffffffffu, 0xffffffffu},
       {0x408f276du, 0x41c83b0eu, 0xa20bc7c6u, 0x6d5451fdu}},
      {{0x243f6a88u, 0x85a308d3u, 0x13198a2eu, 0x03707344u}, {0xa4093822u, 0x299f31d0u},
       {0xd16cfe09u, 0x94fdccebu, 0x5001e420u, 0x24126ea1u}},
  };
  for (const Kat& t : kats) {
    uint32_t out[4];
    Philox4x32_10(t.c, t.k, out);
    for (int i = 0; i < 4; ++i) EXPECT_EQ(out[i], t.want[i]);
  }
  // seed 0, draw 0 is the all-zero vector: 0x6627e8d5e169c58d >> 11 = 0xCC4FD1ABC2D38, times 2^-53
  EXPECT_EQ(PhiloxUniform(0, 0), static_cast<double>(0x6627e8d5e169c58dull >> 11) * 0x1.0p-53);
  EXPECT(PhiloxUniform(0, 0) > 0.399 && PhiloxUniform(0, 0) < 0.4);  // 0x6627... / 2^64 = 0.39904...
  // the seed is the key, the draw number the counter: neither aliases the other
  EXPECT(PhiloxUniform(1, 0) != PhiloxUniform(0, 1));
  uint32_t out[4];
  const uint32_t c1[4] = {7u, 1u, 0u, 0u}, k1[2] = {5u, 9u};
  Philox4x32_10(c1, k1, out);
  EXPECT_EQ(PhiloxUniform((9ull << 32) | 5u, (1ull << 32) | 7u),
            static_cast<double>(((static_cast<uint64_t>(out[0]) << 32) | out[1]) >> 11) * 0x1.0p-53);
}

// The distribution of the batched sampler's own draws, after RunSamplingTest (test/sampling_tests.cpp:262-365):
// identical logits in every row with the scores num_top .. 1 on shuffled token ids, a fresh seeded state per
// row and iteration, 5 rows x 1000 iterations; every token's frequency within 0.015 of its probability and
// tokens outside the kept set never drawn.
void BatchedSamplerDistribution(int k, float p, int vocab_size, float temperature) {
  constexpr int batch_size = 5, num_iter = 1000;
  const int num_top = k > 0 ? k : vocab_size;
  std::vector<float> single(vocab_size, 0.0f);
  std::vector<int32_t> top_indices(vocab_size);
  std::iota(top_indices.begin(), top_indices.end(), 0);
  std::mt19937 shuffle_engine(12345);
  std::shuffle(top_indices.begin(), top_indices.end(), shuffle_engine);
  for (int j = 0; j < num_top; ++j) single[top_indices[j]] = static_cast<float>(num_top - j);
  // expected: softmax(score / T) over the kept prefix (the top-p cut keeps the first j with cumulative >= p)
  std::vector<double> expected(num_top);
  double z = 0.0;
  for (int j = 0; j < num_top; ++j) z += (expected[j] = std::exp((num_top - j) / static_cast<double>(temperature)));
  for (double& e : expected) e /= z;
  if (p < 1.0f) {
    double cum = 0.0, kept = 0.0;
    int keep = num_top;
    for (int j = 0; j < num_top; ++j)
      if ((cum += expected[j]) >= p) {
        keep = j + 1;
        break;
      }
    for (int j = 0; j < num_top; ++j) kept += j < keep ? expected[j] : 0.0;
    for (int j = 0; j < num_top; ++j) expected[j] = j < keep ? expected[j] / kept : 0.0;
  }
  auto sampler = Device()->CreateBatchedSampler(batch_size, vocab_size);
  std::vector<float> all;
  for (int b = 0; b < batch_size; ++b) all.insert(all.end(), single.begin(), single.end());
  auto scores = ToDevice(all);
  std::vector<DeviceSpan<float>> rows;
  for (int b = 0; b < batch_size; ++b) rows.push_back(scores.subspan(static_cast<size_t>(b) * vocab_size, vocab_size));
  const std::vector<BatchedSamplingParams> params(batch_size, BatchedSamplingParams{k, p, temperature});
  std::vector<int> counts(vocab_size, 0);
  std::mt19937 engine(12345);
  std::uniform_int_distribution<int> dist;
  for (int i = 0; i < num_iter; ++i) {
    std::vector<std::unique_ptr<BatchedSamplerState>> owned;
    std::vector<BatchedSamplerState*> states;
    for (int b = 0; b < batch_size; ++b) {
      owned.push_back(sampler->CreateState(dist(engine)));
      states.push_back(owned.back().get());
    }
    for (int32_t t : ToHost(sampler->Sample(rows, params, states, vocab_size))) {
      EXPECT(t >= 0 && t < vocab_size);
      if (t >= 0 && t < vocab_size) counts[t]++;
    }
  }
  const double total = batch_size * num_iter;
  int in_top = 0;
  for (int j = 0; j < num_top; ++j) {
    const double actual = counts[top_indices[j]] / total;
    in_top += counts[top_indices[j]];
    if (expected[j] > 0) EXPECT(std::fabs(actual - expected[j]) < 0.015);
    else EXPECT_EQ(counts[top_indices[j]], 0);
  }
  EXPECT_EQ(in_top, batch_size * num_iter);
}
void BatchedSamplerDistributionTopK() { BatchedSamplerDistribution(5, 1.0f, 13, 0.8f); }         // RandomizedSamplingTopK
void BatchedSamplerDistributionTopPAndK() { BatchedSamplerDistribution(7, 0.75f, 21, 1.0f); }    // RandomizedSamplingTopPAndK
void BatchedSamplerDistributionTopPOnly() { BatchedSamplerDistribution(0, 0.95f, 21, 1.0f); }    // RandomizedSamplingTopPOnly
// one stream, consecutive draws (the counter path): 5000 draws of one request at a 100-id vocabulary
void BatchedSamplerStreamIsUniform() {
  constexpr int vocab_size = 100, draws = 5000;
  auto sampler = Device()->CreateBatchedSampler(1, vocab_size);
  auto state = sampler->CreateState(2024);
  std::array<BatchedSamplerState*, 1> states{state.get()};
  std::array<DeviceSpan<float>, 1> rows{ToDevice(std::vector<float>(vocab_size, 0.5f))};
  const std::array<BatchedSamplingParams, 1> params{BatchedSamplingParams{-1, 1.0f, 1.0f}};  // whole vocabulary, flat
  std::vector<int> counts(vocab_size, 0);
  for (int i = 0; i < draws; ++i) counts[ToHost(sampler->Sample(rows, params, states, vocab_size))[0]]++;
  // chi-square over 100 equally likely ids: 99 degrees of freedom, mean 99, sd 14.1; 170 is five sd away
  double chi2 = 0.0;
  for (int c : counts) chi2 += (c - 50.0) * (c - 50.0) / 50.0;
  EXPECT(chi2 < 170.0 && chi2 > 40.0);
}

// A whole generation against the host model of GreedySearch_Cpu: prompt, min-length, repetition
// penalty, no-repeat n-grams, the four selection methods in rotation, EOS padding, rewind, max_length.  Tokens, done
// flag, sequences and the std::mt19937 state must agree after every step.
void GreedyGenerationMatchesCpuSearch() {
  constexpr int batch = 6, vocab = 2003, max_length = 24, min_length = 6;
  GreedyFixture f(batch, vocab, max_length, {5, 17}, /*pad=*/2);
  GreedyModel model(f.config);
  std::mt19937 gen(99), rng(4321), model_rng(4321);
  std::vector<int32_t> prompt(batch * 3);
  for (auto& t : prompt) t = static_cast<int32_t>(gen() % vocab);
  for (int b = 0; b < batch; b += 2) prompt[b * 3 + 2] = prompt[b * 3];  // "x y x": the bigram rule bans y next
  auto prompt_dev = ToDevice(prompt);
  f.search->AppendTokens(prompt_dev);
  model.AppendPrompt(prompt);
  for (int step = 0; !model.done; ++step) {
    auto logits = RandomLogits(gen, static_cast<size_t>(batch) * vocab, 3.0f);
    for (int b = 0; b < batch; ++b) {
      logits[static_cast<size_t>(b) * vocab + prompt[b * 3]] += 6.0f;       // make the penalty matter
      logits[static_cast<size_t>(b) * vocab + prompt[b * 3 + 1]] += 30.0f;  // the banned id would win
      if ((step + b) % 5 == 4) logits[static_cast<size_t>(b) * vocab + 17] = 40.0f;  // drive rows to EOS
    }
    const float penalty = step % 2 ? 1.3f : 1.0f;
    const int ngram = step % 3 == 2 ? 0 : 2;
    f.SetLogits(logits);
    f.search->ApplyMinLength(min_length);
    f.search->ApplyRepetitionPenalty(penalty);
    f.search->ApplyNoRepeatNgram(ngram);
    model.Process(logits, min_length, penalty, ngram);
    if (step == 3) {  // GetLogits must show the processed values
      const auto seen = ToHost(f.search->GetLogits());
      EXPECT(seen == logits);
    }
    switch (step % 4) {
      case 0: f.search->SampleTopKTopP(40, 0.9f, 0.8f, rng); model.Sample(logits, 40, 0.9f, 0.8f, model_rng); break;
      case 1: f.search->SelectTop(); model.SelectTop(logits); break;
      case 2: f.search->SampleTopP(0.7f, 1.1f, rng); model.Sample(logits, 0, 0.7f, 1.1f, model_rng); break;
      case 3: f.search->SampleTopK(300, 0.6f, rng); model.Sample(logits, 300, 0.0f, 0.6f, model_rng); break;
    }
    EXPECT_EQ(f.NextTokens(), model.next_tokens);
    EXPECT_EQ(f.search->IsDone(), model.done);
    EXPECT_EQ(f.search->GetSequenceLength(), model.length);
    EXPECT(rng == model_rng);
    if (g_failures) return;
  }
  for (int b = 0; b < batch; ++b) {
    const auto seq = ToHost(f.search->GetSequence(b));
    EXPECT(std::equal(seq.begin(), seq.end(), model.sequences.begin() + static_cast<size_t>(b) * max_length));
  }
  // RewindTo: next tokens become the tokens stored AT the rewind index (src/search.cpp:313-324)
  f.search->RewindTo(4);
  EXPECT(!f.search->IsDone());
  EXPECT_EQ(f.search->GetSequenceLength(), 4);
  std::vector<int32_t> at_index(batch);
  for (int b = 0; b < batch; ++b) at_index[b] = model.sequences[static_cast<size_t>(b) * max_length + 4];
  EXPECT_EQ(f.NextTokens(), at_index);
  f.search->RewindTo(0);
  EXPECT_EQ(f.NextTokens(), std::vector<int32_t>(batch, 0));
  // CommitToken on a single-row search (speculative decoding's tail)
  GreedyFixture one(1, 16, 4, {3});
  one.search->CommitToken(7);
  EXPECT_EQ(one.search->GetSequenceLength(), 1);
  one.search->CommitToken(3);
  EXPECT(one.search->IsDone());
  EXPECT_EQ(one.search->GetSequenceLength(), 1);
}

// Beam search against orc_beam_select_top + the oracle's BeamSearchScorer, step by step and on the
// final hypotheses (src/search.cpp:101-176,326-400; src/beam_search_scorer.cpp).
void BeamSearchMatchesCpuSearch() {
  constexpr int batch = 3, beams = 4, vocab = 1501, max_length = 12, prompt_len = 2, pad = 1;
  Config config;
  config.model.vocab_size = vocab;
  config.model.eos_token_id = {7};
  config.model.pad_token_id = pad;
  config.search.batch_size = batch;
  config.search.num_beams = beams;
  config.search.num_return_sequences = 2;
  config.search.max_length = max_length;
  config.search.length_penalty = 1.2f;
  config.search.early_stopping = false;
  auto params = std::make_shared<GeneratorParams>(config);
  params->p_device = Device();
  auto search = params->p_device->CreateBeam(*params);
  const int bb = batch * beams;
  const int32_t eos = 7;
  void* scorer = orc_beam_scorer_create(batch, beams, max_length, pad, &eos, 1, 1.2f, 0);
  std::mt19937 gen(5);
  std::vector<int32_t> prompt(batch * prompt_len);
  for (auto& t : prompt) t = 10 + static_cast<int32_t>(gen() % 100);
  auto prompt_dev = ToDevice(prompt);
  search->AppendTokens(prompt_dev);
  std::vector<int32_t> seq(static_cast<size_t>(bb) * max_length, 0), seq_next(seq.size(), 0);
  for (int i = 0; i < bb; ++i)
    for (int j = 0; j < prompt_len; ++j) seq[static_cast<size_t>(i) * max_length + j] = prompt[(i / beams) * prompt_len + j];
  int length = prompt_len;
  EXPECT_EQ(search->GetSequenceLength(), prompt_len);
  std::vector<float> cs(batch * 2 * beams);
  std::vector<int32_t> ct(cs.size()), ci(cs.size());
  while (length < max_length && !orc_beam_scorer_is_done(scorer)) {
    auto logits = RandomLogits(gen, static_cast<size_t>(bb) * vocab, 2.0f);
    for (int i = 0; i < bb; ++i)
      if (gen() % 3 == 0) logits[static_cast<size_t>(i) * vocab + eos] = 7.5f;  // EOS candidates turn up
    for (int i = 0; i < bb; ++i)  // a token of the row's own history would win if it were not banned
      logits[static_cast<size_t>(i) * vocab + seq[static_cast<size_t>(i) * max_length + length - 1]] += 9.0f;
    auto dev = ToDevice(logits);
    search->SetLogits(dev);
    search->ApplyMinLength(4);
    search->ApplyRepetitionPenalty(1.1f);
    search->ApplyNoRepeatNgram(1);
    for (int i = 0; i < bb; ++i) {
      float* row = logits.data() + static_cast<size_t>(i) * vocab;
      orc_apply_min_length(row, vocab, length, 4, &eos, 1);
      orc_apply_repetition_penalty(row, vocab, seq.data() + static_cast<size_t>(i) * max_length, length, 1.1f);
      orc_apply_no_repeat_ngram(row, vocab, seq.data() + static_cast<size_t>(i) * max_length, length, 1);
    }
    search->SelectTop();
    orc_beam_select_top(logits.data(), batch, beams, vocab, orc_beam_scorer_next_scores(scorer), cs.data(), ct.data(), ci.data());
    orc_beam_scorer_process(scorer, seq.data(), length, cs.data(), ct.data(), ci.data());
    orc_beam_append(seq.data(), seq_next.data(), bb, max_length, length, orc_beam_scorer_next_indices(scorer),
                    orc_beam_scorer_next_tokens(scorer));
    seq.swap(seq_next);
    ++length;
    const auto tokens = ToHost(search->GetNextTokens()), indices = ToHost(search->GetNextIndices());
    EXPECT(std::equal(tokens.begin(), tokens.end(), orc_beam_scorer_next_tokens(scorer)));
    EXPECT(std::equal(indices.begin(), indices.end(), orc_beam_scorer_next_indices(scorer)));
    EXPECT_EQ(search->GetSequenceLength(), length);
    EXPECT_EQ(search->IsDone(), orc_beam_scorer_is_done(scorer) != 0 || length == max_length);
    if (g_failures) break;
  }
  orc_beam_scorer_finalize(scorer, seq.data(), length);
  std::vector<int32_t> want(max_length);
  for (int b = 0; b < batch && !g_failures; ++b)
    for (int r = 0; r < 2; ++r) {
      float score = 0;
      const int n = orc_beam_scorer_hyp(scorer, b, r, want.data(), max_length, &score);
      const auto got = ToHost(search->GetSequence(static_cast<size_t>(b) * 2 + r));
      EXPECT_EQ(static_cast<int>(got.size()), n);
      EXPECT(std::equal(got.begin(), got.end(), want.begin()));
    }
  orc_beam_scorer_destroy(scorer);
}

}  // namespace

int main(int argc, char** argv) {
  const std::string filter = argc > 1 ? argv[1] : "";
  const std::pair<const char*, std::function<void()>> tests[] = {
      {"InterfaceEntryPoints", InterfaceEntryPoints},
      {"DeviceBufferContract", DeviceBufferContract},
      {"LogitsMaskUsesPaddedRowStride", LogitsMaskUsesPaddedRowStride},
      {"DeviceFastPaths", DeviceFastPaths},
      {"SamplingTopKOneIsGreedy", SamplingTopKOneIsGreedy},
      {"SamplingRollbackRestoresRandomState", SamplingRollbackRestoresRandomState},
      {"RollbackRestoresDoneEosAndLengthState", RollbackRestoresDoneEosAndLengthState},
      {"EnforcesOneActiveCheckpoint", EnforcesOneActiveCheckpoint},
      {"BatchedSamplerRollbackRestoresRequestRandomStates", BatchedSamplerRollbackRestoresRequestRandomStates},
      {"ExternalSamplingRollbackRestoresSearchTailState", ExternalSamplingRollbackRestoresSearchTailState},
      {"BatchedSamplerHandlesHeterogeneousRows", BatchedSamplerHandlesHeterogeneousRows},
      {"BatchedSamplerPreservesRngAcrossBatchReorder", BatchedSamplerPreservesRngAcrossBatchReorder},
      {"BatchedSamplerKeepsRngRowsAlignedForContiguousBatch", BatchedSamplerKeepsRngRowsAlignedForContiguousBatch},
      {"BatchedSamplerLargeVocabulary", BatchedSamplerLargeVocabulary},
      {"PhiloxKnownAnswers", PhiloxKnownAnswers},
      {"BatchedSamplerDistributionTopK", BatchedSamplerDistributionTopK},
      {"BatchedSamplerDistributionTopPAndK", BatchedSamplerDistributionTopPAndK},
      {"BatchedSamplerDistributionTopPOnly", BatchedSamplerDistributionTopPOnly},
      {"BatchedSamplerStreamIsUniform", BatchedSamplerStreamIsUniform},
      {"GreedyGenerationMatchesCpuSearch", GreedyGenerationMatchesCpuSearch},
      {"BeamSearchMatchesCpuSearch", BeamSearchMatchesCpuSearch},
  };
  int ran = 0, failed = 0;
  for (auto& [name, fn] : tests) {
    if (std::string(name).find(filter) == std::string::npos) continue;
    std::printf("[ RUN  ] %s\n", name);
    std::fflush(stdout);
    const int before = g_failures;
    try {
      fn();
    } catch (const std::exception& e) {
      std::printf("    EXCEPTION: %s\n", e.what());
      ++g_failures;
    }
    const bool ok = g_failures == before;
    std::printf("[ %s ] %s\n", ok ? " OK " : "FAIL", name);
    std::fflush(stdout);
    ++ran;
    failed += !ok;
  }
  std::printf("%d tests, %d failed\n", ran, failed);
  return failed ? 1 : 0;
}
