// Implementation of the MI355X backend classes declared in hip_backend.h.  Everything numerical is a
// call into libmi355x_search (C ABI); this file owns memory, streams, EOS / done bookkeeping and the
// host side of the random draws.
#include "hip_backend.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <mutex>

namespace Generators {
namespace {

struct HipError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

void HipCheck(hipError_t e, const char* what) {
  if (e != hipSuccess) throw HipError(std::string(what) + ": " + hipGetErrorString(e));
}
#define HIP_CHECK(expr) HipCheck((expr), #expr)

void AbiCheck(int rc) {
  if (rc != MI355X_OK) throw std::runtime_error(std::string("mi355x_search: ") + mi355x_search_last_error());
}

hipStream_t g_stream{};
const char* const kHipTag = "hip";

// Device allocation with a pinned host mirror created on first host access.
struct HipMemory final : DeviceBuffer {
  explicit HipMemory(size_t size) : owned_{true} {
    size_in_bytes_ = size;
    HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&p_device_), size ? size : 16));
  }
  HipMemory(void* p, size_t size) : owned_{false} {
    size_in_bytes_ = size;
    p_device_ = static_cast<uint8_t*>(p);
  }
  ~HipMemory() override {
    if (owned_ && p_device_) (void)hipFree(p_device_);
    if (p_cpu_) (void)hipHostFree(p_cpu_);
  }
  const char* GetType() const override { return kHipTag; }
  void AllocateCpu() override {
    if (!p_cpu_) HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&p_cpu_), size_in_bytes_ ? size_in_bytes_ : 16, hipHostMallocDefault));
  }
  void CopyDeviceToCpu() override {
    AllocateCpu();
    HIP_CHECK(hipMemcpyAsync(p_cpu_, p_device_, size_in_bytes_, hipMemcpyDeviceToHost, g_stream));
    HIP_CHECK(hipStreamSynchronize(g_stream));
  }
  void CopyCpuToDevice() override {
    assert(p_cpu_);
    HIP_CHECK(hipMemcpyAsync(p_device_, p_cpu_, size_in_bytes_, hipMemcpyHostToDevice, g_stream));
  }
  void CopyFrom(size_t begin_dest, DeviceBuffer& source, size_t begin_source, size_t size_in_bytes) override {
    if (source.GetType() == kHipTag) {
      HIP_CHECK(hipMemcpyAsync(p_device_ + begin_dest, source.p_device_ + begin_source, size_in_bytes,
                               hipMemcpyDeviceToDevice, g_stream));
    } else {  // a host-resident buffer of another device type: its p_device_ is host memory
      HIP_CHECK(hipMemcpyAsync(p_device_ + begin_dest, source.p_device_ + begin_source, size_in_bytes,
                               hipMemcpyHostToDevice, g_stream));
      HIP_CHECK(hipStreamSynchronize(g_stream));
    }
  }
  void Zero() override { HIP_CHECK(hipMemsetAsync(p_device_, 0, size_in_bytes_, g_stream)); }
  bool owned_;
};

}  // namespace

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3"): counter-based, so a
// request's stream depends only on (seed, draws so far), never on its position in a batch.
void Philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c[4] = {counter[0], counter[1], counter[2], counter[3]};
  uint32_t k[2] = {key[0], key[1]};
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = 0xD2511F53ull * c[0], p1 = 0xCD9E8D57ull * c[2];
    const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c[1] ^ k[0];
    const uint32_t n1 = static_cast<uint32_t>(p1);
    const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c[3] ^ k[1];
    const uint32_t n3 = static_cast<uint32_t>(p0);
    c[0] = n0, c[1] = n1, c[2] = n2, c[3] = n3;
    k[0] += 0x9E3779B9u;
    k[1] += 0xBB67AE85u;
  }
  for (int i = 0; i < 4; ++i) out[i] = c[i];
}

// Draw number `counter` of the stream `seed`: counter words (lo, hi, 0, 0), key words (lo, hi) of the seed;
// the first two output words give the 53 bits of a double in [0, 1).
double PhiloxUniform(uint64_t seed, uint64_t counter) {
  const uint32_t c[4] = {static_cast<uint32_t>(counter), static_cast<uint32_t>(counter >> 32), 0u, 0u};
  const uint32_t k[2] = {static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)};
  uint32_t o[4];
  Philox4x32_10(c, k, o);
  const uint64_t bits53 = ((static_cast<uint64_t>(o[0]) << 32) | o[1]) >> 11;
  return static_cast<double>(bits53) * 0x1.0p-53;
}

namespace {

struct HipBatchedSampler;
struct HipSamplerState final : BatchedSamplerState {
  const HipBatchedSampler* owner{};
  uint64_t seed{};
  uint64_t counter{};
};

// BatchedSampler (src/smartptrs.h:121-138): one fused launch for all rows, heterogeneous (k, p, T),
// a private random stream per request, transactions by counter snapshot.
struct HipBatchedSampler final : BatchedSampler {
  HipBatchedSampler(DeviceInterface& device, size_t max_batch, int vocab) : max_batch_{max_batch}, vocab_{vocab} {
    AbiCheck(mi355x_search_create(0, static_cast<int>(max_batch), vocab, &ctx_));
    tokens_ = device.Allocate<int32_t>(max_batch);
    for (int i = 0; i < 2; ++i) {
      uniforms_[i] = device.Allocate<double>(max_batch);
      HIP_CHECK(hipEventCreateWithFlags(&copied_[i], hipEventDisableTiming));
    }
  }
  ~HipBatchedSampler() override {
    for (hipEvent_t e : copied_) (void)hipEventDestroy(e);
    mi355x_search_destroy(ctx_);
  }

  std::unique_ptr<BatchedSamplerState> CreateState(int random_seed) override {
    auto s = std::make_unique<HipSamplerState>();
    s->owner = this;
    s->seed = random_seed >= 0 ? static_cast<uint64_t>(random_seed)
                               : (static_cast<uint64_t>(std::random_device{}()) << 32) | std::random_device{}();
    return s;
  }
  bool OwnsState(const BatchedSamplerState& state) const override {
    auto* s = dynamic_cast<const HipSamplerState*>(&state);
    return s && s->owner == this;
  }
  bool SupportsTransactions() const override { return true; }
  void SaveStateForTransaction(std::span<BatchedSamplerState* const> states) override {
    saved_.clear();
    for (auto* st : states) {
      auto* s = Own(st);
      saved_.emplace_back(s, s->counter);
    }
  }
  void RestoreStateForTransaction() override {
    for (auto& [s, c] : saved_) s->counter = c;
    saved_.clear();
  }
  void CommitStateForTransaction() noexcept override { saved_.clear(); }

  DeviceSpan<int32_t> Sample(std::span<DeviceSpan<float>> scores, std::span<const BatchedSamplingParams> params,
                             std::span<BatchedSamplerState* const> states, int vocab_size) override {
    const size_t rows = scores.size();
    if (rows == 0 || rows > max_batch_ || params.size() != rows || states.size() != rows)
      throw std::runtime_error("Batched sampler: row, parameter and state counts must match and fit the batch.");
    if (vocab_size != vocab_) throw std::runtime_error("Batched sampler: vocabulary size differs from the one it was created for.");
    // rows at a constant stride are sampled in place; anything else goes by row pointers
    const float* base = scores[0].Span().data();
    ptrdiff_t stride = rows > 1 ? scores[1].Span().data() - base : vocab_size;
    bool strided = stride >= vocab_size;
    for (size_t r = 0; r < rows && strided; ++r) {
      if (scores[r].size() != static_cast<size_t>(vocab_size)) throw std::runtime_error("Batched sampler: a row is not vocab_size long.");
      strided = scores[r].Span().data() == base + static_cast<ptrdiff_t>(r) * stride;
    }
    std::vector<mi355x_sample_params> prm(rows);
    // two uniform buffers take turns: the host mirror about to be rewritten is the one whose copy to the device
    // was issued two calls ago, and its event says when that copy has read it
    const int slot = turn_;
    turn_ ^= 1;
    HIP_CHECK(hipEventSynchronize(copied_[slot]));
    auto u = uniforms_[slot].CpuSpan();
    for (size_t r = 0; r < rows; ++r) {
      prm[r] = mi355x_sample_params{params[r].k, params[r].p, params[r].temperature};
      auto* s = Own(states[r]);
      u[r] = PhiloxUniform(s->seed, s->counter++);
    }
    uniforms_[slot].CopyCpuToDevice();
    HIP_CHECK(hipEventRecord(copied_[slot], g_stream));
    if (strided) {
      AbiCheck(mi355x_sample(ctx_, g_stream, base, stride, static_cast<int>(rows), vocab_, nullptr, prm[0], prm.data(),
                             uniforms_[slot].Span().data(), tokens_.Span().data(), nullptr, nullptr, nullptr, 0));
    } else {
      // rows scattered over memory: their pointers travel inside the kernel arguments, nothing is packed
      std::vector<const void*> ptrs(rows);
      for (size_t r = 0; r < rows; ++r) ptrs[r] = scores[r].Span().data();
      AbiCheck(mi355x_sample_scattered(ctx_, g_stream, ptrs.data(), MI355X_F32, static_cast<int>(rows), vocab_, nullptr,
                                       prm[0], prm.data(), uniforms_[slot].Span().data(), tokens_.Span().data(), nullptr,
                                       nullptr, nullptr, 0));
    }
    return tokens_.subspan(0, rows);
  }

 private:
  HipSamplerState* Own(BatchedSamplerState* st) const {
    auto* s = dynamic_cast<HipSamplerState*>(st);
    if (!s || s->owner != this) throw std::runtime_error("Batched sampler state belongs to another sampler.");
    return s;
  }
  size_t max_batch_;
  int vocab_;
  mi355x_search_ctx* ctx_{};
  DeviceSpan<int32_t> tokens_;
  DeviceSpan<double> uniforms_[2];
  hipEvent_t copied_[2]{};
  int turn_{};
  std::vector<std::pair<HipSamplerState*, uint64_t>> saved_;
};

int DtypeCode(ONNXTensorElementDataType t) {
  if (t == ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT) return MI355X_F32;
  if (t == ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16) return MI355X_F16;
  return 0;
}

struct HipInterface final : DeviceInterface {
  HipInterface() {
    HIP_CHECK(hipSetDevice(0));
    HIP_CHECK(hipStreamCreate(&g_stream));
  }
  ~HipInterface() override {
    if (scratch_) mi355x_search_destroy(scratch_);
  }
  DeviceType GetType() const override { return DeviceType::AMDGPU; }
  void InitOrt(const OrtApi&, Ort::Allocator& allocator) override { ort_allocator_ = &allocator; }
  Ort::Allocator& GetAllocator() override {
    if (!ort_allocator_) throw std::runtime_error("HIP interface: no ONNX Runtime allocator was provided (InitOrt not called)");
    return *ort_allocator_;
  }
  std::unique_ptr<OrtMemoryInfo> GetMemoryInfo() const override {
    throw std::runtime_error("HIP interface: OrtMemoryInfo requires ONNX Runtime");
  }
  std::shared_ptr<DeviceBuffer> AllocateBase(size_t size) override { return std::make_shared<HipMemory>(size); }
  std::shared_ptr<DeviceBuffer> WrapMemoryBase(void* p, size_t size) override { return std::make_shared<HipMemory>(p, size); }
  std::unique_ptr<Search> CreateGreedy(const GeneratorParams& params) override { return std::make_unique<GreedySearch_Hip>(params); }
  std::unique_ptr<Search> CreateBeam(const GeneratorParams& params) override { return std::make_unique<BeamSearch_Hip>(params); }
  std::unique_ptr<BatchedSampler> CreateBatchedSampler(size_t max_batch_size, int vocab_size) override {
    return std::make_unique<HipBatchedSampler>(*this, max_batch_size, vocab_size);
  }
  void Synchronize() override { HIP_CHECK(hipStreamSynchronize(g_stream)); }
  // src/smartptrs.h:208-210: true when the pair is converted on the device, false when the caller
  // has to fall back; equal types throw, as in the CPU and CUDA interfaces.
  bool Cast(void* input, void* output, ONNXTensorElementDataType input_type, ONNXTensorElementDataType output_type,
            size_t element_count) override {
    if (input_type == output_type) throw std::runtime_error("Cast - input and output types are the same");
    std::lock_guard<std::mutex> lock(mutex_);
    const int rc = mi355x_cast(Scratch(1, 64), g_stream, input, static_cast<int>(input_type), output,
                               static_cast<int>(output_type), element_count);
    if (rc == MI355X_E_UNSUPPORTED) return false;
    AbiCheck(rc);
    return true;
  }
  void LaunchAddLogitsMask(float* batch_logits, int batch_beam_size, int vocab_size, const uint32_t* logits_mask) override {
    std::lock_guard<std::mutex> lock(mutex_);
    mi355x_logits_xform xf{};
    xf.mask = logits_mask;
    xf.repetition_penalty = 1.0f;
    AbiCheck(mi355x_process_logits(Scratch(batch_beam_size, vocab_size), g_stream, batch_logits, vocab_size,
                                   batch_beam_size, vocab_size, &xf));
  }
  void GetAvailableMemory(size_t& free_bytes, size_t& total_bytes) override { HIP_CHECK(hipMemGetInfo(&free_bytes, &total_bytes)); }
  void* GetCudaStream() override { return g_stream; }

  bool ArgMax(const void* logits, ONNXTensorElementDataType type, int num_rows, int vocab_size, int32_t* out_tokens) override {
    const int dt = DtypeCode(type);
    if (!dt) return false;
    std::lock_guard<std::mutex> lock(mutex_);
    EnsureSmall(num_rows);
    AbiCheck(mi355x_argmax(Scratch(num_rows, vocab_size), g_stream, logits, dt, vocab_size, num_rows, vocab_size, nullptr,
                           small_tokens_.Span().data()));
    auto host = small_tokens_.CopyDeviceToCpu();
    std::copy_n(host.data(), num_rows, out_tokens);
    return true;
  }
  bool ArgMaxDevice(const void* logits, ONNXTensorElementDataType type, int num_rows, int vocab_size,
                    DeviceSpan<int32_t> out_tokens) override {
    const int dt = DtypeCode(type);
    if (!dt || out_tokens.size() < static_cast<size_t>(num_rows)) return false;
    std::lock_guard<std::mutex> lock(mutex_);
    AbiCheck(mi355x_argmax(Scratch(num_rows, vocab_size), g_stream, logits, dt, vocab_size, num_rows, vocab_size, nullptr,
                           out_tokens.Span().data()));
    return true;
  }
  bool TopKScores(const void* logits, ONNXTensorElementDataType type, int num_rows, int vocab_size, int k,
                  int32_t* out_tokens, float* out_scores) override {
    const int dt = DtypeCode(type);
    if (!dt || k < 1 || k > vocab_size) return false;  // any k, as the CUDA add-on's (src/cuda/interface.cpp:503-553)
    std::lock_guard<std::mutex> lock(mutex_);
    EnsureSmall(static_cast<size_t>(num_rows) * k);
    AbiCheck(mi355x_topk_scores(Scratch(num_rows, vocab_size), g_stream, logits, dt, vocab_size, num_rows, vocab_size, k,
                                small_tokens_.Span().data(), small_scores_.Span().data()));
    HIP_CHECK(hipMemcpyAsync(out_tokens, small_tokens_.Span().data(), sizeof(int32_t) * num_rows * k, hipMemcpyDeviceToHost, g_stream));
    HIP_CHECK(hipMemcpyAsync(out_scores, small_scores_.Span().data(), sizeof(float) * num_rows * k, hipMemcpyDeviceToHost, g_stream));
    HIP_CHECK(hipStreamSynchronize(g_stream));
    return true;
  }

 private:
  mi355x_search_ctx* Scratch(int rows, int vocab) {
    if (!scratch_ || rows > scratch_rows_ || vocab > scratch_vocab_) {
      // The workspace grows in steps (rows to the next power of two from 16, the vocabulary to the next multiple of
      // 64K ids from 256K), so that a caller whose shapes creep up -- one more row of a speculative round, a larger
      // model -- pays for a new context (a synchronisation, hipFree and hipMalloc) a few times, not at every call.
      HIP_CHECK(hipStreamSynchronize(g_stream));
      if (scratch_) mi355x_search_destroy(scratch_);
      scratch_ = nullptr;
      int want_rows = std::max(16, scratch_rows_);
      while (want_rows < rows) want_rows *= 2;
      int want_vocab = std::max(262144, scratch_vocab_);
      while (want_vocab < vocab) want_vocab += 65536;
      scratch_rows_ = want_rows;
      scratch_vocab_ = want_vocab;
      AbiCheck(mi355x_search_create(0, scratch_rows_, scratch_vocab_, &scratch_));
    }
    return scratch_;
  }
  void EnsureSmall(size_t n) {
    if (small_tokens_.size() < n) {
      small_tokens_ = Allocate<int32_t>(n);
      small_scores_ = Allocate<float>(n);
    }
  }
  Ort::Allocator* ort_allocator_{};
  std::mutex mutex_;
  mi355x_search_ctx* scratch_{};
  int scratch_rows_{}, scratch_vocab_{};
  DeviceSpan<int32_t> small_tokens_;
  DeviceSpan<float> small_scores_;
};

void FillEos(const Config::Model& model, mi355x_logits_xform& xf) {
  if (model.eos_token_id.size() > MI355X_MAX_EOS) throw std::runtime_error("more EOS ids than the HIP backend supports");
  xf.n_eos = static_cast<int32_t>(model.eos_token_id.size());
  for (int i = 0; i < xf.n_eos; ++i) xf.eos_ids[i] = model.eos_token_id[i];
}

}  // namespace

DeviceInterface* GetHipInterface() {
  static std::unique_ptr<HipInterface> g_device = std::make_unique<HipInterface>();
  return g_device.get();
}

// ---------------------------------------------------------------------------------------------------------
GreedySearch_Hip::GreedySearch_Hip(const GeneratorParams& params) : Search{params} {
  const int batch = params.search.batch_size;
  AbiCheck(mi355x_search_create(0, batch, params.config.model.vocab_size, &ctx_));
  auto& dev = *params.p_device;
  next_tokens_ = dev.Allocate<int32_t>(batch);
  next_tokens_.Zero();
  std::fill(next_tokens_.CpuSpan().begin(), next_tokens_.CpuSpan().end(), 0);
  sequence_lengths_ = dev.Allocate<int32_t>(params.BatchBeamSize());
  sequence_lengths_.Zero();
  uniforms_ = dev.Allocate<double>(batch);
  uniforms_.Zero();
  draws_used_ = dev.Allocate<int32_t>(1);
  draws_used_.Zero();
  kept_count_ = dev.Allocate<int32_t>(batch);
  state_ = dev.Allocate<int32_t>(batch + 1);
  state_.Zero();
  tx_state_ = dev.Allocate<int32_t>(batch + 1);
  if (params.config.model.eos_token_id.size() > MI355X_MAX_EOS)
    throw std::runtime_error("more EOS ids than the HIP backend supports");
  eos_ids_.assign(params.config.model.eos_token_id.begin(), params.config.model.eos_token_id.end());
}

GreedySearch_Hip::~GreedySearch_Hip() { mi355x_search_destroy(ctx_); }

void GreedySearch_Hip::ResetDone() {
  done_ = false;
  state_.Zero();
}

void GreedySearch_Hip::SetLogits(DeviceSpan<float> logits) {
  next_token_scores_ = logits;
  ClearPending();
}

DeviceSpan<float> GreedySearch_Hip::GetLogits() const {
  Materialize();
  return next_token_scores_;
}

// The three processors are deferred and fused into the next selection in the order the kernels apply
// them (min-length, repetition penalty, n-gram ban: the order RunStandardDecodingStep calls them in,
// src/standard_decoding_strategy.cpp:29-32).  A call that arrives out of that order first applies
// what is pending.
void GreedySearch_Hip::ApplyMinLength(int min_length) {
  if (sequences_.GetSequenceLength() >= min_length) return;
  if (pending_penalty_ != 1.0f || pending_ngram_ > 0) Materialize();
  pending_min_length_ = true;
}

void GreedySearch_Hip::ApplyRepetitionPenalty(float penalty) {
  if (penalty == 1.0f) return;
  if (pending_penalty_ != 1.0f || pending_ngram_ > 0) Materialize();
  pending_penalty_ = penalty;
}

// Search_Cpu::ApplyNoRepeatNgram (src/search.cpp:432-469) on the device (the reference's CUDA search
// rejects the option, src/search.h:125-130).
void GreedySearch_Hip::ApplyNoRepeatNgram(int ngram_size) {
  if (ngram_size <= 0 || sequences_.GetSequenceLength() < ngram_size) return;
  if (pending_ngram_ > 0) Materialize();
  pending_ngram_ = ngram_size;
}

void GreedySearch_Hip::ClearPending() const {
  pending_min_length_ = false;
  pending_penalty_ = 1.0f;
  pending_ngram_ = 0;
}

mi355x_logits_xform* GreedySearch_Hip::PendingXform() {
  if (!pending_min_length_ && pending_penalty_ == 1.0f && pending_ngram_ == 0) return nullptr;
  xf_ = mi355x_logits_xform{};
  xf_.repetition_penalty = pending_penalty_;
  if ((pending_penalty_ != 1.0f || pending_ngram_ > 0) && sequences_.GetSequenceLength() > 0) {
    xf_.history = sequences_.GetSequences().Span().data();
    xf_.history_stride = sequences_.max_length_;
    xf_.history_len = sequences_.GetSequenceLength();
    xf_.no_repeat_ngram_size = pending_ngram_;
  }
  if (pending_min_length_) {
    xf_.apply_min_length = 1;
    FillEos(params_->config.model, xf_);
  }
  return &xf_;
}

void GreedySearch_Hip::Materialize() const {
  auto* self = const_cast<GreedySearch_Hip*>(this);
  if (auto* xf = self->PendingXform()) {
    const int vocab = params_->config.model.vocab_size;
    AbiCheck(mi355x_process_logits(ctx_, g_stream, self->next_token_scores_.Span().data(), vocab,
                                   params_->search.batch_size, vocab, xf));
  }
  ClearPending();
}

// The tail of a step runs on the device like the CUDA search's LaunchNextTokensTail
// (src/cuda/search_cuda.cpp:268-288): finished rows are padded, EOS rows marked, the tokens appended
// and the all-rows-finished flag raised by one kernel over the device-resident state (per-row EOS
// flags followed by the flag).
void GreedySearch_Hip::LaunchTail(int32_t* tokens) {
  const int batch = params_->BatchBeamSize();
  AbiCheck(mi355x_greedy_tail(ctx_, g_stream, tokens, state_.Span().data(), batch, eos_ids_.data(),
                              static_cast<int>(eos_ids_.size()), params_->config.model.pad_token_id,
                              sequences_.GetSequences().Span().data(), sequences_.max_length_,
                              sequences_.GetSequenceLength(), state_.Span().data() + batch));
}

// CompleteGeneration of the CUDA search (src/cuda/search_cuda.cpp:290-308): one synchronisation brings
// back the (padded) tokens and the flag; the length advances only if the step did not finish.
void GreedySearch_Hip::FinishStep() {
  const int batch = params_->BatchBeamSize();
  int32_t all_finished = 0;
  HIP_CHECK(hipMemcpyAsync(next_tokens_.CpuSpan().data(), next_tokens_.Span().data(), sizeof(int32_t) * batch,
                           hipMemcpyDeviceToHost, g_stream));
  HIP_CHECK(hipMemcpyAsync(&all_finished, state_.Span().data() + batch, sizeof(int32_t), hipMemcpyDeviceToHost, g_stream));
  HIP_CHECK(hipStreamSynchronize(g_stream));
  if (all_finished) done_ = true;
  if (done_) return;
  sequences_.AfterAppendNextTokens(next_tokens_, batch);
  if (sequences_.GetSequenceLength() == params_->search.max_length) done_ = true;
}

void GreedySearch_Hip::SelectTop() {
  const int batch = params_->search.batch_size, vocab = params_->config.model.vocab_size;
  AbiCheck(mi355x_argmax(ctx_, g_stream, next_token_scores_.Span().data(), MI355X_F32, vocab, batch, vocab,
                         PendingXform(), next_tokens_.Span().data()));
  ClearPending();
  LaunchTail(next_tokens_.Span().data());
  FinishStep();
}

void GreedySearch_Hip::CommitToken(int32_t token) {
  next_tokens_.CpuSpan()[0] = token;
  next_tokens_.CopyCpuToDevice();
  LaunchTail(next_tokens_.Span().data());
  FinishStep();
}

bool GreedySearch_Hip::BindNextTokensSlot(DeviceSpan<int32_t> slot) {
  if (params_->BatchBeamSize() != 1 || slot.size() != 1) return false;
  bound_slot_ = slot;  // the span's shared_ptr keeps the caller's buffer alive
  return true;
}

// The batched sampler has written this search's token into the bound element of the shared buffer:
// the tail runs on it in place (so the caller's single copy of the buffer to the host already shows
// the padding) and the result is mirrored into next_tokens_.
void GreedySearch_Hip::OnNextTokensSampled() {
  if (bound_slot_.size() != 1) throw std::runtime_error("OnNextTokensSampled without a bound next-token slot");
  LaunchTail(bound_slot_.Span().data());
  HIP_CHECK(hipMemcpyAsync(next_tokens_.Span().data(), bound_slot_.Span().data(), sizeof(int32_t),
                           hipMemcpyDeviceToDevice, g_stream));
  external_pending_ = true;
}

void GreedySearch_Hip::CompleteGeneration() {
  if (!external_pending_) return;
  external_pending_ = false;
  FinishStep();
}

void GreedySearch_Hip::Sample(int k, float p, float temperature, std::mt19937& rng) {
  const int batch = params_->search.batch_size, vocab = params_->config.model.vocab_size;
  const int cap = k > 1 ? std::min(k, vocab) : vocab;
  if (cap > kept_capacity_) {
    kept_ids_ = params_->p_device->Allocate<int32_t>(static_cast<size_t>(batch) * cap);
    kept_probs_ = params_->p_device->Allocate<float>(static_cast<size_t>(batch) * cap);
    kept_capacity_ = cap;
  }
  // The next `batch` canonical doubles of the caller's engine, taken from a copy of it: std::discrete_distribution
  // consumes one per row, none for a row that keeps a single token or is finished, so how many this step uses is
  // only known once the kept sets are.
  {
    std::mt19937 peek = rng;
    auto u = uniforms_.CpuSpan();
    for (int b = 0; b < batch; ++b) u[b] = std::generate_canonical<double, std::numeric_limits<double>::digits>(peek);
    uniforms_.CopyCpuToDevice();
  }
  AbiCheck(mi355x_sample(ctx_, g_stream, next_token_scores_.Span().data(), vocab, batch, vocab, PendingXform(),
                         mi355x_sample_params{k, p, temperature}, nullptr, uniforms_.Span().data(),
                         next_tokens_.Span().data(), kept_count_.Span().data(), kept_ids_.Span().data(),
                         kept_probs_.Span().data(), kept_capacity_));
  ClearPending();
  // SampleCategoricalToken for every row in the order the CPU loop serves them from `rng`, on the device: which
  // of the doubles prepared above a row takes depends on the kept counts of the rows before it.
  AbiCheck(mi355x_draw_in_order(ctx_, g_stream, kept_count_.Span().data(), kept_ids_.Span().data(), kept_probs_.Span().data(),
                                kept_capacity_, batch, state_.Span().data(), uniforms_.Span().data(),
                                next_tokens_.Span().data(), draws_used_.Span().data()));
  LaunchTail(next_tokens_.Span().data());
  HIP_CHECK(hipMemcpyAsync(draws_used_.CpuSpan().data(), draws_used_.Span().data(), sizeof(int32_t), hipMemcpyDeviceToHost, g_stream));
  FinishStep();  // synchronises
  if (draws_used_.CpuSpan()[0] < 0) throw std::runtime_error("a row's kept set outgrew the lists it was sampled from");
  // the engine ends where std::discrete_distribution would have left it: two outputs per consumed double
  rng.discard(2ull * static_cast<unsigned long long>(draws_used_.CpuSpan()[0]));
}

void GreedySearch_Hip::AppendTokens(DeviceSpan<int32_t>& next_tokens) {
  const int batch = params_->search.batch_size;
  auto host = next_tokens.CpuSpan();
  const size_t per_row = host.size() / batch;
  if (sequences_.GetSequenceLength() + per_row > static_cast<size_t>(sequences_.max_length_))
    throw std::runtime_error("User-defined tokens exceed max_length.");
  next_tokens.CopyCpuToDevice();
  HIP_CHECK(hipMemcpy2DAsync(sequences_.GetSequences().Span().data() + sequences_.GetSequenceLength(),
                             sizeof(int32_t) * sequences_.max_length_, next_tokens.Span().data(), sizeof(int32_t) * per_row,
                             sizeof(int32_t) * per_row, batch, hipMemcpyDeviceToDevice, g_stream));
  for (int b = 0; b < batch; ++b) next_tokens_.CpuSpan()[b] = host[b * per_row + per_row - 1];
  next_tokens_.CopyCpuToDevice();
  sequences_.AfterAppendNextTokens(next_tokens, batch);
  ResetDone();  // prompt tokens do not count towards EOS / done (src/search.cpp:298-311)
}

void GreedySearch_Hip::RewindTo(size_t index) {
  ResetDone();
  auto host = next_tokens_.CpuSpan();
  if (index > 0) {
    HIP_CHECK(hipMemcpy2DAsync(host.data(), sizeof(int32_t), sequences_.GetSequences().Span().data() + index,
                               sizeof(int32_t) * sequences_.max_length_, sizeof(int32_t), params_->BatchBeamSize(),
                               hipMemcpyDeviceToHost, g_stream));
    HIP_CHECK(hipStreamSynchronize(g_stream));
  } else {
    std::fill(host.begin(), host.end(), 0);
  }
  next_tokens_.CopyCpuToDevice();
  sequences_.RewindTo(index);
}

void GreedySearch_Hip::SaveStateForTransactionImpl(bool) {
  auto host = next_tokens_.CpuSpan();
  tx_next_tokens_.assign(host.begin(), host.end());
  auto lengths = sequence_lengths_.CopyDeviceToCpu();
  tx_sequence_lengths_.assign(lengths.begin(), lengths.end());
  HIP_CHECK(hipMemcpyAsync(tx_state_.Span().data(), state_.Span().data(), sizeof(int32_t) * state_.size(),
                           hipMemcpyDeviceToDevice, g_stream));
  tx_done_ = done_;
}

void GreedySearch_Hip::RestoreStateForTransactionImpl() {
  std::copy(tx_next_tokens_.begin(), tx_next_tokens_.end(), next_tokens_.CpuSpan().begin());
  next_tokens_.CopyCpuToDevice();
  std::copy(tx_sequence_lengths_.begin(), tx_sequence_lengths_.end(), sequence_lengths_.CpuSpan().begin());
  sequence_lengths_.CopyCpuToDevice();
  external_pending_ = false;
  HIP_CHECK(hipMemcpyAsync(state_.Span().data(), tx_state_.Span().data(), sizeof(int32_t) * state_.size(),
                           hipMemcpyDeviceToDevice, g_stream));
  done_ = tx_done_;
}

// ---------------------------------------------------------------------------------------------------------
BeamSearch_Hip::BeamSearch_Hip(const GeneratorParams& params) : Search{params} {
  assert(params.search.num_beams > 1);
  const int bb = params.BatchBeamSize();
  AbiCheck(mi355x_search_create(0, bb, params.config.model.vocab_size, &ctx_));
  std::vector<int32_t> eos(params.config.model.eos_token_id.begin(), params.config.model.eos_token_id.end());
  AbiCheck(mi355x_beam_scorer_create(ctx_, params.search.batch_size, params.search.num_beams, params.search.max_length,
                                     params.config.model.pad_token_id, eos.data(), static_cast<int>(eos.size()),
                                     params.search.length_penalty, params.search.early_stopping, &scorer_));
  auto& dev = *params.p_device;
  sequence_lengths_ = dev.Allocate<int32_t>(bb);
  sequence_lengths_.Zero();
  const size_t nc = static_cast<size_t>(params.search.batch_size) * 2 * params.search.num_beams;
  cand_scores_ = dev.Allocate<float>(nc);
  cand_tokens_ = dev.Allocate<int32_t>(nc);
  cand_indices_ = dev.Allocate<int32_t>(nc);
}

BeamSearch_Hip::~BeamSearch_Hip() {
  mi355x_beam_scorer_destroy(scorer_);
  mi355x_search_destroy(ctx_);
}

DeviceSpan<int32_t> BeamSearch_Hip::GetNextTokens() {
  return params_->p_device->WrapMemory<int32_t>(
      {const_cast<int32_t*>(mi355x_beam_scorer_next_tokens(scorer_)), static_cast<size_t>(params_->BatchBeamSize())});
}
DeviceSpan<int32_t> BeamSearch_Hip::GetNextIndices() {
  return params_->p_device->WrapMemory<int32_t>(
      {const_cast<int32_t*>(mi355x_beam_scorer_next_indices(scorer_)), static_cast<size_t>(params_->BatchBeamSize())});
}

bool BeamSearch_Hip::IsDone() const {
  int done = 0;
  AbiCheck(mi355x_beam_scorer_is_done(scorer_, g_stream, &done));
  return done != 0;
}

void BeamSearch_Hip::ApplyMinLength(int min_length) {
  if (length_ >= min_length) return;
  mi355x_logits_xform xf{};
  xf.repetition_penalty = 1.0f;
  xf.apply_min_length = 1;
  FillEos(params_->config.model, xf);
  const int vocab = params_->config.model.vocab_size;
  AbiCheck(mi355x_process_logits(ctx_, g_stream, next_token_scores_.Span().data(), vocab, params_->BatchBeamSize(), vocab, &xf));
}

void BeamSearch_Hip::ApplyRepetitionPenalty(float penalty) {
  if (penalty == 1.0f || length_ == 0) return;
  mi355x_logits_xform xf{};
  int len = 0;
  xf.history = mi355x_beam_scorer_sequences(scorer_, &len);
  xf.history_stride = params_->search.max_length;
  xf.history_len = len;
  xf.repetition_penalty = penalty;
  const int vocab = params_->config.model.vocab_size;
  AbiCheck(mi355x_process_logits(ctx_, g_stream, next_token_scores_.Span().data(), vocab, params_->BatchBeamSize(), vocab, &xf));
}

void BeamSearch_Hip::ApplyNoRepeatNgram(int ngram_size) {
  if (ngram_size <= 0 || length_ < ngram_size) return;
  mi355x_logits_xform xf{};
  int len = 0;
  xf.history = mi355x_beam_scorer_sequences(scorer_, &len);
  xf.history_stride = params_->search.max_length;
  xf.history_len = len;
  xf.repetition_penalty = 1.0f;
  xf.no_repeat_ngram_size = ngram_size;
  const int vocab = params_->config.model.vocab_size;
  AbiCheck(mi355x_process_logits(ctx_, g_stream, next_token_scores_.Span().data(), vocab, params_->BatchBeamSize(), vocab, &xf));
}

void BeamSearch_Hip::SelectTop() {
  const int vocab = params_->config.model.vocab_size;
  AbiCheck(mi355x_beam_search_step(scorer_, g_stream, next_token_scores_.Span().data(), MI355X_F32, vocab, vocab));
  ++length_;
  sequences_.RewindTo(length_);  // keeps Search::GetSequenceLength() in step with the device store
}

void BeamSearch_Hip::AppendTokens(DeviceSpan<int32_t>& next_tokens) {
  auto host = next_tokens.CpuSpan();
  const int per_row = static_cast<int>(host.size() / params_->search.batch_size);
  if (per_row > sequences_.max_length_) throw std::runtime_error("User-defined tokens exceed max_length.");
  AbiCheck(mi355x_beam_scorer_set_prompt(scorer_, g_stream, host.data(), per_row));
  length_ = per_row;
  sequences_.RewindTo(length_);
}

DeviceSpan<int32_t> BeamSearch_Hip::GetSequence(size_t index) {
  return GetSequence(index / params_->search.num_return_sequences, index % params_->search.num_return_sequences);
}

DeviceSpan<int32_t> BeamSearch_Hip::GetSequence(size_t batch_id, size_t beam_id) {
  std::vector<int32_t> tokens(params_->search.max_length);
  int n = 0;
  float score = 0.0f;
  const int rc = mi355x_beam_scorer_hypothesis(scorer_, g_stream, static_cast<int>(batch_id), static_cast<int>(beam_id),
                                               tokens.data(), static_cast<int>(tokens.size()), &n, &score);
  if (rc != MI355X_OK) throw std::out_of_range(mi355x_search_last_error());
  auto span = params_->p_device->Allocate<int32_t>(n);
  std::copy_n(tokens.begin(), n, span.CpuSpan().begin());
  span.CopyCpuToDevice();
  hypotheses_.push_back(span);
  return span;
}

}  // namespace Generators

extern "C" uint32_t GetInterfaceVersion() { return Generators::kDeviceInterfaceVersion; }

extern "C" Generators::DeviceInterface* GetInterface(GenaiInterface*, const char* deviceType, const OrtApi*) {
  const std::string t = deviceType ? deviceType : "";
  if (t != "AMDGPU" && t != "HIP" && t != "MI355X") return nullptr;
  return Generators::GetHipInterface();
}
