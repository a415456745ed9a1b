// The plug-in contract a search/sampling backend has to satisfy, restated from the reference so the
// MI355X backend can be compiled and tested where neither the reference headers' dependencies
// (ONNX Runtime) nor its build system exist.  Type names, member names, virtual-function ORDER and
// semantics follow src/smartptrs.h:26-268 (DeviceBuffer, DeviceSpan, BatchedSampler, DeviceType,
// DeviceInterface), src/search.h:31-161 (Search), src/sequences.h:5-42 (Sequences),
// src/generators.h:79-116 (GeneratorParams) and src/config.h (Config::Model / Config::Search fields the
// path reads).  Inside the reference tree, define MI355X_USE_REFERENCE_HEADERS and include
// "generators.h" + "search.h" instead: hip_backend.cpp uses only names that exist there.
//
// ONNX Runtime types appear only as opaque names; no ORT function is called by the backend.
#pragma once
#include <cassert>
#include <cstdint>
#include <cstring>
#include <memory>
#include <random>
#include <span>
#include <stdexcept>
#include <string>
#include <vector>

struct OrtApi;
struct OrtMemoryInfo;
namespace Ort {
struct Allocator;
struct Float16_t;
}  // namespace Ort
enum ONNXTensorElementDataType : int {
  ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED = 0,
  ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT = 1,
  ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32 = 6,
  ONNX_TENSOR_ELEMENT_DATA_TYPE_INT64 = 7,
  ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16 = 10,
  ONNX_TENSOR_ELEMENT_DATA_TYPE_BFLOAT16 = 16,
};

namespace Generators {

struct Search;
struct Sequences;
struct GeneratorParams;
struct ProviderOptions;
struct DeviceInterface;

inline constexpr uint32_t kDeviceInterfaceVersion = 1;  // src/smartptrs.h:171

// ---- memory ------------------------------------------------------------------------------------------
struct DeviceBuffer : std::enable_shared_from_this<DeviceBuffer> {
  virtual ~DeviceBuffer() {}
  virtual const char* GetType() const = 0;
  virtual void AllocateCpu() = 0;
  virtual void CopyDeviceToCpu() = 0;
  virtual void CopyCpuToDevice() = 0;
  virtual void CopyFrom(size_t begin_dest, DeviceBuffer& source, size_t begin_source, size_t size_in_bytes) = 0;
  virtual void Zero() = 0;
  virtual void CopyFromCpu(const void* source, size_t size_in_bytes) {
    assert(size_in_bytes == size_in_bytes_);
    AllocateCpu();
    std::memcpy(p_cpu_, source, size_in_bytes);
    CopyCpuToDevice();
  }
  uint8_t* p_device_{};
  uint8_t* p_cpu_{};
  size_t size_in_bytes_{};
};

template <typename T>
struct DeviceSpan {
  DeviceSpan() = default;
  DeviceSpan(std::shared_ptr<DeviceBuffer>&& memory)
      : p_device_memory_{std::move(memory)}, begin_{}, length_{p_device_memory_->size_in_bytes_ / sizeof(T)} {}

  bool empty() const { return length_ == 0; }
  size_t size() const { return length_; }
  operator DeviceSpan<const T>() const { return DeviceSpan<const T>(*p_device_memory_, begin_, length_); }
  DeviceSpan<T> subspan(size_t begin, size_t length) { return DeviceSpan<T>(*p_device_memory_, begin_ + begin, length); }
  bool SameBufferAs(const DeviceSpan<T>& other) const { return p_device_memory_ == other.p_device_memory_; }

  std::span<T> Span() { return {reinterpret_cast<T*>(p_device_memory_->p_device_) + begin_, length_}; }
  std::span<T> CpuSpan() {
    p_device_memory_->AllocateCpu();
    return {reinterpret_cast<T*>(p_device_memory_->p_cpu_) + begin_, length_};
  }
  std::span<T> CopyDeviceToCpu() {
    p_device_memory_->CopyDeviceToCpu();
    return {reinterpret_cast<T*>(p_device_memory_->p_cpu_) + begin_, length_};
  }
  void CopyCpuToDevice() { p_device_memory_->CopyCpuToDevice(); }
  void CopyFromCpu(std::span<const T> source) {
    assert(source.size() == size());
    p_device_memory_->CopyFromCpu(source.data(), source.size_bytes());
  }
  void Zero() { p_device_memory_->Zero(); }
  void CopyFrom(const DeviceSpan<const T>& source) {
    assert(source.size() == size());
    p_device_memory_->CopyFrom(begin_ * sizeof(T), *source.p_device_memory_, source.begin_ * sizeof(T), length_ * sizeof(T));
  }

 private:
  DeviceSpan(DeviceBuffer& memory, size_t begin, size_t length)
      : p_device_memory_{memory.shared_from_this()}, begin_{begin}, length_{length} {}
  std::shared_ptr<DeviceBuffer> p_device_memory_;
  size_t begin_{}, length_{};
  template <typename U>
  friend struct DeviceSpan;
};

// ---- batched sampler (engine seam) ---------------------------------------------------------------------
struct BatchedSamplerState {
  virtual ~BatchedSamplerState() = default;
};
struct BatchedSamplingParams {
  int k{};
  float p{};
  float temperature{};
};
struct BatchedSampler {
  virtual ~BatchedSampler() = default;
  virtual std::unique_ptr<BatchedSamplerState> CreateState(int random_seed) = 0;
  virtual bool OwnsState(const BatchedSamplerState& state) const = 0;
  virtual bool SupportsTransactions() const { return false; }
  virtual void SaveStateForTransaction(std::span<BatchedSamplerState* const>) {
    throw std::logic_error("Batched sampler does not support transactions.");
  }
  virtual void RestoreStateForTransaction() { throw std::logic_error("Batched sampler does not support transactions."); }
  virtual void CommitStateForTransaction() noexcept {}
  virtual DeviceSpan<int32_t> Sample(std::span<DeviceSpan<float>> scores, std::span<const BatchedSamplingParams> params,
                                     std::span<BatchedSamplerState* const> states, int vocab_size) = 0;
};

enum struct DeviceType { CPU, CUDA, DML, WEBGPU, QnnHtp, QnnGpu, OpenVINO, NvTensorRtRtx, RyzenAI, AMDGPU, MAX };

struct StateSlotDesc {
  uint8_t* base;
  uint64_t slot_bytes;
};

// ---- configuration subset read by the path ---------------------------------------------------------------
struct Config {
  struct Model {
    int pad_token_id{};
    std::vector<int> eos_token_id;
    int vocab_size{};
  } model;
  struct Search {
    bool do_sample{};
    int min_length{};
    int max_length{};
    int batch_size{1};
    int num_beams{1};
    int num_return_sequences{1};
    float repetition_penalty{1.0f};
    int top_k{50};
    float top_p{};
    float temperature{1.0f};
    bool early_stopping{true};
    int no_repeat_ngram_size{};
    float length_penalty{1.0f};
    int random_seed{-1};
  } search;
};

struct GeneratorParams : std::enable_shared_from_this<GeneratorParams> {
  explicit GeneratorParams(const Config& c) : config{c}, search{c.search} {}
  const Config& config;
  Config::Search search;
  int BatchBeamSize() const { return search.num_beams * search.batch_size; }
  DeviceInterface* p_device{};
};

// ---- device interface: virtual order is the ABI ----------------------------------------------------------
struct DeviceInterface {
  virtual ~DeviceInterface() {}
  virtual DeviceType GetType() const = 0;
  virtual void InitOrt(const OrtApi& api, Ort::Allocator& allocator) = 0;
  virtual Ort::Allocator& GetAllocator() = 0;
  virtual std::unique_ptr<OrtMemoryInfo> GetMemoryInfo() const = 0;
  virtual Ort::Allocator* GetHostAccessibleAllocator() { return nullptr; }
  virtual DeviceInterface* GetHostAccessibleDevice() { return nullptr; }
  virtual void InitDeviceAllocators(const ProviderOptions*, int) {}
  virtual int GetDeviceId(const ProviderOptions*) { return 0; }

  template <typename T>
  DeviceSpan<T> Allocate(size_t count) { return DeviceSpan<T>(AllocateBase(sizeof(T) * count)); }
  virtual std::shared_ptr<DeviceBuffer> AllocateBase(size_t size) = 0;
  template <typename T>
  DeviceSpan<T> WrapMemory(std::span<T> memory) {
    return DeviceSpan<T>(WrapMemoryBase(const_cast<std::remove_const_t<T>*>(memory.data()), memory.size_bytes()));
  }
  virtual std::shared_ptr<DeviceBuffer> WrapMemoryBase(void* memory, size_t size) = 0;

  virtual std::unique_ptr<Search> CreateGreedy(const GeneratorParams& params) = 0;
  virtual std::unique_ptr<Search> CreateBeam(const GeneratorParams& params) = 0;
  virtual std::unique_ptr<BatchedSampler> CreateBatchedSampler(size_t, int) { return {}; }
  virtual void Synchronize() = 0;
  virtual bool Cast(void*, void*, ONNXTensorElementDataType, ONNXTensorElementDataType, size_t) { return false; }
  virtual bool UpdatePositionIds(void*, int, int, int, ONNXTensorElementDataType) { return false; }
  virtual bool UpdateAttentionMask(void*, void*, int, int, int, int, bool, ONNXTensorElementDataType) { return false; }
  virtual void LaunchAddLogitsMask(float*, int, int, const uint32_t*) { assert(false); }
  virtual void UpdateCacheIndirection(int32_t*, const int32_t*, const int32_t*, int, int, int, int, int) { assert(false); }
  virtual void ReorderPastStates(void*, const void*, int, int, int, int, int) { assert(false); }
  virtual void CopyCrossQK(float*, void**, int, int, int, int, int, const int*, int, int, int) { assert(false); }
  virtual void CopyCrossQK(Ort::Float16_t*, void**, int, int, int, int, int, const int*, int, int, int) { assert(false); }
  virtual void FinalizeCrossQK(int, int, int, int, int, int, int, const float*, float*, int, const int*) { assert(false); }
  virtual void FinalizeCrossQK(int, int, int, int, int, int, int, const Ort::Float16_t*, Ort::Float16_t*, int, const int*) { assert(false); }
  virtual void GetAvailableMemory(size_t&, size_t&) { assert(false); }
  virtual void ShapeInitSessionProviderOptions(ProviderOptions&, const ProviderOptions*) const {}
  virtual bool SupportsPhi3RopeRewind(const Config&) const { return true; }
  virtual void* GetCudaStream() {
    assert(false);
    return nullptr;
  }
  virtual bool ArgMax(const void*, ONNXTensorElementDataType, int, int, int32_t*) { return false; }
  virtual bool TopKScores(const void*, ONNXTensorElementDataType, int, int, int, int32_t*, float*) { return false; }
  virtual bool ArgMaxDevice(const void*, ONNXTensorElementDataType, int, int, DeviceSpan<int32_t>) { return false; }
  virtual bool CopyStateSlots(const void*, int, int, int) { return false; }
};

// ---- sequences -------------------------------------------------------------------------------------------
struct Sequences {
  explicit Sequences(const GeneratorParams& params) : max_length_{params.search.max_length}, current_length_{0} {
    const size_t n = static_cast<size_t>(params.BatchBeamSize()) * max_length_;
    sequences_ = params.p_device->Allocate<int32_t>(n);
    if (params.search.num_beams > 1) sequences_next_ = params.p_device->Allocate<int32_t>(n);
  }
  DeviceSpan<int32_t> GetSequence(size_t batch_beam_index) {
    return sequences_.subspan(batch_beam_index * max_length_, current_length_);
  }
  DeviceSpan<int32_t> GetSequences() { return sequences_; }
  DeviceSpan<int32_t> GetNextSequences() { return sequences_next_; }
  int GetSequenceLength() const { return current_length_; }
  void AfterAppendNextTokens(DeviceSpan<int32_t>& next_tokens, size_t batch_beam_size) {
    current_length_ += static_cast<int>(next_tokens.size() / batch_beam_size);
    if (!sequences_next_.empty()) std::swap(sequences_, sequences_next_);
  }
  void RewindTo(size_t index) { current_length_ = static_cast<int>(index); }
  const int max_length_;

 private:
  DeviceSpan<int32_t> sequences_, sequences_next_;
  int current_length_;
};

// ---- search: virtual order is the ABI ----------------------------------------------------------------------
struct Search {
  explicit Search(const GeneratorParams& params) : params_{params.shared_from_this()}, sequences_{*params_} {}
  virtual ~Search() = default;
  virtual DeviceSpan<int32_t> GetNextTokens() = 0;
  virtual DeviceSpan<int32_t> GetNextIndices() = 0;
  virtual DeviceSpan<int32_t> GetSequenceLengths() = 0;
  int GetSequenceLength() const { return sequences_.GetSequenceLength(); }
  virtual DeviceSpan<int32_t> GetSequence(size_t index) { return sequences_.GetSequence(index); }
  virtual DeviceSpan<float> GetLogits() const = 0;
  virtual void SetLogits(DeviceSpan<float> logits) = 0;
  virtual bool IsDone() const = 0;
  virtual void DeferCompletion(bool) {}
  virtual void CompleteGeneration() {}
  virtual bool BindNextTokensSlot(DeviceSpan<int32_t>) { return false; }
  virtual bool SupportsBatchedSampling() const { return false; }
  virtual void OnNextTokensSampled() {}

  void SaveStateForTransaction() { StartTransactionCheckpoint(true); }
  void SaveStateForExternalSamplingTransaction() { StartTransactionCheckpoint(false); }
  void QueueStateRestoreForTransaction() {
    if (!transaction_checkpoint_active_) throw std::logic_error("Search transaction checkpoint is not active.");
    if (transaction_restore_pending_) throw std::logic_error("Search transaction restore is already pending.");
    sequences_.RewindTo(transaction_sequence_length_);
    RestoreStateForTransactionImpl();
    transaction_restore_pending_ = true;
  }
  void RestoreStateForTransaction() {
    QueueStateRestoreForTransaction();
    SynchronizeStateForTransactionImpl();
    CompleteStateRestoreForTransaction();
  }
  void CompleteStateRestoreForTransaction() {
    if (!transaction_checkpoint_active_ || !transaction_restore_pending_)
      throw std::logic_error("Search transaction restore is not pending.");
    CompleteStateRestoreForTransactionImpl();
    transaction_restore_pending_ = false;
    transaction_checkpoint_active_ = false;
  }
  void CommitStateForTransaction() {
    if (!transaction_checkpoint_active_ || transaction_restore_pending_)
      throw std::logic_error("Search transaction checkpoint is not active.");
    transaction_checkpoint_active_ = false;
  }

  virtual void SelectTop() = 0;
  virtual void CommitToken(int32_t) { assert(false); }
  virtual void SampleTopP(float, float, std::mt19937&) { assert(false); }
  virtual void SampleTopK(int, float, std::mt19937&) { assert(false); }
  virtual void SampleTopKTopP(int, float, float, std::mt19937&) { assert(false); }
  virtual void ApplyMinLength(int min_length) = 0;
  virtual void ApplyRepetitionPenalty(float penalty) = 0;
  virtual void ApplyNoRepeatNgram(int ngram_size) {
    if (ngram_size <= 0) return;
    throw std::runtime_error("no_repeat_ngram_size is only supported for CPU search");
  }
  virtual void AppendTokens(DeviceSpan<int32_t>&) { assert(false); }
  virtual void RewindTo(size_t) { assert(false); }

  std::shared_ptr<const GeneratorParams> params_;
  Sequences sequences_;

 protected:
  virtual void SaveStateForTransactionImpl(bool) {}
  virtual void RestoreStateForTransactionImpl() {}
  virtual void SynchronizeStateForTransactionImpl() {}
  virtual void CompleteStateRestoreForTransactionImpl() {}

 private:
  void StartTransactionCheckpoint(bool checkpoint_local_state) {
    if (transaction_checkpoint_active_) throw std::logic_error("Search transaction checkpoint is already active.");
    transaction_sequence_length_ = sequences_.GetSequenceLength();
    SaveStateForTransactionImpl(checkpoint_local_state);
    transaction_checkpoint_active_ = true;
  }
  bool transaction_checkpoint_active_{};
  bool transaction_restore_pending_{};
  int transaction_sequence_length_{};
};

}  // namespace Generators

// Host services the loader hands to an add-on (src/cuda/interface.h:4-21); unused by this backend but
// part of the GetInterface signature.
struct GenaiInterface;
