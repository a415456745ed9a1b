/* mi355x_search.h -- C ABI of the MI355X (gfx950) search & sampling library.
 *
 * One entry point per group of functions on onnxruntime-genai's per-step search-and-sampling path.
 * Each declaration cites the reference interface it stands in for (paths relative to the reference
 * tree).  All pointers marked "device" are HIP device pointers on the context's GPU; "host" pointers
 * are ordinary host memory.  Every call is asynchronous on `stream` (a hipStream_t passed as void*)
 * unless stated otherwise.  Return value: 0 on success, a negative MI355X_E_* code on failure, with a
 * thread-local message available from mi355x_search_last_error().
 *
 * Graph capture: every entry point only launches kernels on `stream` (mi355x_sample* with per-row parameters that
 * put rows in several selection modes also on two streams of the context's own, which fork from `stream` behind
 * an event and join it again before the call returns: part of the capture like any fork and join), with workspace
 * from the context, and can be captured into a HIP graph -- except the synchronous ones (create / destroy, *_is_done,
 * *_hypothesis, *_fallback_rows, *_wait_gave_up, beam_scorer_set_prompt) and the two that advance a scorer's
 * host-side state (mi355x_beam_scorer_step, mi355x_beam_search_step: the sequence length and the buffer the
 * sequences live in are part of the launch, so a replay would repeat one step; they return
 * MI355X_E_UNSUPPORTED on a capturing stream).  The three calls that take a table from a caller's HOST array
 * (mi355x_sample* with per-row parameters for more than 64 rows, mi355x_logits_handoff with token_index,
 * mi355x_kv_gather) copy it into pinned memory of the context when they are called and record a copy from
 * there, so the caller's array is not read again at a replay; every such call captured takes one of the
 * context's 56 permanent staging slots (MI355X_E_UNSUPPORTED once they are used up).
 *
 * Versions: MI355X_ABI_VERSION names the layout of the structures below and the set of entry points;
 * mi355x_search_abi_version() returns the value the loaded library was built with, so a caller built
 * against another header can tell before it passes a structure.
 *
 * Tie rule everywhere: equal scores are ordered by ascending index (lowest index wins).
 * -0.0 and +0.0 compare equal.  NaN scores order below every number, except in mi355x_argmax, which
 * reproduces the reference's strict '>' scan (a NaN at index 0 is never beaten).
 */
#ifndef MI355X_SEARCH_H_
#define MI355X_SEARCH_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355X_OK 0
#define MI355X_E_INVALID (-1)     /* bad argument (null pointer, size out of range, ...) */
#define MI355X_E_HIP (-2)         /* a HIP runtime call failed */
#define MI355X_E_CAPACITY (-3)    /* rows/vocab exceed what the context was created for */
#define MI355X_E_UNSUPPORTED (-4) /* valid request this build does not implement */

#define MI355X_MAX_EOS 16

#define MI355X_ABI_VERSION 3
int mi355x_search_abi_version(void);

/* Element type of a logits / KV tensor (values follow ONNXTensorElementDataType where one exists:
 * FLOAT = 1, FLOAT16 = 10, the types DeviceInterface::ArgMax/TopKScores accept, src/smartptrs.h:249). */
#define MI355X_F32 1
#define MI355X_I32 6
#define MI355X_I64 7
#define MI355X_F16 10
#define MI355X_BF16 16

typedef struct mi355x_search_ctx mi355x_search_ctx;

/* Logits processing fused into every selection entry point, applied per element in the reference's
 * order (src/standard_decoding_strategy.cpp:24-32; LogitsPenaltyProcessor::Apply,
 * src/sampling_distribution.h:100-110): grammar mask -> min-length -> repetition penalty ->
 * no-repeat-n-gram ban.
 *   mask     device [rows, (vocab-1)/32+1] uint32, bit set = token allowed, else the logit becomes
 *            lowest() (src/constrained_logits_processor.cpp:246-258, layout :174-183); NULL = none.
 *   history  device [rows, history_stride] int32 token ids, the first history_len of each row valid
 *            (Sequences::GetSequence, src/sequences.h:18); every DISTINCT in-range id has its logit
 *            s replaced by s<0 ? s*penalty : s/penalty (src/sampling_distribution.h:41-62).
 *            NULL or penalty == 1.0f = none.  history_stride 0 lets all rows share one buffer.  (All
 *            history_stride ids of a row may be read, whatever its length: the buffer holds them all.)
 *   eos_ids  with apply_min_length != 0 each in-range id gets lowest()
 *            (src/sampling_distribution.h:26-35; the caller evaluates current_length < min_length).
 *   history_lens  optional device [rows] int32: row r uses the first history_lens[r] ids of its
 *            history row instead of history_len, and -- when min_length > 0 -- gets the EOS masking
 *            only if history_lens[r] < min_length.  This is the (current_length, prefix) pair of
 *            ComputeTargetTokenSelection (src/speculative_sampling.h:59-79), where the verify rows
 *            of one sequence see prefixes that grow by one proposal token per row
 *            (src/speculative_decoding_strategy.cpp:645-656).
 *   no_repeat_ngram_size  n > 0: every id that followed an earlier occurrence of the row's last n-1
 *            history ids gets lowest(), after the penalty (ApplyNoRepeatNgramToLogits,
 *            src/sampling_distribution.h:64-79; Search_Cpu::ApplyNoRepeatNgram,
 *            src/search.cpp:432-469).  Needs history.
 *   mask_allowed_max  optional promise about `mask`: no row's mask has more than this many bits set
 *            (0 = unknown).  The grammar engine builds the mask on the host (ComputeMask,
 *            src/constrained_logits_processor.cpp:157-188), where the count is one popcount pass.  When the
 *            bound fits the sort buffer of the sparse-mask kernel (about 16000 ids together with the history),
 *            nucleus rows are finished by that one kernel and the dense kernels are not launched at all; a row
 *            that breaks the promise is still sampled correctly, by the exact path (slowly).
 */
typedef struct mi355x_logits_xform {
  const uint32_t* mask;
  const int32_t* history;
  int32_t history_stride;
  int32_t history_len;
  float repetition_penalty;
  int32_t apply_min_length;
  int32_t n_eos;
  int32_t eos_ids[MI355X_MAX_EOS];
  const int32_t* history_lens;
  int32_t min_length;
  int32_t no_repeat_ngram_size;
  int32_t mask_allowed_max;
} mi355x_logits_xform;

/* (k, p, temperature) of one row: BatchedSamplingParams, src/smartptrs.h:113-117.  Meaning as in
 * ComputeSampledCategorical (src/sampling_distribution.h:233-297): k > 1 keeps the k best, then
 * 0 < p < 1 cuts the nucleus inside them; k <= 1 takes the nucleus of the whole vocabulary
 * (p <= 0 keeps the single best token, i.e. greedy). */
typedef struct mi355x_sample_params {
  int32_t k;
  float p;
  float temperature;
} mi355x_sample_params;

/* Creates a context on HIP device `device` with workspace for up to max_rows rows of up to max_vocab
 * logits (allocates device memory; synchronous).  One context serves one stream at a time. */
int mi355x_search_create(int device, int max_rows, int max_vocab, mi355x_search_ctx** out);
void mi355x_search_destroy(mi355x_search_ctx* ctx);
const char* mi355x_search_last_error(void);
/* Device bytes held by the context's workspace. */
size_t mi355x_search_workspace_bytes(const mi355x_search_ctx* ctx);

/* In-place logits processing: stands in for DeviceInterface::LaunchAddLogitsMask
 * (src/smartptrs.h:218), Search::ApplyMinLength and Search::ApplyRepetitionPenalty
 * (src/search.h:122-123; CPU src/search.cpp:407-430).  logits: device [rows] rows of `vocab` floats,
 * row r starting at logits + r*row_stride. */
int mi355x_process_logits(mi355x_search_ctx* ctx, void* stream, float* logits, int64_t row_stride,
                          int rows, int vocab, const mi355x_logits_xform* xf);

/* Greedy argmax per row: GreedySearch_Cpu::SelectTop / ArgMax (src/search.cpp:178-192,
 * src/search.h:9-29) and DeviceInterface::ArgMaxDevice (src/smartptrs.h:258).  dtype MI355X_F32,
 * MI355X_F16 (widened exactly like FastFloat16ToFloat32, src/models/utils.cpp:103-109) or MI355X_BF16
 * (BFloat16ToFloat32, :84-86).
 * xf may be NULL.  out_tokens: device [rows] int32. */
int mi355x_argmax(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype,
                  int64_t row_stride, int rows, int vocab, const mi355x_logits_xform* xf,
                  int32_t* out_tokens);

/* mi355x_argmax without a context and without any allocation.  It has no counterpart in the
 * reference: it exists for callers that cannot allocate device memory where they call (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc).  Same arguments, same results
 * and same errors as mi355x_argmax, except:
 *   - the device is the calling thread's current HIP device, which `stream` must belong to;
 *   - the kernels' per-row partial results live in a static device array of
 *     MI355X_ARGMAX_STATIC_MAX_ROWS rows (48 KiB, held by every GPU the library is loaded on until
 *     the process ends); more rows fail with MI355X_E_CAPACITY;
 *   - xf->no_repeat_ngram_size > 0 fails with MI355X_E_UNSUPPORTED (its bitmaps need a context).
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream, or otherwise ordered, are safe.  The call itself clears the slots
 * it is about to use (with a kernel, no memset node) and calls neither hipMalloc nor hipFree.
 * The array's address is looked up once per device, by mi355x_search_create or by the first call; a first call
 * on a stream that records a graph is refused (MI355X_E_UNSUPPORTED), later ones can be captured. */
#define MI355X_ARGMAX_STATIC_MAX_ROWS 4096
int mi355x_argmax_static(void* stream, const void* logits, int dtype, int64_t row_stride, int rows,
                         int vocab, const mi355x_logits_xform* xf, int32_t* out_tokens);

/* Per-row k best (token id, raw fp32 score), best first: DeviceInterface::TopKScores
 * (src/smartptrs.h:254).  dtype MI355X_F32, MI355X_F16 or MI355X_BF16 (the scores of sixteen-bit rows are
 * the widened values).  out_tokens/out_scores: device [rows, k].  1 <= k <= vocab: up to 64 from the fused
 * kernel's candidate lists, up to 8192 from the candidate lists of the large-k sampling route, beyond that
 * from the exact path's whole-row sort (the CUDA add-on serves any k as well, src/cuda/interface.cpp:503-553). */
int mi355x_topk_scores(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype,
                       int64_t row_stride, int rows, int vocab, int k, int32_t* out_tokens,
                       float* out_scores);

/* Top-k / top-p / top-k+top-p sampling of one token per row: GreedySearch_Cpu::SampleTopK,
 * SampleTopP, SampleTopKTopP (src/search.cpp:203-254) = ComputeSampledCategorical +
 * SampleCategoricalToken (src/sampling_distribution.h:218-297), and BatchedSampler::Sample
 * (src/smartptrs.h:134-137).
 *   params            used for every row when per_row_params is NULL.
 *   per_row_params    HOST [rows], heterogeneous parameters (copied by the call: up to 64 rows travel
 *                     inside the kernel arguments, larger batches through pinned staging memory of the
 *                     context and one asynchronous copy to a table in it).
 *   uniforms          device [rows] doubles in [0,1): row r's categorical draw, the value
 *                     std::discrete_distribution would take from generate_canonical<double,53>.
 *                     A row whose kept set has one token ignores its uniform.
 *   out_tokens        device [rows] int32 -- or pinned host memory the device can address (hipHostMalloc): the
 *                     kernel stores every row's token there itself, as the reference mirrors its results through
 *                     pinned memory (src/cuda/interface.cpp:51-60), so no copy follows the launch; a host that
 *                     filled the buffer with -1 sees the tokens arrive without synchronising the stream.  The
 *                     same holds for the out_tokens of mi355x_argmax and for next_tokens / done of
 *                     mi355x_greedy_tail.
 *   kept_count/kept_ids/kept_probs  optional device outputs [rows], [rows,kept_capacity] x2: the
 *                     kept distribution (ids best first, renormalised fp32 probabilities), truncated
 *                     to kept_capacity entries per row; kept_count holds the untruncated size.
 */
int mi355x_sample(mi355x_search_ctx* ctx, void* stream, const float* logits, int64_t row_stride,
                  int rows, int vocab, const mi355x_logits_xform* xf, mi355x_sample_params params,
                  const mi355x_sample_params* per_row_params, const double* uniforms,
                  int32_t* out_tokens, int32_t* kept_count, int32_t* kept_ids, float* kept_probs,
                  int kept_capacity);

/* mi355x_sample on rows of any supported element type: dtype MI355X_F32, MI355X_F16 or MI355X_BF16, row_stride
 * in elements.  Sixteen-bit logits are read as they are and widened in registers exactly as the reference
 * widens them before the search sees them (Logits::Get casts the model's fp16/bf16 output to fp32,
 * src/models/logits.cpp:72-76, with FastFloat16ToFloat32 / BFloat16ToFloat32, src/models/utils.cpp:84-109):
 * the results equal mi355x_sample on the widened copy, without the pass that writes and re-reads it. */
int mi355x_sample_typed(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype,
                        int64_t row_stride, int rows, int vocab, const mi355x_logits_xform* xf,
                        mi355x_sample_params params, const mi355x_sample_params* per_row_params,
                        const double* uniforms, int32_t* out_tokens, int32_t* kept_count,
                        int32_t* kept_ids, float* kept_probs, int kept_capacity);

/* mi355x_sample_typed on rows that do not lie at a constant stride: BatchedSampler::Sample receives one span per
 * request (src/smartptrs.h:134-137; the CUDA sampler packs such rows with a kernel first,
 * src/cuda/cuda_sampling.cu:390-449).  row_ptrs: HOST array of `rows` device pointers, one per row of `vocab`
 * elements; they travel inside the kernel arguments (64 rows per launch), so nothing is packed or copied and
 * the call can be captured into a graph.  Row r of mask / history / uniforms / outputs belongs to row_ptrs[r]. */
int mi355x_sample_scattered(mi355x_search_ctx* ctx, void* stream, const void* const* row_ptrs, int dtype,
                            int rows, int vocab, const mi355x_logits_xform* xf,
                            mi355x_sample_params params, const mi355x_sample_params* per_row_params,
                            const double* uniforms, int32_t* out_tokens, int32_t* kept_count,
                            int32_t* kept_ids, float* kept_probs, int kept_capacity);

/* Softmax / log-softmax with temperature, in place, one row per `vocab` floats:
 * Softmax and LogSoftMax (src/softmax.h:26-47).  Sums are accumulated in index order in fp32 exactly
 * as the reference does, so results are bit-identical to it. */
int mi355x_softmax(mi355x_search_ctx* ctx, void* stream, float* scores, int64_t row_stride, int rows,
                   int vocab, float temperature, int log_softmax);

/* Beam-search candidate selection: BeamSearch_Cpu::SelectTop up to the scorer call
 * (src/search.cpp:101-164).  logits: device [batch*beams] rows (fp32, fp16 or bf16); beam_scores: device
 * [batch*beams].  Per batch entry the 2*beams best of the beams*vocab values
 * log_softmax(row)+beam_score, best first: out_scores/out_tokens/out_beam_indices device
 * [batch, 2*beams] (beam index relative to the batch entry).  beams <= 16. */
int mi355x_beam_select(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype,
                       int64_t row_stride, int batch, int beams, int vocab, const float* beam_scores,
                       float* out_scores, int32_t* out_tokens, int32_t* out_beam_indices);

/* Device-resident BeamSearchScorer + Sequences (src/beam_search_scorer.{h,cpp}, src/sequences.{h,cpp},
 * BeamSearch_Cpu::AppendNextTokensToSequences src/search.cpp:354-381). */
typedef struct mi355x_beam_scorer mi355x_beam_scorer;
int mi355x_beam_scorer_create(mi355x_search_ctx* ctx, int batch, int beams, int max_length,
                              int pad_token_id, const int32_t* eos_ids, int n_eos,
                              float length_penalty, int early_stopping, mi355x_beam_scorer** out);
void mi355x_beam_scorer_destroy(mi355x_beam_scorer* s);
/* Sets the prompt: tokens HOST [batch, prompt_len], replicated to every beam (BeamSearch_Cpu::AppendTokens,
 * src/search.cpp:326-343). */
int mi355x_beam_scorer_set_prompt(mi355x_beam_scorer* s, void* stream, const int32_t* tokens,
                                  int prompt_len);
/* One BeamSearchScorer::Process + AppendNextTokensToSequences on the candidates produced by
 * mi355x_beam_select (device [batch, 2*beams]). */
int mi355x_beam_scorer_step(mi355x_beam_scorer* s, void* stream, const float* cand_scores,
                            const int32_t* cand_tokens, const int32_t* cand_beam_indices);
/* BeamSearch_Cpu::SelectTop as one call (src/search.cpp:101-176: log-softmax of every beam's row plus its running
 * score, the 2*beams best candidates per batch entry, BeamSearchScorer::Process, AppendNextTokensToSequences):
 * mi355x_beam_select with the scorer's own next scores as beam scores and candidate buffers of its own, then
 * mi355x_beam_scorer_step.  logits: device [batch*beams, row_stride], fp32, fp16 or bf16. */
int mi355x_beam_search_step(mi355x_beam_scorer* s, void* stream, const void* logits, int dtype,
                            int64_t row_stride, int vocab);
/* Device views valid until the next step: next beam scores [batch*beams], tokens, indices
 * (GetNextScores/GetNextTokens/GetNextIndices, src/beam_search_scorer.h:52-54). */
const float* mi355x_beam_scorer_next_scores(const mi355x_beam_scorer* s);
const int32_t* mi355x_beam_scorer_next_tokens(const mi355x_beam_scorer* s);
const int32_t* mi355x_beam_scorer_next_indices(const mi355x_beam_scorer* s);
/* Current sequences: device [batch*beams, max_length]; *length = tokens valid per row. */
const int32_t* mi355x_beam_scorer_sequences(const mi355x_beam_scorer* s, int* length);
/* Synchronises `stream` and reports IsDone() (all batch entries done or max_length reached). */
int mi355x_beam_scorer_is_done(mi355x_beam_scorer* s, void* stream, int* done);
/* BeamSearchScorer::Finalize + GetBeamHypotheses (src/beam_search_scorer.cpp:173-202): synchronous;
 * copies hypothesis `index` (0 = best) of batch entry `batch` to HOST out (capacity tokens), returns
 * its length in *length and its score in *score. */
int mi355x_beam_scorer_hypothesis(mi355x_beam_scorer* s, void* stream, int batch, int index,
                                  int32_t* out, int capacity, int* length, float* score);

/* KV-cache beam reorder: DefaultKeyValueCache::PickPastState (src/models/kv_cache.cpp:710-740):
 * for every tensor t and row j, past[t][j] = present[t][beam_indices[j]], blocks of block_bytes
 * bytes (any size; blocks and tensors aligned to 16 bytes move with 128-bit accesses, others with the
 * widest access they are aligned to).  present/past: HOST arrays of n_tensors device pointers (copied by the
 * call into pinned staging memory of the context, from where one asynchronous copy takes them to the device);
 * beam_indices: device [rows]. */
int mi355x_kv_gather(mi355x_search_ctx* ctx, void* stream, const void* const* present,
                     void* const* past, int n_tensors, const int32_t* beam_indices, int rows,
                     size_t block_bytes);

/* Speculative-decoding verification on dense distributions: ComputeAcceptProb, the accept loop of
 * SpeculativeDecodingStrategy::RunRound (src/speculative_decoding_strategy.cpp:718-762) and
 * SampleCorrectionToken / bonus sampling (src/speculative_sampling.h:32-57,140-146).
 *   p_target, p_draft  device [batch, K+1, vocab] fp32 probabilities (row K of p_target = bonus row)
 *   draft_tokens       device [batch, K]
 *   accept_u           device [batch, K] floats in [0,1) (uniform_real_distribution<float> draws)
 *   sample_u           device [batch] doubles in [0,1) (the round's single categorical draw)
 *   accepted_len, final_token  device [batch] outputs.
 */
int mi355x_spec_verify(mi355x_search_ctx* ctx, void* stream, const float* p_target,
                       const float* p_draft, const int32_t* draft_tokens, const float* accept_u,
                       const double* sample_u, int batch, int K, int vocab, int32_t* accepted_len,
                       int32_t* final_token);

/* Speculative-decoding verification on SPARSE selections, the form the reference's strategies use:
 * the kept sets mi355x_sample returns (kept_count / kept_ids / kept_probs) for the K+1 verify rows of
 * each sequence are the TargetTokenSelection rows of SpeculativeDecodingStrategy::RunRound.
 *   target_count [batch, K+1], target_ids / target_probs [batch, K+1, target_capacity]  device; row i
 *                judges proposal token i, row K supplies the bonus token.
 *   draft_count [batch, K], draft_ids / draft_probs [batch, K, draft_capacity]  device; the proposal's
 *                own distributions (mode 0 only, else NULL).
 *   proposal     device [batch, K] proposed token ids.
 *   mode 0       stochastic accept loop (src/speculative_decoding_strategy.cpp:718-762) with
 *                GetSparseTokenProbability, ComputeAcceptProb, SampleCorrectionToken and
 *                SampleSparseToken (src/speculative_sampling.h:22-57,140-146).  accept_u: device
 *                [batch, K] uniform_real_distribution<float> draws in the order the loop takes them;
 *                sample_u: device [batch, K+1] doubles, entry e = the generate_canonical<double,53>
 *                value the engine would yield after e accept draws (the loop's single categorical draw
 *                follows one accept draw per evaluated position).
 *   mode 1       VerifyDeterministicProposal (src/speculative_sampling.h:96-127): sample_u [batch, K+1]
 *                holds the categorical draws in the order rows with at least two entries consume them;
 *                accept_u unused.
 *   mode 2       greedy targets: entry 0 of every target row is its greedy token; no draws.
 *   accepted_len, final_token, engine_draws  device [batch] outputs; engine_draws = 32-bit engine outputs
 *                the reference would have consumed (a categorical draw over fewer than two entries takes
 *                none), so the caller can advance its std::mt19937 by that many.
 * A sequence with a row whose count exceeds its capacity or is below 1 reports accepted_len = final_token = -1.
 * 1 <= K <= 64. */
int mi355x_spec_verify_sparse(mi355x_search_ctx* ctx, void* stream, const int32_t* target_count,
                              const int32_t* target_ids, const float* target_probs, int target_capacity,
                              const int32_t* draft_count, const int32_t* draft_ids,
                              const float* draft_probs, int draft_capacity, const int32_t* proposal,
                              const float* accept_u, const double* sample_u, int batch, int K, int mode,
                              int32_t* accepted_len, int32_t* final_token, int32_t* engine_draws);

/* The draws of a batch in the order ONE engine serves them: GreedySearch_Cpu::SampleTopK/TopP/TopKTopP walk the
 * rows in order and call SampleCategoricalToken with the search's single std::mt19937 (src/search.cpp:207-243,
 * src/sampling_distribution.h:218-227); std::discrete_distribution consumes one canonical double per row -- none
 * for a row whose kept set holds one token, and finished rows are not sampled at all.  The caller computes the
 * next `rows` canonical doubles of (a copy of) its engine into uniform_pool; row r draws with
 * uniform_pool[number of consuming rows before r] from the kept set mi355x_sample left on the device
 * (kept_count [rows], kept_ids / kept_probs [rows, kept_capacity], kept_capacity >= every count), and
 * *draws_used (device int32, may be null) tells the caller how many doubles to discard from the real engine
 * (two mt19937 outputs each); it is -1 when some kept_count exceeds kept_capacity (a row would then draw from a
 * truncated set: the tokens of such a call must not be used).  skip_rows: device [rows] int32, non-zero = finished row (consumes nothing; its
 * token is its best id), or null.  out_tokens device [rows]. */
int mi355x_draw_in_order(mi355x_search_ctx* ctx, void* stream, const int32_t* kept_count,
                         const int32_t* kept_ids, const float* kept_probs, int kept_capacity, int rows,
                         const int32_t* skip_rows, const double* uniform_pool, int32_t* out_tokens,
                         int32_t* draws_used);

/* Tail of a greedy / sampling step on the device: Launch_CheckForEOSAndPad followed by
 * Launch_AppendNextTokensToSequences (src/cuda/search_cuda.cu:33-48,80-117), i.e. PadIfAlreadyEOS,
 * SetNextToken and AppendNextTokensToSequences of the CPU search (src/search.cpp:194-201,256-296):
 * a row that has already produced EOS gets pad_token_id; a row whose token is an EOS id is marked; the
 * (possibly padded) tokens are written to column current_length of the sequences; *done becomes 1 once
 * every row is marked (it is never cleared here).  As in the CUDA search the append is unconditional
 * while current_length < max_length: the caller advances its length only if the step did not finish.
 *   next_tokens  device [batch] in/out      eos_seen  device [batch] int32 flags in/out
 *   eos_ids      HOST [n_eos], n_eos <= MI355X_MAX_EOS
 *   sequences    device [batch, max_length]  done  device int32 */
int mi355x_greedy_tail(mi355x_search_ctx* ctx, void* stream, int32_t* next_tokens, int32_t* eos_seen,
                       int batch, const int32_t* eos_ids, int n_eos, int32_t pad_token_id,
                       int32_t* sequences, int max_length, int current_length, int32_t* done);

/* Element-wise type conversion on the device: DeviceInterface::Cast (src/smartptrs.h:208-210; CPU
 * src/cpu/interface.cpp:74-106).  Supported pairs, with the CPU path's arithmetic: F16->F32
 * (FastFloat16ToFloat32), BF16->F32 (BFloat16ToFloat32), F32->F16 (FastFloat32ToFloat16), F32->BF16
 * (upper 16 bits), I32->I64.  MI355X_E_INVALID when the two types are equal (the reference throws),
 * MI355X_E_UNSUPPORTED for any other pair (the reference's optional-capability "false"). */
int mi355x_cast(mi355x_search_ctx* ctx, void* stream, const void* in, int in_dtype, void* out,
                int out_dtype, size_t count);

/* Logits hand-off before the path: Logits::Get (src/models/logits.cpp:33-82) copies the logits of each
 * row's last real token out of the model's [rows, seq_len, vocab] output and widens fp16/bf16 to fp32;
 * here both happen in one pass.  raw: device, dtype MI355X_F32 / MI355X_F16 / MI355X_BF16;
 * token_index: HOST [rows] positions inside seq_len (copied by the call, through pinned staging memory of the
 * context), or NULL for seq_len - 1;
 * out: device [rows] rows of vocab floats, row r at out + r*out_stride. */
int mi355x_logits_handoff(mi355x_search_ctx* ctx, void* stream, const void* raw, int dtype, int rows,
                          int seq_len, int vocab, const int32_t* token_index, float* out,
                          int64_t out_stride);

/* Diagnostics: number of rows, since the context was created, that the single-pass fast paths
 * declined and the exact general path finished (synchronises `stream`). */
int mi355x_search_fallback_rows(mi355x_search_ctx* ctx, void* stream, unsigned* rows);

/* Failure handling of the top-k path (no counterpart in the reference).  The workgroup that finishes
 * a row waits for the candidate lists of the row's other workgroups by polling, at most `polls`
 * times (default 2^21, a few seconds); a wait that gives up hands its row to the exact path and
 * makes every later call on the context use the exact path for top-k rows, so that results stay
 * correct and no kernel ever waits without bound.  mi355x_search_wait_gave_up reports whether that
 * has happened (synchronises `stream`).  mi355x_search_set_poll_limit exists for tests of this
 * recovery: 0 lets every wait that is not satisfied at once give up. */
int mi355x_search_wait_gave_up(mi355x_search_ctx* ctx, void* stream, int* gave_up);
int mi355x_search_set_poll_limit(mi355x_search_ctx* ctx, int polls);
/* The exact sums of long rows (mi355x_softmax, mi355x_beam_select from 16384 logits per row on) have a bounded
 * wait of their own: a 4096-logit segment's workgroup polls, under the same limit, for the sums of the row's
 * earlier segments, which workgroups of the same launch publish.  A wait that gives up costs time only: the
 * segment is then added element by element, and the result is the same.  *segments = how many segments that has
 * happened to on this context (synchronises `stream`; no counterpart in the reference). */
int mi355x_search_sum_waits_gave_up(mi355x_search_ctx* ctx, void* stream, unsigned* segments);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_SEARCH_H_ */
