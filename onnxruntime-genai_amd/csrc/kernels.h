// Argument blocks and launch entry points shared between the host API (api.cpp) and the kernels.
#pragma once
#include <hip/hip_runtime.h>
#include "device_utils.h"

namespace ms {

// Shape of the fused sampling kernel: 512 threads x 16 float4 = one 32K-logit chunk per workgroup.
// Many logits per lane keep the per-wave selection overhead small against the streaming work, few
// chunks per row keep the finishing merge shallow (a 128K vocabulary is four sorted lists, two merge
// levels), and thread t's float4s (t, t+512, t+1024, ...) make every wave an even sample of the chunk.
constexpr int kSChunk = 32768;        // logits per workgroup of the streaming kernels
constexpr int kTopkBlock = 512;       // threads of a workgroup that streams a top-k row (16 128-bit loads each) ...
constexpr int kNucleusBlock = 1024;   // ... and a nucleus row (8 each: lighter threads, twice the waves in flight)
constexpr int kSMaxWaves = 16;
// Polls (about a microsecond each) after which a finishing workgroup stops waiting for another
// workgroup's list and lets the exact path compute the row: a few seconds by default.
constexpr int kDefaultPollLimit = 1 << 21;
constexpr int kSmallCap = 64;        // sorted candidates a chunk publishes on the k<=64 path
constexpr int kListCap = 128;        // candidates a chunk can hold before its sort
constexpr int kAllCap = 1024;        // slots a finishing workgroup ranks (16 chunks x kSmallCap)
constexpr int kNucleusCap = 16384;   // sorted nucleus candidates held in LDS by the finish kernel
constexpr int kFinishBlock = 1024;

constexpr int kEmitArgmax = 2;
constexpr int kArgmaxFusedMinBlocks = 1;  // rows x 32768-id chunks from which mi355x_argmax uses the fused kernel
constexpr int kModeTopkSmall = 0;
constexpr int kModeNucleus = 1;
constexpr int kModeGeneral = 2;
constexpr int kModeTopkLarge = 3;  // 64 < k <= kLargeKMax: streamed and finished by the nucleus kernels
// The per-chunk bound of such rows is the k-th best of what the 1024 threads of a nucleus workgroup offer: their
// maxima up to k = 512 (tight up to half the threads: about 1.4 k elements reach it), their four best elements
// each beyond that (about 1.1 k elements reach the k-th best of those 4096).
constexpr int kLargeKMax = 8192;
constexpr int kLargeKOneOffer = 512;  // up to here one offer per thread is enough

// Heterogeneous (k, p, T) of a batch of at most kInlineParamRows rows travel inside the kernel
// arguments, as a second argument of kernel variants of their own, so that no copy to the device
// precedes the launch and the kernels of the uniform case keep their small argument block.
constexpr int kInlineParamRows = 64;
struct InlineParams {
  mi355x_sample_params row[kInlineParamRows];
  const void* row_ptr[kInlineParamRows];  // where each row starts, for rows scattered over memory; null: row_stride apart
};

struct SideStreams {
  hipStream_t side[2];
  hipEvent_t fork, join[2];
};

struct SampleArgs {
  const void* logits;   // rows of fp32, fp16 or bf16 values (dtype), row_stride elements apart
  int64_t row_stride;
  int rows, vocab, chunks;
  int dtype;            // MI355X_F32 / MI355X_F16 / MI355X_BF16 (0 counts as fp32)
  Xform xf;
  mi355x_sample_params uniform;
  const mi355x_sample_params* per_row;  // device, or null
  const double* uniforms;
  int32_t* out_tokens;
  int32_t* kept_count;
  int32_t* kept_ids;
  float* kept_probs;
  int kept_capacity;
  // workspace
  u64* cand_small;        // [rows][chunks][kSmallCap]; zero between launches (published, then cleared by the finisher)
  uint32_t* chunk_cnt;    // [rows][chunks]
  uint32_t* chunk_max;    // [rows][chunks]
  uint32_t* chunk_thr;    // [rows][chunks]: order key of the score below which a nucleus chunk listed nothing
  u64* chunk_next;        // [rows][chunks]
  u64* big;               // [rows][big_stride]
  u64* big2;              // [rows][big_stride] second buffer of the exact path's radix sort, or null
  size_t big_stride;
  uint32_t* fallback_rows;  // [0] cumulative count (modulo 2^32) of rows finished by the general path; [1] non-zero once a wait gave up
  int poll_limit;           // polls a finishing workgroup waits for another workgroup's list
  int emit_topk;            // 1: write the k best (id, raw score) per row instead of sampling; 2 (kEmitArgmax): the
                            // best id only, k = 1, with ArgMax's rule that a NaN at id 0 wins (src/search.h:9-29)
  float* out_scores;        // [rows, k], emit_topk == 1 only (out_tokens is [rows, k] then)
  uint32_t* row_done;       // [rows] or null: nucleus rows under a grammar mask that the sparse-mask kernel finished
  int sparse_only;          // the sparse-mask kernel is the only one launched for nucleus rows: a row it cannot
                            // finish goes to the exact path inside it
  int exact_kernel;         // rows whose parameters alone send them to the exact path have a kernel of their own
};

struct ArgmaxArgs {
  const void* logits;
  int64_t row_stride;
  int rows, vocab, chunks;
  Xform xf;
  int32_t* out_tokens;
  u64* row_best;         // [rows], zero between launches
  uint32_t* row_arrive;  // [rows], zero between launches
};

constexpr int kBeamMaxCand = 32;  // 2 * beams, beams <= 16

// Multi-workgroup exact sequential sum (seqsum_kernels.hip).
constexpr int kSegElems = 4096;   // elements per segment
constexpr int kSegSubs = 64;      // parts of a segment with composed steps of their own (64 elements each)
constexpr int kMaxSegs = 1024;    // segments per row the walk kernel can hold
constexpr int kSeqSumMinVocab = 16384;  // shorter rows are summed by one workgroup in one launch

struct SeqSumArgs {
  const void* x;
  int64_t row_stride;
  int rows, vocab, segs;
  float inv_temp;
  uint32_t* seg_max;  // [rows][segs] order keys
  double* seg_sum;    // [rows][segs]
  int4* seg_step;     // [rows][segs]: d0, d1, binade, unused; binade -2: powers of two may fall inside the segment and
                      // its parts have records of their own
  int4* sub_step;     // [rows][segs][kSegSubs]: (d0, d1) of a 64-element part under the binade in sub_se, then under the next
  int* sub_se;        // [rows][segs][kSegSubs]: that binade; -1: the walk adds the part element by element
  float* e;           // [rows][e_stride] exponentials
  size_t e_stride;
  float* out_max;     // [rows]
  float* out_sum;     // [rows]
  int poll_limit;     // polls a segment's workgroup spends on an earlier segment's sum before it gives up
  uint32_t* gave_up;  // counts the segments whose wait gave up
};

struct SpecSparseArgs {
  const int32_t* t_count;  // [batch, K+1]
  const int32_t* t_ids;    // [batch, K+1, t_cap]
  const float* t_probs;
  int t_cap;
  const int32_t* d_count;  // [batch, K]
  const int32_t* d_ids;    // [batch, K, d_cap]
  const float* d_probs;
  int d_cap;
  const int32_t* proposal;  // [batch, K]
  const float* accept_u;    // [batch, K]
  const double* sample_u;   // [batch, K+1]
  int K;
  int mode;
  float* residual;  // workspace [batch, residual_stride]
  size_t residual_stride;
  int32_t* accepted_len;
  int32_t* final_token;
  int32_t* engine_draws;
};

struct BeamArgs {
  const void* logits;
  int64_t row_stride;
  int batch, beams, vocab;
  const float* beam_scores;   // [batch*beams]
  const float* row_max;       // [batch*beams] maximum and exact sum of exp(x - max) per row, or null:
  const float* row_sum;       //   the row kernel then computes them itself
  float* row_scores;          // workspace [batch*beams][kBeamMaxCand]
  int32_t* row_tokens;        // workspace [batch*beams][kBeamMaxCand]
  float* out_scores;          // [batch][2*beams]
  int32_t* out_tokens;
  int32_t* out_beams;
  // segmented path (long rows): every kSegElems-element segment of a row lists its 2*beams largest logits
  u64* seg_cand;              // workspace [batch*beams][segs][2*beams] keys (raw logit, token), best first
  uint32_t* seg_max;          // [batch*beams][segs] order keys of the segment maxima (read by the exact sum)
  int segs;
};
constexpr int kBeamFinCap = 4096;  // beams * segs * 2*beams keys one finishing workgroup holds

// Device-resident BeamSearchScorer state (all pointers device memory).
struct ScorerState {
  int batch, beams, max_length, pad, early_stopping, n_eos;
  int eos[MI355X_MAX_EOS];
  float* next_scores;     // [batch*beams]
  int32_t* next_tokens;
  int32_t* next_indices;
  float* hyp_score;       // [batch][beams], best first
  int* hyp_len;           // [batch][beams]
  int* hyp_slot;          // [batch][beams+1]: rank -> token row
  int32_t* hyp_tokens;    // [batch][beams+1][max_length]
  int* hyp_used;          // [batch]
  int* done;              // [batch]
  int* not_done;          // [1]
  const float* pow_table; // [max_length+1]: powf(length, length_penalty), computed by the host libm
  int* pending;           // [batch]: entries whose "can a later candidate still improve" test waits for all entries' candidates
  unsigned* arrive;       // [1]: workgroups of a fused selection + scorer launch that are through; 0 between launches
};

// What one scorer step works on besides its state: the sequences as they are, the buffer the extended ones go to.
struct ScorerStep {
  ScorerState s;
  const int32_t* sequences;
  int32_t* sequences_next;
  int sequence_length;
};

}  // namespace ms

extern "C" {
hipError_t ms_sample_init();
// `table`, when not null, holds the parameters of rows 0 .. a->rows-1 (a->rows <= kInlineParamRows).
// any_nucleus / any_large_k / any_other: some row may be in nucleus mode / a top-k row with
// 64 < k <= kLargeKMax / in another mode (each mode has kernels of its own); a->exact_kernel: some row's
// parameters send it to the exact path.
// sides, when not null: streams and events of the context on which the kernels of a call whose rows are in several
// modes run side by side (each mode's kernels skip the other modes' rows and share no state with them): they fork
// from `stream` behind an event, and `stream` waits for them before the exact rows' kernel and before the call returns.
hipError_t ms_launch_sample(const ms::SampleArgs* a, const ms::InlineParams* table, bool any_other, bool any_nucleus,
                            bool any_large_k, hipStream_t stream, const ms::SideStreams* sides);
hipError_t ms_launch_argmax(const ms::ArgmaxArgs* a, int dtype, hipStream_t stream);
hipError_t ms_launch_process_logits(float* logits, int64_t row_stride, int rows, int vocab,
                                    const ms::Xform* xf, hipStream_t stream);
hipError_t ms_launch_softmax(float* scores, int64_t row_stride, int rows, int vocab, float temperature,
                             int log_softmax, hipStream_t stream);
// Writes, for every row, the bitmap of ids the no-repeat-n-gram rule bans (mask layout) into `ban`.
hipError_t ms_launch_ngram_ban(const ms::Xform* xf, int rows, int vocab, int ngram, uint32_t* ban, hipStream_t stream);
hipError_t ms_launch_draw_in_order(const int32_t* kept_count, const int32_t* kept_ids, const float* kept_probs, int cap, int rows,
                                    const int32_t* skip, const double* pool, int32_t* out_tokens, int32_t* draws_used,
                                    hipStream_t stream);
hipError_t ms_launch_kv_gather(const void* const* present_dev, void* const* past_dev, int n_tensors,
                               const int32_t* beam_indices, int rows, size_t block_bytes, int width,
                               hipStream_t stream);
hipError_t ms_launch_spec_verify(const float* p_target, const float* p_draft, const int32_t* draft_tokens,
                                 const float* accept_u, const double* sample_u, int batch, int K, int vocab,
                                 int32_t* accepted_len, int32_t* final_token, hipStream_t stream);
hipError_t ms_launch_greedy_tail(int32_t* next_tokens, int32_t* eos_seen, int batch, const int32_t* eos_ids, int n_eos,
                                 int32_t pad, int32_t* sequences, int max_length, int current_length, int32_t* done,
                                 hipStream_t stream);
hipError_t ms_launch_spec_verify_sparse(const ms::SpecSparseArgs* a, int batch, hipStream_t stream);
hipError_t ms_launch_cast(const void* in, void* out, size_t count, int kind, hipStream_t stream);
hipError_t ms_launch_logits_handoff(const void* raw, int kind, int rows, int seq_len, int vocab,
                                    const int32_t* token_index, float* out, int64_t out_stride, hipStream_t stream);
hipError_t ms_launch_beam_select(const ms::BeamArgs* a, int dtype, hipStream_t stream);
hipError_t ms_launch_beam_exp_step(const ms::SeqSumArgs* q, const ms::BeamArgs* a, int dtype, hipStream_t stream);
// step != null: every batch entry's workgroup goes on with the entry's scorer step (ms_launch_scorer_step's work).
hipError_t ms_launch_beam_finish(const ms::BeamArgs* a, int dtype, const ms::ScorerStep* step, hipStream_t stream);
hipError_t ms_launch_seqsum(const ms::SeqSumArgs* a, int dtype, hipStream_t stream);  // its three launches
hipError_t ms_launch_seqsum_max(const ms::SeqSumArgs* a, int dtype, hipStream_t stream);
hipError_t ms_launch_seqsum_walk(const ms::SeqSumArgs* a, hipStream_t stream);
hipError_t ms_launch_softmax_apply(float* scores, int64_t row_stride, const ms::SeqSumArgs* a, int log_softmax,
                                   hipStream_t stream);
hipError_t ms_launch_scorer_step(const ms::ScorerState* s, const int32_t* sequences, int32_t* sequences_next,
                                 int sequence_length, const float* cs, const int32_t* ct, const int32_t* ci,
                                 hipStream_t stream);
hipError_t ms_launch_scorer_finalize(const ms::ScorerState* s, const int32_t* sequences, int sequence_length,
                                     hipStream_t stream);
}
