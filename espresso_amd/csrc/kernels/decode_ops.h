// Argument blocks and launchers of the per-token kernels (kernels/decode_ops.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace esp {

constexpr int kMaxStepRows = 32;   // rows of one step: 16 sequences x (current, proposed) in a batched verify pass

// The rows (tokens) of one step, passed by value so that no host-to-device copy is needed.
struct StepRows {
    int count;
    int token[kMaxStepRows];
    int pos[kMaxStepRows];
    int seq[kMaxStepRows];
};

struct QkvPostArgs {
    const float *qkv;      // [rows][attnDim + 2 kvDim] in the fused matrix's row order
    const float *q_norm;   // [head_dim] or null
    const float *k_norm;   // [head_dim] or null
    float norm_eps;
    int n_head, n_kv_head, head_dim, max_seq;
    const float *rope_cos;  // [max_seq][head_dim/2]
    const float *rope_sin;
    const int *pos;         // [rows]
    const int *seq;         // [rows]
    float *q_out;           // [rows][attnDim]
    void *k_cache;          // this layer: [seq][max_seq][kvDim]
    void *v_cache;          // this layer: [seq][max_seq][kvDim]
    size_t cache_seq_stride;  // elements per sequence (kvDim * max_seq)
    // `qkv` may still be the split-K partial sums of its GEMM: `splits` planes, `plane` floats apart, added in split order
    // on load (0 or 1: qkv is complete)
    int splits;
    size_t plane;
};

struct AttentionArgs {
    const float *q;         // [rows][attnDim]
    const void *k_cache;
    const void *v_cache;
    size_t cache_seq_stride;
    int n_head, n_kv_head, head_dim, max_seq;
    const int *pos;
    const int *seq;
    uint16_t *ctx_f16;      // [rows][attnDim]
    // partial results of the split-prefix kernel: [rows][kvHeads][splits][group][head_dim + 2] floats
    float *split_scratch;
    // partial results of attention_partial_kernel: [rows][heads][attention_head_splits][head_dim + 4] floats
    float *head_partials;
    // launch_attention_prompt only, all three or none: the context as split rows (hi = fp16(v), lo = fp16((v - hi) * 2048),
    // sub-block sums; SplitRowsView) instead of ctx_f16, with the queries and the softmax weights split the same way
    uint16_t *ctx_hi, *ctx_lo, *ctx_sums;
};
constexpr int kAttentionMaxSplits = 32;
// Slices of the prefix the grouped-query attention kernel works on in parallel (fixed per runtime).
int attention_split_count(int max_seq, int head_dim);

hipError_t launch_embed(const void *table, bool table_is_f16, const int *tokens, int rows, int d, float *hidden, hipStream_t s);
hipError_t launch_rmsnorm(const float *x, const float *w, float eps, int rows, int d, uint16_t *out_f16,
                          unsigned long long *argmax_cells, hipStream_t s);
// RMSNorm of rows that are still split-K partial sums [splits][rows][d] (`plane` = rows * d floats apart): adds them in
// split order (+ residual), writes the sums to y and the normalised fp16 rows to out_f16.  d % 4 == 0, d <= 8192.
bool rmsnorm_reduce_supported(int d);
hipError_t launch_rmsnorm_reduce(const float *partial, int splits, size_t plane, const float *residual, float *y, const float *w, float eps,
                                 int rows, int d, uint16_t *out_f16, hipStream_t s);
hipError_t launch_qkv_post(const QkvPostArgs &a, int rows, bool kv_f16, hipStream_t s);
hipError_t launch_attention(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s);
// Causal attention of `rows` rows that are ONE sequence at consecutive positions (a prompt block), on the matrix cores.
// Head dim 64 or 128, 1, 2 or 4 query heads per KV head (attention_prompt_supported); Q, K, V, P as fp16, fp32 sums.
bool attention_prompt_supported(int n_head, int n_kv_head, int head_dim);
hipError_t launch_attention_prompt(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s);
// Attention that stops at per-split partial states (head_dim 64 or 128, up to kMaxStepRows rows); the GEMV that reads
// the context merges them (GemvParams::merge_partials).  attention_head_splits: slices per query head.
int attention_head_splits(int max_seq);
hipError_t launch_attention_partials(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s);
hipError_t launch_swiglu(const float *gu, int rows, int hidden, uint16_t *act_f16, hipStream_t s);
// Scratch of the two-launch argmax: kMaxStepRows x 128 partial (value, index) pairs.
struct ArgmaxScratch {
    float *part_value = nullptr;
    int *part_index = nullptr;
};
constexpr int kArgmaxScratchSlots = kMaxStepRows * 128;
hipError_t launch_argmax(const float *logits, int rows, int vocab, int *out_token, float *out_value, const ArgmaxScratch &scratch,
                         hipStream_t s);
hipError_t launch_set_rows(const StepRows &rows, int *tokens, int *pos, int *seq, hipStream_t s);
hipError_t launch_greedy_feed(const int *next_token, int seq, int *visible, int *tokens, int *pos, int *seqs, int *log,
                              int *log_count, int log_capacity, hipStream_t s);
// A greedy step's end in two launches instead of four: the argmax slices of the row of logits, then one workgroup
// that reduces them, feeds the token as launch_greedy_feed does and writes its embedding row to hidden[0..d).
hipError_t launch_greedy_step_tail(const float *logits, int vocab, int *out_token, const ArgmaxScratch &scratch, int seq, int *visible,
                                   int *tokens, int *pos, int *seqs, int *log, int *log_count, int log_capacity, const void *table,
                                   bool table_is_f16, int d, float *hidden, int eos, hipStream_t s);
// The same two steps for a head GEMV that left one (value, index) pair per workgroup instead of logits (EPI_ARGMAX):
// `blocks` pairs per row in scratch, rows `blocks` apart.
hipError_t launch_argmax_final(const ArgmaxScratch &scratch, int blocks, int rows, int *out_token, hipStream_t s);
hipError_t launch_greedy_tail(const ArgmaxScratch &scratch, int blocks, int *out_token, int seq, int *visible, int *tokens, int *pos, int *seqs,
                              int *log, int *log_count, int log_capacity, const void *table, bool table_is_f16, int d, float *hidden,
                              int eos, hipStream_t s);
// log_count points at three ints: tokens logged so far, stopped (set by the kernel when it emits the stop token `eos` while the third
// int, set by the host, is non-zero), stop enabled.  A stopped sequence's replays emit nothing and recompute the row they computed last.
hipError_t launch_set_ints(int *dst0, int v0, int *dst1, int v1, hipStream_t s);

// Device-resident state of the exact two-token loop over one sequence (generateIncrementalExactTwoTokenDraftLlama,
// RealModelInferenceEngine.swift:6014-6190): what the host loop keeps in local variables, so that whole passes (draft step,
// two-row verify step, acceptance) replay as one captured graph without a host decision in between.
struct TwoTokenState {
    int current;        // the last emitted token; neither model has consumed it yet
    int full_pos;       // the target's visible token count
    int accepted_prev;  // the pass before accepted its proposal: the draft still owes the row (proposed_prev, full_pos - 1)
    int proposed_prev, exact1_prev;
    int proposed;       // this pass's proposal (set between the draft step and the verify step)
    int emitted, budget, all, max_seq, eos, reference_accounting;
    int done;           // no further pass may run on the device (end of the loop, or a pass that needs a host decision)
    int stopped;        // the loop itself is over (stop token, budget, context)
    int passes, committed_total, accepted_total, reference_accepted_total;
};
// After the draft's two rows went through its head: the proposal becomes row 1 of the target's verify step; the draft's
// successor of the row it owed is compared for the reference's accepted count.
// `embed`: the kernel also fetches the embedding rows of the two tokens (whether it changed them or not) into the model's hidden
// rows, so that the trunk pass after it starts without an embedding launch.
struct EmbedTarget {
    const void *table = nullptr;   // [vocab][d] fp16 or fp32
    int table_is_f16 = 0, d = 0;
    float *hidden = nullptr;       // [2][d]
    float *keep_row1 = nullptr;    // when set: row 1 of `hidden` (the model's last output) is copied here before the rows are overwritten
};
hipError_t launch_two_token_verify_rows(TwoTokenState *state, const int *draft_head_tokens, int *target_tokens, int *target_pos, const EmbedTarget &embed,
                                        hipStream_t s);
// After the target's two rows went through its head: emits one or two tokens into log, keeps the matching hidden row of the
// target (d floats from hidden_rows into last_hidden), advances the state and writes the draft's two rows of the next pass.
// The same loop over up to sixteen sequences in lock step (rows 2 s and 2 s + 1 of both models belong to sequence s), and the plain
// greedy loop over several sequences: per-sequence variables in device memory, every pass one captured graph.
constexpr int kMaxLoopSequences = kMaxStepRows / 2;
struct TwoTokenBatchState {
    int n_seq, budget, passes;
    int current[kMaxLoopSequences], full_pos[kMaxLoopSequences], accepted_prev[kMaxLoopSequences], proposed_prev[kMaxLoopSequences];
    int proposed[kMaxLoopSequences], can_two[kMaxLoopSequences], live[kMaxLoopSequences], emitted[kMaxLoopSequences];
    int committed[kMaxLoopSequences], accepted[kMaxLoopSequences];
};
hipError_t launch_two_token_batch_verify_rows(TwoTokenBatchState *state, const int *draft_head_tokens, int *target_tokens, int *target_pos, hipStream_t s);
// log: [n_seq][budget] tokens; last_hidden: [sequence][d]
hipError_t launch_two_token_batch_accept(TwoTokenBatchState *state, int n_seq, const int *target_head_tokens, int *log, const float *hidden_rows,
                                         float *last_hidden, int d, int *draft_tokens, int *draft_pos, hipStream_t s);
// Greedy step of n sequences: the head's tokens become the next rows at the next positions and go to log[step][n].
hipError_t launch_batch_greedy_feed(const int *head_tokens, int n, int *tokens, int *pos, int *log, int *step, int capacity_steps, hipStream_t s);
hipError_t launch_two_token_accept(TwoTokenState *state, const int *target_head_tokens, int *log, int log_capacity, const float *hidden_rows,
                                   float *last_hidden, int d, int *draft_tokens, int *draft_pos, const EmbedTarget &draft_embed, hipStream_t s);
hipError_t launch_copy_rows(const float *src, float *dst, int rows, int d, hipStream_t s);

}  // namespace esp
