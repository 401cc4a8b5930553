// Device-resident llama decoder state: the MI355X counterpart of the reference's
// CPUExactLlamaRuntime (Sources/RealModelInference/RealModelInferenceEngine.swift:548-850).
#pragma once

#include <string>
#include <vector>

#include "context.h"
#include "kernels/decode_ops.h"

namespace esp {

// weight slots; names follow LayerWeightPaths (Sources/ModelSupport/LayerWeightPaths.swift:22-84)
enum WeightSlot : int {
    SLOT_TOKEN_EMBEDDING = 0, SLOT_FINAL_NORM = 1, SLOT_LM_HEAD = 2,
    SLOT_RMS_ATT = 10, SLOT_WQ = 11, SLOT_WK = 12, SLOT_WV = 13, SLOT_WO = 14,
    SLOT_RMS_FFN = 15, SLOT_W1 = 16, SLOT_W2 = 17, SLOT_W3 = 18, SLOT_Q_NORM = 19, SLOT_K_NORM = 20,
};

struct LlamaConfig {
    int n_layer = 0, n_head = 0, n_kv_head = 0, d_model = 0, head_dim = 0, hidden_dim = 0, vocab = 0, max_seq = 0;
    float norm_eps = 1e-5f, rope_theta = 10000.0f;
    int eos_token = -1;
    int kv_format = FMT_F32;  // FMT_F32 or FMT_F16
    int max_sequences = 1;    // independent KV caches
    int attention_dim() const { return n_head * head_dim; }
    int kv_dim() const { return n_kv_head * head_dim; }
};

constexpr int kPrefillBlockRows = 512;        // rows per MFMA prefill block
constexpr int kStepsPerGraph = 8;             // greedy steps in the longer of the two captured step graphs
constexpr int kMatrixPrefillMinTokens = 32;   // shorter prompts take the exact per-token path
constexpr size_t kGemmWorkspaceFloats = (size_t)8 << 20;

// What a device-resident generation loop over two runtimes (target + draft) keeps between calls, owned by the target: its state
// and token log in device memory and the captured graphs of its passes.  The graphs hold pointers into both runtimes, so the
// session names the partner by an identifier no later runtime can have, and both runtimes' graph epochs (which change whenever a
// runtime's kernels for a step change): a session that does not match is rebuilt, never replayed.
struct DeviceLoopSession {
    unsigned long long partner_id = 0, epoch = 0, partner_epoch = 0;
    void *state = nullptr;
    int *log = nullptr;
    int log_capacity = 0;
    hipGraphExec_t one = nullptr, many = nullptr;   // one pass; several passes in a row
};

class LlamaRuntime {
  public:
    static int create(const LlamaConfig &config, LlamaRuntime **out);
    ~LlamaRuntime();

    const LlamaConfig &config() const { return c_; }
    bool finalized() const { return finalized_; }

    // Copies the bytes.  Matrices: GGUF block layout, row-major [rows, cols]; norms: f32 or f16 vectors;
    // embedding: f32 or f16 table.
    int set_weight(int layer, int slot, int format, const void *data, size_t bytes);
    // Fuses wq|wk|wv and w1|w3, uploads everything, builds the RoPE table.
    int finalize();

    int reset();                                  // all sequences (:616-635)
    int visible(int seq) const;
    int set_visible(int seq, int count);          // rollback = lower the visible length
    // Runs the trunk over `rows` (token, position, sequence); positions are written into the KV caches.
    // Does not change the visible counts.
    int forward_rows(const StepRows &rows);
    // forward one token at the sequence's visible position and keep its hidden state (:672-680)
    int advance(int seq, uint32_t token);
    int prefill(int seq, const uint32_t *tokens, int count);   // (:637-645)
    // Final norm + LM head + first-max argmax of kept hidden states (:663-670, :825-849).
    int select_greedy(int seq, uint32_t *token);
    // Head over rows of the most recent forward_rows(); tokens[i] for row i.
    int head_rows(int count, uint32_t *tokens);
    // Keep row `row` of the most recent forward_rows() as sequence `seq`'s last hidden state.
    int keep_row(int row, int seq);
    // `steps` greedy tokens from the sequence's current state (select, then advance, per token) as
    // replays of captured HIP graphs (eight steps per graph while that many are left, then one); the host synchronises once at the end.
    int continue_greedy(int seq, int steps, uint32_t *out_tokens);
    // The same, ending early at the configuration's stop token: the stop token is emitted (it is the last of *produced tokens) and not
    // consumed.  The step graph notices it on the device; the host looks once per 32 replays.
    int continue_greedy_until_stop(int seq, int steps, uint32_t *out_tokens, int *produced);
    void set_use_graph(bool enabled) { use_graph_ = enabled; }
    // Prompts of kMatrixPrefillMinTokens or more run in blocks through the MFMA kernels (default on).
    void set_matrix_prefill(bool enabled) { matrix_prefill_ = enabled; }
    // Decode steps of one or two rows: attention as one launch that leaves partial states, merged by the wo GEMV
    // (on by default where the shapes allow); off = the split kernel plus the merge kernel.
    void set_merged_attention(bool enabled);
    // Decode steps of one or two rows feed every layer GEMV that has the form (matrix-core Q4_K) hi / lo fp16 pairs of the fp32
    // activations instead of their fp16 roundings (default on; ESPRESSO_HIP_SPLIT_ACTIVATIONS=0 at creation switches it off).
    void set_split_activations(bool enabled);
    bool split_activations() const { return split_activations_; }
    bool merged_attention_in_use() const { return !layers_.empty() && wo_merges_attention(layers_[0], 1); }
    int read_last_hidden(int seq, float *out);
    int read_logits(int seq, float *out);         // runs the head on the kept hidden state

    size_t weight_bytes_per_token() const { return weight_bytes_; }
    // what the weights hold in HBM: the packed matrices, the tiled copies the matrix-core GEMVs read beside them, the embedding table
    size_t resident_weight_bytes() const { return resident_weight_bytes_; }

    // Steps whose rows (token, position, sequence) already sit in the device arrays below: generation loops that keep
    // their decisions on the device enqueue these, also under stream capture.  Nothing here synchronises.
    int *device_row_tokens() { return d_tokens_; }
    int *device_row_positions() { return d_pos_; }
    int *device_row_sequences() { return d_seq_; }
    const int *device_head_tokens() const { return d_out_tokens_; }
    const float *device_hidden_rows() const { return hidden_; }
    float *device_last_hidden(int seq) { return last_hidden_ + (size_t)seq * c_.d_model; }
    int enqueue_device_rows(int rows, bool embedded = false) { return enqueue_trunk(rows, embedded); }   // embedding (unless the rows hold it already), then every layer
    EmbedTarget device_embed_target() { EmbedTarget e; e.table = embedding_; e.table_is_f16 = embedding_f16_ ? 1 : 0; e.d = c_.d_model; e.hidden = hidden_; return e; }
    int enqueue_device_head(int rows) { return run_head(hidden_, rows); }         // final norm, head, first-max arg-max per row
    bool graph_replay_enabled() const { return use_graph_ && !timing_enabled_; }
    unsigned long long id() const { return id_; }
    // changes whenever the kernels a captured graph would hold have changed (switches of this runtime, esp_set_tuning): holders
    // of captured passes compare it before they replay
    unsigned long long graph_epoch() { sync_tuning(); return graph_epoch_; }
    DeviceLoopSession &loop_session() { return loop_session_; }
    void release_loop_session();   // destroys the session's graphs and frees its buffers

    // Per-kernel timing with HIP events on the library stream.  While enabled, every launch of the
    // kernels below is bracketed by an event pair; collect_kernel_times() synchronises and adds the
    // elapsed times to the totals.
    enum KernelClass { K_QKV = 0, K_WO, K_GATE_UP, K_DOWN, K_HEAD, K_ATTENTION, K_EVENT_PAIR, K_CLASS_COUNT };
    void set_kernel_timing(bool enabled) { timing_enabled_ = enabled; }
    int collect_kernel_times(double total_us[K_CLASS_COUNT], long launches[K_CLASS_COUNT], bool reset);
    size_t kernel_bytes(int kernel_class) const;   // algorithmic bytes of one batch-1 launch
    // mean_us: launches back to back between two events; kernel_only_us (optional): the same launches with events
    // of their own per launch (the kernels' own durations, as a kernel trace reports them)
    int time_kernel_class(int kernel_class, int iters, double *mean_us, double *kernel_only_us = nullptr);

  private:
    LlamaRuntime() = default;
    struct HostTensor { int format = -1; std::vector<uint8_t> bytes; };
    struct HostLayer { HostTensor rms_att, wq, wk, wv, wo, rms_ffn, w1, w2, w3, q_norm, k_norm; };
    struct Layer {
        float *rms_att = nullptr, *rms_ffn = nullptr, *q_norm = nullptr, *k_norm = nullptr;
        DeviceMatrix wqkv, wo, w13, w2;
        void *k_cache = nullptr, *v_cache = nullptr;
    };
    int upload_vector(const HostTensor &t, size_t count, float **out, const char *what);
    // want_logits: the full-vocabulary logits are needed in logits_ (otherwise one or two rows take the head whose
    // epilogue is the arg-max and store none)
    int run_head(const float *hidden_rows, int count, bool want_logits = false);
    bool head_fuses_argmax() const { return fused_head_argmax_ && gemv_supports_argmax(lm_head_); }
    // embedded: hidden_ already holds the rows' embeddings; final_out: where the last layer writes (default hidden_)
    int enqueue_trunk(int rows, bool embedded = false, float *final_out = nullptr);
    int prefill_block(int seq, const uint32_t *tokens, int rows, int base);
    int enqueue_layers_matrix(int rows, bool one_sequence_consecutive = false);
    bool matrix_prefill_supported() const;
    bool wo_merges_attention(const Layer &L, int rows) const;
    int capture_step_graph(int seq);
    int capture_steps(int seq, int count, hipGraphExec_t *out);
    int replay_steps(int seq, int steps);
    HostTensor *host_slot(int layer, int slot);

    LlamaConfig c_;
    bool finalized_ = false;
    HostTensor h_embedding_, h_final_norm_, h_lm_head_;
    std::vector<HostLayer> h_layers_;

    void *embedding_ = nullptr;
    bool embedding_f16_ = true;
    float *final_norm_ = nullptr;
    DeviceMatrix lm_head_;
    std::vector<Layer> layers_;
    float *rope_cos_ = nullptr, *rope_sin_ = nullptr;
    // activations for up to kMaxStepRows rows
    float *hidden_ = nullptr, *qkv_ = nullptr, *q_ = nullptr, *gu_ = nullptr, *logits_ = nullptr, *last_hidden_ = nullptr;
    uint16_t *xn_ = nullptr, *ctx_ = nullptr, *act_ = nullptr;
    // prompt blocks with split activations: the lo planes and sub-block sums beside xn_, ctx_ and act_ (SplitRowsView)
    uint16_t *xn_lo_ = nullptr, *ctx_lo_ = nullptr, *act_lo_ = nullptr, *xn_sums_ = nullptr, *ctx_sums_ = nullptr, *act_sums_ = nullptr;
    bool split_blocks_supported() const;
    int enqueue_layers_split(int rows);
    int *d_tokens_ = nullptr, *d_pos_ = nullptr, *d_seq_ = nullptr, *d_out_tokens_ = nullptr;
    std::vector<int> visible_;
    size_t weight_bytes_ = 0, resident_weight_bytes_ = 0;
    // captured greedy step per sequence (head -> feed -> trunk -> keep), and its device-side state
    bool use_graph_ = true;
    std::vector<hipGraphExec_t> step_graphs_, multi_graphs_;   // one step, kStepsPerGraph steps
    unsigned long long id_ = 0, graph_epoch_ = 1;
    unsigned tuning_epoch_ = 0;   // the kernel-selection epoch (gemv_tuning_epoch) this runtime's captured graphs were made under
    void drop_captured_graphs();
    void sync_tuning();
    DeviceLoopSession loop_session_;
    int *d_visible_ = nullptr, *d_log_ = nullptr, *d_log_count_ = nullptr;
    ArgmaxScratch argmax_scratch_;
    int head_partial_capacity_ = 0;      // (value, index) slots per row for the head's per-workgroup candidates
    bool fused_head_argmax_ = true;      // ESPRESSO_HIP_FUSED_HEAD_ARGMAX=0: head GEMV stores logits, separate arg-max launches
    float *attn_scratch_ = nullptr;
    bool matrix_prefill_ = true;
    bool merged_attention_ = true;
    bool split_activations_ = true;
    bool prompt_attention_ = false;   // prompt blocks run attention on the matrix cores
    float *gemm_workspace_ = nullptr;
    GemmSplitSharedK gemm_shared_k_;   // the device's pool for launch_gemm_split's hand-over between workgroups (not owned)

    struct TimedLaunch { int kernel_class; hipEvent_t start, stop; };
    bool timing_enabled_ = false;
    std::vector<TimedLaunch> timed_;        // pending pairs
    std::vector<hipEvent_t> event_pool_;
    double time_total_us_[K_CLASS_COUNT] = {};
    long time_launches_[K_CLASS_COUNT] = {};
    hipEvent_t take_event();
    int time_begin(int kernel_class);
    int time_end();
};

}  // namespace esp

struct ESPLlamaRuntime {
    esp::LlamaRuntime *rt;
};
