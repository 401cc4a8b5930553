#include "llama_runtime.h"

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>

namespace esp {
namespace {

// fp16 bits -> float on the host (weights arrive as raw bytes)
float half_to_float_host(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, mant = h & 0x3FFu, f;
    if (exp == 0) {
        if (mant == 0) f = sign;
        else {
            int e = -1;
            do { mant <<= 1; e++; } while ((mant & 0x400u) == 0);
            f = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3FFu) << 13);
        }
    } else if (exp == 31) f = sign | 0x7F800000u | (mant << 13);
    else f = sign | ((exp + 112u) << 23) | (mant << 13);
    float out;
    std::memcpy(&out, &f, 4);
    return out;
}

template <typename T>
void free_device(T *&p) {
    if (p) (void)hipFree(p);
    p = nullptr;
}

}  // namespace

int LlamaRuntime::create(const LlamaConfig &c, LlamaRuntime **out) {
    *out = nullptr;
    // validateRuntimeConfig (RealModelInferenceEngine.swift:7615-7634)
    if (c.n_layer <= 0 || c.n_head <= 0 || c.n_kv_head <= 0 || c.d_model <= 0 || c.head_dim <= 0 ||
        c.hidden_dim <= 0 || c.vocab <= 0 || c.max_seq <= 0)
        return fail(ESP_ERR_INVALID_ARGUMENT, "llama config: every dimension must be positive");
    if (c.n_head % c.n_kv_head != 0)
        return fail(ESP_ERR_INVALID_ARGUMENT, "llama config: nHead %d is not a multiple of nKVHead %d", c.n_head, c.n_kv_head);
    if (c.head_dim % 2 != 0) return fail(ESP_ERR_INVALID_ARGUMENT, "llama config: headDim %d must be even", c.head_dim);
    if (c.kv_format != FMT_F32 && c.kv_format != FMT_F16)
        return fail(ESP_ERR_INVALID_ARGUMENT, "llama config: KV cache format must be f32 or f16");
    if (c.max_sequences < 1 || c.max_sequences > kMaxStepRows)
        return fail(ESP_ERR_INVALID_ARGUMENT, "llama config: max_sequences must be 1..%d", kMaxStepRows);
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    static std::atomic<unsigned long long> next_id{1};
    LlamaRuntime *rt = new LlamaRuntime();
    rt->id_ = next_id.fetch_add(1);
    rt->c_ = c;
    rt->h_layers_.resize(c.n_layer);
    rt->visible_.assign(c.max_sequences, 0);
    *out = rt;
    return ESP_OK;
}

LlamaRuntime::~LlamaRuntime() {
    free_device(embedding_);
    free_device(final_norm_);
    matrix_release(&lm_head_);
    for (Layer &L : layers_) {
        free_device(L.rms_att); free_device(L.rms_ffn); free_device(L.q_norm); free_device(L.k_norm);
        matrix_release(&L.wqkv); matrix_release(&L.wo); matrix_release(&L.w13); matrix_release(&L.w2);
        free_device(L.k_cache); free_device(L.v_cache);
    }
    free_device(rope_cos_); free_device(rope_sin_);
    free_device(hidden_); free_device(qkv_); free_device(q_); free_device(gu_); free_device(logits_);
    free_device(last_hidden_); free_device(xn_); free_device(ctx_); free_device(act_);
    free_device(xn_lo_); free_device(ctx_lo_); free_device(act_lo_); free_device(xn_sums_); free_device(ctx_sums_); free_device(act_sums_);
    free_device(d_tokens_); free_device(d_pos_); free_device(d_seq_); free_device(d_out_tokens_);
    free_device(d_visible_); free_device(d_log_); free_device(d_log_count_);
    free_device(attn_scratch_);
    free_device(gemm_workspace_);
    free_device(argmax_scratch_.part_value); free_device(argmax_scratch_.part_index);
    for (hipGraphExec_t g : step_graphs_) if (g) (void)hipGraphExecDestroy(g);
    for (hipGraphExec_t g : multi_graphs_) if (g) (void)hipGraphExecDestroy(g);
    release_loop_session();
    for (TimedLaunch &t : timed_) { (void)hipEventDestroy(t.start); (void)hipEventDestroy(t.stop); }
    for (hipEvent_t e : event_pool_) (void)hipEventDestroy(e);
}

hipEvent_t LlamaRuntime::take_event() {
    if (!event_pool_.empty()) {
        hipEvent_t e = event_pool_.back();
        event_pool_.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

int LlamaRuntime::time_begin(int kernel_class) {
    if (!timing_enabled_) return ESP_OK;
    TimedLaunch t{kernel_class, take_event(), take_event()};
    if (!t.start || !t.stop) return fail(ESP_ERR_OUT_OF_MEMORY, "hipEventCreate failed");
    ESP_HIP_TRY(hipEventRecord(t.start, context().stream));
    timed_.push_back(t);
    return ESP_OK;
}

int LlamaRuntime::time_end() {
    if (!timing_enabled_) return ESP_OK;
    ESP_HIP_TRY(hipEventRecord(timed_.back().stop, context().stream));
    return ESP_OK;
}

int LlamaRuntime::collect_kernel_times(double total_us[K_CLASS_COUNT], long launches[K_CLASS_COUNT], bool reset) {
    ESP_HIP_TRY(hipStreamSynchronize(context().stream));
    for (TimedLaunch &t : timed_) {
        float ms = 0.0f;
        ESP_HIP_TRY(hipEventElapsedTime(&ms, t.start, t.stop));
        time_total_us_[t.kernel_class] += (double)ms * 1e3;
        time_launches_[t.kernel_class] += 1;
        event_pool_.push_back(t.start);
        event_pool_.push_back(t.stop);
    }
    timed_.clear();
    for (int k = 0; k < K_CLASS_COUNT; k++) {
        if (total_us) total_us[k] = time_total_us_[k];
        if (launches) launches[k] = time_launches_[k];
        if (reset) { time_total_us_[k] = 0; time_launches_[k] = 0; }
    }
    return ESP_OK;
}

// Launches the GEMV of one class for every layer in turn (the head: the same matrix), `iters` rounds, between
// two events: back-to-back dependent launches at the real shapes over the real weights, which no cache can hold
// across a round.  The epilogues write into the step's buffers, so sequence state is garbage afterwards.
// The decode step (one or two rows) runs attention as a single launch that leaves per-head partial states, and
// the wo GEMV merges them while staging, when the head size and the matrix allow it.
bool LlamaRuntime::wo_merges_attention(const Layer &L, int rows) const {
    return merged_attention_ && c_.n_head % c_.n_kv_head == 0 && rows <= 2 &&
           L.wo.cols == c_.attention_dim() && gemv_merges_attention_partials(L.wo, rows, c_.head_dim);
}

int LlamaRuntime::time_kernel_class(int kernel_class, int iters, double *mean_us, double *kernel_only_us) {
    if (!finalized_ || iters < 1 || !mean_us) return fail(ESP_ERR_INVALID_ARGUMENT, "time_kernel_class: bad argument");
    if (kernel_class < K_QKV || kernel_class > K_HEAD) return fail(ESP_ERR_INVALID_ARGUMENT, "time_kernel_class: class %d", kernel_class);
    hipStream_t s = context().stream;
    const int kd = c_.kv_dim();
    const bool kv16 = c_.kv_format == FMT_F16;
    auto launch = [&](const Layer *L, hipEvent_t start = nullptr, hipEvent_t stop = nullptr) -> hipError_t {
        GemvParams g;
        g.batch = 1;
        g.start_event = start;
        g.stop_event = stop;
        switch (kernel_class) {
        case K_QKV:
            if (L->q_norm) { g.w = L->wqkv; g.norm_x = hidden_; g.norm_w = L->rms_att; g.norm_eps = c_.norm_eps; g.y = qkv_; g.epilogue = EPI_STORE_F32; break; }
            g.w = L->wqkv; g.norm_x = hidden_; g.norm_w = L->rms_att; g.norm_eps = c_.norm_eps; g.epilogue = EPI_QKV_ROPE;
            g.qkv.n_head = c_.n_head; g.qkv.n_kv_head = c_.n_kv_head; g.qkv.head_dim = c_.head_dim; g.qkv.max_seq = c_.max_seq;
            g.qkv.rope_cos = rope_cos_; g.qkv.rope_sin = rope_sin_; g.qkv.pos = d_pos_; g.qkv.seq = d_seq_;
            g.qkv.q_out = q_; g.qkv.k_cache = L->k_cache; g.qkv.v_cache = L->v_cache;
            g.qkv.cache_seq_stride = (size_t)kd * c_.max_seq; g.qkv.kv_f16 = kv16 ? 1 : 0;
            break;
        case K_WO:
            g.w = L->wo; g.x = ctx_; g.y = hidden_; g.residual = hidden_; g.epilogue = EPI_ADD_RESIDUAL;
            if (wo_merges_attention(*L, 1)) { g.x = nullptr; g.merge_partials = attn_scratch_; g.merge_head_dim = c_.head_dim; }
            break;
        case K_GATE_UP:
            g.w = L->w13; g.norm_x = hidden_; g.norm_w = L->rms_ffn; g.norm_eps = c_.norm_eps; g.out_f16 = act_; g.epilogue = EPI_SWIGLU_F16;
            g.split_out = split_activations_ && gemv_splits_activations(L->w2, 1);
            break;
        case K_DOWN: g.w = L->w2; g.x = act_; g.y = hidden_; g.residual = hidden_; g.epilogue = EPI_ADD_RESIDUAL; break;
        default:
            g.w = lm_head_; g.norm_x = hidden_; g.norm_w = final_norm_; g.norm_eps = c_.norm_eps; g.y = logits_; g.epilogue = EPI_STORE_F32;
            if (head_fuses_argmax()) {   // what a greedy step launches
                g.y = nullptr; g.epilogue = EPI_ARGMAX;
                g.argmax_value = argmax_scratch_.part_value; g.argmax_index = argmax_scratch_.part_index; g.argmax_capacity = head_partial_capacity_;
            }
            break;
        }
        // what the decode step launches: split activations wherever the GEMV takes them (not for fp16 rows given unsplit)
        g.split_x = kernel_class != K_HEAD && !(g.x == ctx_ && kernel_class == K_WO) && split_activations_ && gemv_splits_activations(g.w, 1);
        return launch_gemv(g, s);
    };
    StepRows rows{};
    rows.count = 1;
    ESP_HIP_TRY(launch_set_rows(rows, d_tokens_, d_pos_, d_seq_, s));
    hipEvent_t t0 = take_event(), t1 = take_event();
    if (!t0 || !t1) return fail(ESP_ERR_OUT_OF_MEMORY, "time_kernel_class: events");
    const int per_round = kernel_class == K_HEAD ? 1 : (int)layers_.size();
    for (int i = 0; i < per_round; i++) ESP_HIP_TRY(launch(kernel_class == K_HEAD ? nullptr : &layers_[(size_t)i]));   // warm-up round
    ESP_HIP_TRY(hipEventRecord(t0, s));
    for (int r = 0; r < iters; r++)
        for (int i = 0; i < per_round; i++) ESP_HIP_TRY(launch(kernel_class == K_HEAD ? nullptr : &layers_[(size_t)i]));
    ESP_HIP_TRY(hipEventRecord(t1, s));
    ESP_HIP_TRY(hipEventSynchronize(t1));
    float ms = 0.0f;
    ESP_HIP_TRY(hipEventElapsedTime(&ms, t0, t1));
    event_pool_.push_back(t0);
    event_pool_.push_back(t1);
    *mean_us = (double)ms * 1e3 / ((double)iters * per_round);
    if (kernel_only_us) {
        // the same launches again, each with events of its own that take the kernel's start and end
        std::vector<hipEvent_t> ev((size_t)iters * per_round * 2, nullptr);
        for (hipEvent_t &e : ev) if (!(e = take_event())) return fail(ESP_ERR_OUT_OF_MEMORY, "time_kernel_class: events");
        for (int r = 0, k = 0; r < iters; r++)
            for (int i = 0; i < per_round; i++, k += 2)
                ESP_HIP_TRY(launch(kernel_class == K_HEAD ? nullptr : &layers_[(size_t)i], ev[(size_t)k], ev[(size_t)k + 1]));
        ESP_HIP_TRY(hipStreamSynchronize(s));
        double total = 0.0;
        for (size_t k = 0; k < ev.size(); k += 2) {
            ESP_HIP_TRY(hipEventElapsedTime(&ms, ev[k], ev[k + 1]));
            total += ms;
        }
        for (hipEvent_t e : ev) event_pool_.push_back(e);
        *kernel_only_us = total * 1e3 / ((double)iters * per_round);
    }
    return ESP_OK;
}

size_t LlamaRuntime::kernel_bytes(int kernel_class) const {
    if (!finalized_ || layers_.empty()) return 0;
    const Layer &L = layers_[0];
    auto io = [](const DeviceMatrix &m) { return m.bytes() + (size_t)m.cols * 2 + (size_t)m.rows * 4; };
    switch (kernel_class) {
    case K_QKV: return io(L.wqkv);
    case K_WO: return io(L.wo);
    case K_GATE_UP: return io(L.w13);
    case K_DOWN: return io(L.w2);
    case K_HEAD: return io(lm_head_) - (head_fuses_argmax() ? (size_t)lm_head_.rows * 4 : 0);   // the fused head stores no logits
    default: return 0;
    }
}

LlamaRuntime::HostTensor *LlamaRuntime::host_slot(int layer, int slot) {
    switch (slot) {
    case SLOT_TOKEN_EMBEDDING: return &h_embedding_;
    case SLOT_FINAL_NORM: return &h_final_norm_;
    case SLOT_LM_HEAD: return &h_lm_head_;
    default: break;
    }
    if (layer < 0 || layer >= c_.n_layer) return nullptr;
    HostLayer &L = h_layers_[layer];
    switch (slot) {
    case SLOT_RMS_ATT: return &L.rms_att;
    case SLOT_WQ: return &L.wq;
    case SLOT_WK: return &L.wk;
    case SLOT_WV: return &L.wv;
    case SLOT_WO: return &L.wo;
    case SLOT_RMS_FFN: return &L.rms_ffn;
    case SLOT_W1: return &L.w1;
    case SLOT_W2: return &L.w2;
    case SLOT_W3: return &L.w3;
    case SLOT_Q_NORM: return &L.q_norm;
    case SLOT_K_NORM: return &L.k_norm;
    default: return nullptr;
    }
}

int LlamaRuntime::set_weight(int layer, int slot, int format, const void *data, size_t bytes) {
    if (finalized_) return fail(ESP_ERR_INVALID_ARGUMENT, "set_weight after finalize");
    HostTensor *t = host_slot(layer, slot);
    if (!t) return fail(ESP_ERR_INVALID_ARGUMENT, "set_weight: no slot %d in layer %d", slot, layer);
    if (!data || !format_supported(format)) return fail(ESP_ERR_INVALID_ARGUMENT, "set_weight: null data or unknown format %d", format);
    const size_t d = c_.d_model, ad = c_.attention_dim(), kd = c_.kv_dim(), hd = c_.hidden_dim;
    size_t elems = 0;
    switch (slot) {
    case SLOT_TOKEN_EMBEDDING: case SLOT_LM_HEAD: elems = (size_t)c_.vocab * d; break;
    case SLOT_FINAL_NORM: case SLOT_RMS_ATT: case SLOT_RMS_FFN: elems = d; break;
    case SLOT_WQ: case SLOT_WO: elems = ad * d; break;
    case SLOT_WK: case SLOT_WV: elems = kd * d; break;
    case SLOT_W1: case SLOT_W2: case SLOT_W3: elems = hd * d; break;
    case SLOT_Q_NORM: case SLOT_K_NORM: elems = (size_t)c_.head_dim; break;
    }
    const bool is_vector = slot == SLOT_FINAL_NORM || slot == SLOT_RMS_ATT || slot == SLOT_RMS_FFN ||
                           slot == SLOT_Q_NORM || slot == SLOT_K_NORM || slot == SLOT_TOKEN_EMBEDDING;
    if (is_vector && format != FMT_F32 && format != FMT_F16)
        return fail(ESP_ERR_UNSUPPORTED, "set_weight: slot %d takes f32 or f16 values", slot);
    if (elems % format_block_elems(format) != 0 || bytes != format_bytes(format, elems))
        return fail(ESP_ERR_INVALID_ARGUMENT, "set_weight: slot %d expects %zu elements (%zu bytes in format %d), got %zu bytes",
                    slot, elems, format_bytes(format, elems), format, bytes);
    t->format = format;
    t->bytes.assign(static_cast<const uint8_t *>(data), static_cast<const uint8_t *>(data) + bytes);
    return ESP_OK;
}

int LlamaRuntime::upload_vector(const HostTensor &t, size_t count, float **out, const char *what) {
    if (t.format < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "finalize: missing weight %s", what);
    std::vector<float> v(count);
    if (t.format == FMT_F32) std::memcpy(v.data(), t.bytes.data(), count * 4);
    else for (size_t i = 0; i < count; i++) v[i] = half_to_float_host((uint16_t)(t.bytes[2 * i] | (t.bytes[2 * i + 1] << 8)));
    int rc = device_alloc(out, count);
    if (rc != ESP_OK) return rc;
    ESP_HIP_TRY(hipMemcpy(*out, v.data(), count * 4, hipMemcpyHostToDevice));
    return ESP_OK;
}

int LlamaRuntime::finalize() {
    if (finalized_) return ESP_OK;
    const int d = c_.d_model, ad = c_.attention_dim(), kd = c_.kv_dim(), hd = c_.hidden_dim, half = c_.head_dim / 2;
    int rc;
    // ---- top level ----
    if (h_embedding_.format < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "finalize: missing token embedding");
    embedding_f16_ = h_embedding_.format == FMT_F16;
    {
        uint8_t *p = nullptr;
        if ((rc = device_alloc(&p, h_embedding_.bytes.size())) != ESP_OK) return rc;
        embedding_ = p;
        ESP_HIP_TRY(hipMemcpy(embedding_, h_embedding_.bytes.data(), h_embedding_.bytes.size(), hipMemcpyHostToDevice));
    }
    if ((rc = upload_vector(h_final_norm_, d, &final_norm_, "rms_final")) != ESP_OK) return rc;
    if (h_lm_head_.format < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "finalize: missing lm_head");
    if ((rc = matrix_upload(h_lm_head_.format, h_lm_head_.bytes.data(), c_.vocab, d, &lm_head_)) != ESP_OK) return rc;
    weight_bytes_ = lm_head_.bytes();
    resident_weight_bytes_ = lm_head_.resident_bytes() + h_embedding_.bytes.size();

    // ---- layers ----
    layers_.resize(c_.n_layer);
    const size_t cache_elems = (size_t)c_.max_sequences * kd * c_.max_seq;
    const size_t cache_bytes = cache_elems * (c_.kv_format == FMT_F16 ? 2 : 4);
    std::vector<uint8_t> fused;
    for (int l = 0; l < c_.n_layer; l++) {
        HostLayer &H = h_layers_[l];
        Layer &L = layers_[l];
        const HostTensor *need[] = {&H.wq, &H.wk, &H.wv, &H.wo, &H.w1, &H.w2, &H.w3};
        for (const HostTensor *t : need)
            if (t->format < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "finalize: layer %d is missing a projection weight", l);
        if (H.wq.format != H.wk.format || H.wq.format != H.wv.format)
            return fail(ESP_ERR_UNSUPPORTED, "finalize: layer %d wq/wk/wv must share one format", l);
        if (H.w1.format != H.w3.format) return fail(ESP_ERR_UNSUPPORTED, "finalize: layer %d w1/w3 must share one format", l);
        if ((rc = upload_vector(H.rms_att, d, &L.rms_att, "rms_att")) != ESP_OK) return rc;
        if ((rc = upload_vector(H.rms_ffn, d, &L.rms_ffn, "rms_ffn")) != ESP_OK) return rc;
        // q_norm/k_norm are optional and only used when both exist (:6585-6607)
        if (H.q_norm.format >= 0 && H.k_norm.format >= 0) {
            if ((rc = upload_vector(H.q_norm, c_.head_dim, &L.q_norm, "q_norm")) != ESP_OK) return rc;
            if ((rc = upload_vector(H.k_norm, c_.head_dim, &L.k_norm, "k_norm")) != ESP_OK) return rc;
        }
        // fused QKV: q and k rows reordered so that the two rows of a RoPE pair (j, j + half) are
        // adjacent; v rows in natural order.
        {
            const size_t rb = format_bytes(H.wq.format, d);
            fused.resize((size_t)(ad + 2 * kd) * rb);
            size_t o = 0;
            auto put_rope_rows = [&](const HostTensor &t, int heads) {
                for (int h = 0; h < heads; h++)
                    for (int j = 0; j < half; j++) {
                        std::memcpy(&fused[o], &t.bytes[(size_t)(h * c_.head_dim + j) * rb], rb); o += rb;
                        std::memcpy(&fused[o], &t.bytes[(size_t)(h * c_.head_dim + j + half) * rb], rb); o += rb;
                    }
            };
            put_rope_rows(H.wq, c_.n_head);
            put_rope_rows(H.wk, c_.n_kv_head);
            std::memcpy(&fused[o], H.wv.bytes.data(), (size_t)kd * rb);
            if ((rc = matrix_upload(H.wq.format, fused.data(), ad + 2 * kd, d, &L.wqkv)) != ESP_OK) return rc;
        }
        // fused gate/up: rows interleaved (g0, u0, g1, u1, ...)
        {
            const size_t rb = format_bytes(H.w1.format, d);
            fused.resize((size_t)2 * hd * rb);
            for (int i = 0; i < hd; i++) {
                std::memcpy(&fused[(size_t)(2 * i) * rb], &H.w1.bytes[(size_t)i * rb], rb);
                std::memcpy(&fused[(size_t)(2 * i + 1) * rb], &H.w3.bytes[(size_t)i * rb], rb);
            }
            if ((rc = matrix_upload(H.w1.format, fused.data(), 2 * hd, d, &L.w13)) != ESP_OK) return rc;
        }
        if ((rc = matrix_upload(H.wo.format, H.wo.bytes.data(), d, ad, &L.wo)) != ESP_OK) return rc;
        if ((rc = matrix_upload(H.w2.format, H.w2.bytes.data(), d, hd, &L.w2)) != ESP_OK) return rc;
        weight_bytes_ += L.wqkv.bytes() + L.wo.bytes() + L.w13.bytes() + L.w2.bytes();
        resident_weight_bytes_ += L.wqkv.resident_bytes() + L.wo.resident_bytes() + L.w13.resident_bytes() + L.w2.resident_bytes();
        uint8_t *kc = nullptr, *vc = nullptr;
        if ((rc = device_alloc(&kc, cache_bytes)) != ESP_OK) return rc;
        L.k_cache = kc;
        if ((rc = device_alloc(&vc, cache_bytes)) != ESP_OK) return rc;
        L.v_cache = vc;
        H = HostLayer{};  // drop the host copy
    }
    h_embedding_ = HostTensor{}; h_lm_head_ = HostTensor{};
    fused.clear(); fused.shrink_to_fit();

    // ---- RoPE table, computed on the host with the reference's float expressions (:6759-6762) ----
    {
        std::vector<float> cs((size_t)c_.max_seq * half), sn((size_t)c_.max_seq * half);
        for (int p = 0; p < c_.max_seq; p++)
            for (int j = 0; j < half; j++) {
                const float frequency = 1.0f / powf(c_.rope_theta, (float)(2 * j) / (float)c_.head_dim);
                const float angle = (float)p * frequency;
                cs[(size_t)p * half + j] = cosf(angle);
                sn[(size_t)p * half + j] = sinf(angle);
            }
        if ((rc = device_alloc(&rope_cos_, cs.size())) != ESP_OK) return rc;
        if ((rc = device_alloc(&rope_sin_, sn.size())) != ESP_OK) return rc;
        ESP_HIP_TRY(hipMemcpy(rope_cos_, cs.data(), cs.size() * 4, hipMemcpyHostToDevice));
        ESP_HIP_TRY(hipMemcpy(rope_sin_, sn.data(), sn.size() * 4, hipMemcpyHostToDevice));
    }
    // ---- activations ----
    const size_t R = kPrefillBlockRows > kMaxStepRows ? kPrefillBlockRows : kMaxStepRows, RS = kMaxStepRows;
    if ((rc = device_alloc(&hidden_, R * d)) != ESP_OK) return rc;
    if ((rc = device_alloc(&qkv_, R * (ad + 2 * kd))) != ESP_OK) return rc;
    if ((rc = device_alloc(&q_, R * ad)) != ESP_OK) return rc;
    if ((rc = device_alloc(&gu_, R * 2 * hd)) != ESP_OK) return rc;
    if ((rc = device_alloc(&logits_, RS * c_.vocab)) != ESP_OK) return rc;
    if ((rc = device_alloc(&last_hidden_, (size_t)c_.max_sequences * d)) != ESP_OK) return rc;
    if ((rc = device_alloc(&xn_, R * (size_t)(d > hd ? d : hd))) != ESP_OK) return rc;
    if ((rc = device_alloc(&ctx_, R * ad)) != ESP_OK) return rc;
    if ((rc = device_alloc(&act_, R * hd)) != ESP_OK) return rc;
    if (d % 256 == 0 && ad % 256 == 0 && hd % 256 == 0) {   // split rows for prompt blocks (Q4_K models)
        if ((rc = device_alloc(&xn_lo_, R * (size_t)d)) != ESP_OK) return rc;
        if ((rc = device_alloc(&ctx_lo_, R * (size_t)ad)) != ESP_OK) return rc;
        if ((rc = device_alloc(&act_lo_, R * (size_t)hd)) != ESP_OK) return rc;
        if ((rc = device_alloc(&xn_sums_, R * (size_t)(d / 16))) != ESP_OK) return rc;
        if ((rc = device_alloc(&ctx_sums_, R * (size_t)(ad / 16))) != ESP_OK) return rc;
        if ((rc = device_alloc(&act_sums_, R * (size_t)(hd / 16))) != ESP_OK) return rc;
    }
    if ((rc = device_alloc(&d_tokens_, R)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_pos_, R)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_seq_, R)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_out_tokens_, R)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_visible_, (size_t)c_.max_sequences)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_log_, (size_t)c_.max_seq)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_log_count_, 3)) != ESP_OK) return rc;   // tokens logged, stopped, stop enabled (greedy_tail_kernel)
    step_graphs_.assign(c_.max_sequences, nullptr);
    multi_graphs_.assign(c_.max_sequences, nullptr);
    // one (value, index) pair per workgroup of the head GEMV and row: a workgroup owns eight rows, or the grid is persistent
    head_partial_capacity_ = (c_.vocab + 7) / 8 > 4096 ? (c_.vocab + 7) / 8 : 4096;
    const size_t argmax_slots = (size_t)2 * head_partial_capacity_ > (size_t)kArgmaxScratchSlots ? (size_t)2 * head_partial_capacity_ : (size_t)kArgmaxScratchSlots;
    if ((rc = device_alloc(&argmax_scratch_.part_value, argmax_slots)) != ESP_OK) return rc;
    if ((rc = device_alloc(&argmax_scratch_.part_index, argmax_slots)) != ESP_OK) return rc;
    {
        const size_t per_row = (size_t)c_.n_kv_head * kAttentionMaxSplits * (c_.n_head / c_.n_kv_head) * (c_.head_dim + 2);
        if ((rc = device_alloc(&attn_scratch_, R * per_row)) != ESP_OK) return rc;
    }
    if ((rc = device_alloc(&gemm_workspace_, kGemmWorkspaceFloats)) != ESP_OK) return rc;
    if (gemm_split_shared_k_pool(&gemm_shared_k_) != hipSuccess) {   // without the pool the prompt GEMM keeps its plain grid
        (void)hipGetLastError();
        gemm_shared_k_ = GemmSplitSharedK{};
    }
    {
        const char *pa = getenv("ESPRESSO_HIP_PROMPT_ATTENTION");   // "0": prompt blocks keep the single-query attention kernel
        prompt_attention_ = attention_prompt_supported(c_.n_head, c_.n_kv_head, c_.head_dim) && !(pa && pa[0] == '0');
        const char *fh = getenv("ESPRESSO_HIP_FUSED_HEAD_ARGMAX");   // "0": the head stores logits and separate launches pick the token
        fused_head_argmax_ = !(fh && fh[0] == '0');
        const char *sa = getenv("ESPRESSO_HIP_SPLIT_ACTIVATIONS");   // "0": activations rounded to fp16 once
        if (sa && sa[0] == '0') split_activations_ = false;
    }
    finalized_ = true;
    return reset();
}

int LlamaRuntime::reset() {
    if (!finalized_) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    Context &ctx = context();
    const size_t cache_bytes = (size_t)c_.max_sequences * c_.kv_dim() * c_.max_seq * (c_.kv_format == FMT_F16 ? 2 : 4);
    for (Layer &L : layers_) {
        ESP_HIP_TRY(hipMemsetAsync(L.k_cache, 0, cache_bytes, ctx.stream));
        ESP_HIP_TRY(hipMemsetAsync(L.v_cache, 0, cache_bytes, ctx.stream));
    }
    ESP_HIP_TRY(hipMemsetAsync(last_hidden_, 0, (size_t)c_.max_sequences * c_.d_model * 4, ctx.stream));
    ESP_HIP_TRY(hipStreamSynchronize(ctx.stream));
    std::fill(visible_.begin(), visible_.end(), 0);
    return ESP_OK;
}

int LlamaRuntime::visible(int seq) const {
    return seq >= 0 && seq < c_.max_sequences ? visible_[seq] : -1;
}

int LlamaRuntime::set_visible(int seq, int count) {
    if (seq < 0 || seq >= c_.max_sequences || count < 0 || count > c_.max_seq)
        return fail(ESP_ERR_OUT_OF_RANGE, "set_visible(seq %d, count %d) out of range", seq, count);
    visible_[seq] = count;
    return ESP_OK;
}

int LlamaRuntime::forward_rows(const StepRows &rows) {
    if (!finalized_) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    if (rows.count < 1 || rows.count > kMaxStepRows) return fail(ESP_ERR_INVALID_ARGUMENT, "forward_rows: %d rows", rows.count);
    for (int i = 0; i < rows.count; i++) {
        if (rows.token[i] < 0 || rows.token[i] >= c_.vocab)
            return fail(ESP_ERR_OUT_OF_RANGE, "token %d is outside vocab %d", rows.token[i], c_.vocab);   // (:687-689)
        if (rows.pos[i] < 0 || rows.pos[i] >= c_.max_seq)
            return fail(ESP_ERR_OUT_OF_RANGE, "position %d exceeds context %d", rows.pos[i], c_.max_seq);  // (:673-677)
        if (rows.seq[i] < 0 || rows.seq[i] >= c_.max_sequences)
            return fail(ESP_ERR_OUT_OF_RANGE, "sequence %d of %d", rows.seq[i], c_.max_sequences);
    }
    ESP_HIP_TRY(launch_set_rows(rows, d_tokens_, d_pos_, d_seq_, context().stream));
    return enqueue_trunk(rows.count);
}

// The trunk over `M` rows whose (token, position, sequence) already sit in d_tokens_/d_pos_/d_seq_.
int LlamaRuntime::enqueue_trunk(int M, bool embedded, float *final_out) {
    hipStream_t s = context().stream;
    const int d = c_.d_model, ad = c_.attention_dim(), kd = c_.kv_dim(), hd = c_.hidden_dim;
    const bool kv16 = c_.kv_format == FMT_F16;
    int rc = ESP_OK;
    if (!embedded) ESP_HIP_TRY(launch_embed(embedding_, embedding_f16_, d_tokens_, M, d, hidden_, s));
    if (timing_enabled_) {   // an empty event pair: the overhead the pairs around real kernels carry
        if ((rc = time_begin(K_EVENT_PAIR)) != ESP_OK) return rc;
        if ((rc = time_end()) != ESP_OK) return rc;
    }
    // more than two rows (batched sequences, batched verify): one pass over the weights on the matrix cores
    if (M > 2 && matrix_prefill_ && matrix_prefill_supported()) return enqueue_layers_matrix(M);
    for (Layer &L : layers_) {
        // both RMSNorms of the layer run inside the staging of the GEMV that consumes them
        GemvParams g;
        g.w = L.wqkv; g.norm_x = hidden_; g.norm_w = L.rms_att; g.norm_eps = c_.norm_eps; g.batch = M;
        // Activations reach the matrix cores as hi / lo fp16 pairs wherever the GEMV has that form (GemvParams::split_x)
        g.split_x = split_activations_ && gemv_splits_activations(L.wqkv, M);
        const size_t cache_seq_stride = (size_t)kd * c_.max_seq;
        if (L.q_norm) {
            // per-head q/k norm needs whole heads before RoPE: plain GEMV, then the post kernel
            g.y = qkv_; g.epilogue = EPI_STORE_F32;
            if ((rc = time_begin(K_QKV)) != ESP_OK) return rc;
            ESP_HIP_TRY(launch_gemv(g, s));
            if ((rc = time_end()) != ESP_OK) return rc;
            QkvPostArgs qa{};
            qa.qkv = qkv_; qa.q_norm = L.q_norm; qa.k_norm = L.k_norm; qa.norm_eps = c_.norm_eps;
            qa.n_head = c_.n_head; qa.n_kv_head = c_.n_kv_head; qa.head_dim = c_.head_dim; qa.max_seq = c_.max_seq;
            qa.rope_cos = rope_cos_; qa.rope_sin = rope_sin_; qa.pos = d_pos_; qa.seq = d_seq_;
            qa.q_out = q_; qa.k_cache = L.k_cache; qa.v_cache = L.v_cache; qa.cache_seq_stride = cache_seq_stride;
            ESP_HIP_TRY(launch_qkv_post(qa, M, kv16, s));
        } else {
            g.epilogue = EPI_QKV_ROPE;
            g.qkv.n_head = c_.n_head; g.qkv.n_kv_head = c_.n_kv_head; g.qkv.head_dim = c_.head_dim; g.qkv.max_seq = c_.max_seq;
            g.qkv.rope_cos = rope_cos_; g.qkv.rope_sin = rope_sin_; g.qkv.pos = d_pos_; g.qkv.seq = d_seq_;
            g.qkv.q_out = q_; g.qkv.k_cache = L.k_cache; g.qkv.v_cache = L.v_cache;
            g.qkv.cache_seq_stride = cache_seq_stride; g.qkv.kv_f16 = kv16 ? 1 : 0;
            if ((rc = time_begin(K_QKV)) != ESP_OK) return rc;
            ESP_HIP_TRY(launch_gemv(g, s));
            if ((rc = time_end()) != ESP_OK) return rc;
        }
        AttentionArgs aa{};
        aa.q = q_; aa.k_cache = L.k_cache; aa.v_cache = L.v_cache; aa.cache_seq_stride = cache_seq_stride;
        aa.n_head = c_.n_head; aa.n_kv_head = c_.n_kv_head; aa.head_dim = c_.head_dim; aa.max_seq = c_.max_seq;
        aa.pos = d_pos_; aa.seq = d_seq_; aa.ctx_f16 = ctx_;
        aa.split_scratch = attn_scratch_;
        aa.head_partials = attn_scratch_;
        // one attention launch instead of two where the wo GEMV can merge the partial states in its staging
        const bool merge_in_wo = wo_merges_attention(L, M);
        if ((rc = time_begin(K_ATTENTION)) != ESP_OK) return rc;
        if (merge_in_wo) ESP_HIP_TRY(launch_attention_partials(aa, M, kv16, s));
        else ESP_HIP_TRY(launch_attention(aa, M, kv16, s));
        if ((rc = time_end()) != ESP_OK) return rc;
        g = GemvParams{};
        g.batch = M;
        g.w = L.wo; g.x = ctx_; g.y = hidden_; g.residual = hidden_; g.epilogue = EPI_ADD_RESIDUAL;
        if (merge_in_wo) {
            g.x = nullptr; g.merge_partials = attn_scratch_; g.merge_head_dim = c_.head_dim;
            g.split_x = split_activations_ && gemv_splits_activations(L.wo, M);   // the merge leaves fp32 values to split
        }
        if ((rc = time_begin(K_WO)) != ESP_OK) return rc;
        ESP_HIP_TRY(launch_gemv(g, s));
        if ((rc = time_end()) != ESP_OK) return rc;
        g.w = L.w13; g.x = nullptr; g.merge_partials = nullptr; g.norm_x = hidden_; g.norm_w = L.rms_ffn; g.norm_eps = c_.norm_eps;
        g.y = nullptr; g.residual = nullptr; g.out_f16 = act_; g.epilogue = EPI_SWIGLU_F16;
        const bool split_down = split_activations_ && gemv_splits_activations(L.w2, M);   // act_ then holds hi / lo row pairs
        g.split_x = split_activations_ && gemv_splits_activations(L.w13, M);
        g.split_out = split_down;
        if ((rc = time_begin(K_GATE_UP)) != ESP_OK) return rc;
        ESP_HIP_TRY(launch_gemv(g, s));
        if ((rc = time_end()) != ESP_OK) return rc;
        g.w = L.w2; g.x = act_; g.norm_x = nullptr; g.norm_w = nullptr; g.split_x = split_down; g.split_out = false;
        g.y = final_out && &L == &layers_.back() ? final_out : hidden_;   // the last layer's output may go straight to its keeper
        g.residual = hidden_; g.out_f16 = nullptr; g.epilogue = EPI_ADD_RESIDUAL;
        if ((rc = time_begin(K_DOWN)) != ESP_OK) return rc;
        ESP_HIP_TRY(launch_gemv(g, s));
        if ((rc = time_end()) != ESP_OK) return rc;
    }
    (void)ad;
    return ESP_OK;
}

void LlamaRuntime::drop_captured_graphs() {
    for (auto &g : step_graphs_) if (g) { (void)hipGraphExecDestroy(g); g = nullptr; }
    for (auto &g : multi_graphs_) if (g) { (void)hipGraphExecDestroy(g); g = nullptr; }
    graph_epoch_++;
}

// esp_set_tuning changes which kernels launch_gemv picks: graphs captured before it would keep replaying the old ones.
void LlamaRuntime::sync_tuning() {
    const unsigned e = gemv_tuning_epoch();
    if (e == tuning_epoch_) return;
    tuning_epoch_ = e;
    drop_captured_graphs();
}

void LlamaRuntime::set_split_activations(bool enabled) {
    if (enabled == split_activations_) return;
    split_activations_ = enabled;
    drop_captured_graphs();   // captured with the other kernels
}

void LlamaRuntime::set_merged_attention(bool enabled) {
    if (enabled == merged_attention_) return;
    merged_attention_ = enabled;
    drop_captured_graphs();   // captured with the other path
}

void LlamaRuntime::release_loop_session() {
    DeviceLoopSession &ss = loop_session_;
    if (ss.one) (void)hipGraphExecDestroy(ss.one);
    if (ss.many) (void)hipGraphExecDestroy(ss.many);
    if (ss.state) (void)hipFree(ss.state);
    if (ss.log) (void)hipFree(ss.log);
    ss = DeviceLoopSession{};
}

int LlamaRuntime::keep_row(int row, int seq) {
    if (row < 0 || row >= kPrefillBlockRows || seq < 0 || seq >= c_.max_sequences)
        return fail(ESP_ERR_OUT_OF_RANGE, "keep_row(%d, %d)", row, seq);
    ESP_HIP_TRY(launch_copy_rows(hidden_ + (size_t)row * c_.d_model, last_hidden_ + (size_t)seq * c_.d_model, 1, c_.d_model,
                                 context().stream));
    return ESP_OK;
}

int LlamaRuntime::advance(int seq, uint32_t token) {
    if (seq < 0 || seq >= c_.max_sequences) return fail(ESP_ERR_OUT_OF_RANGE, "sequence %d of %d", seq, c_.max_sequences);
    if (visible_[seq] >= c_.max_seq)
        return fail(ESP_ERR_OUT_OF_RANGE, "runtime position %d exceeds context %d", visible_[seq], c_.max_seq);
    if (token >= (uint32_t)c_.vocab) return fail(ESP_ERR_OUT_OF_RANGE, "token %u is outside vocab %d", token, c_.vocab);
    StepRows rows{};
    rows.count = 1; rows.token[0] = (int)token; rows.pos[0] = visible_[seq]; rows.seq[0] = seq;
    int rc = forward_rows(rows);
    if (rc != ESP_OK) return rc;
    if ((rc = keep_row(0, seq)) != ESP_OK) return rc;
    visible_[seq] += 1;
    return ESP_OK;
}

int LlamaRuntime::prefill(int seq, const uint32_t *tokens, int count) {
    if (count <= 0 || !tokens) return fail(ESP_ERR_INVALID_ARGUMENT, "Prompt tokens must not be empty");
    if (seq < 0 || seq >= c_.max_sequences) return fail(ESP_ERR_OUT_OF_RANGE, "sequence %d of %d", seq, c_.max_sequences);
    visible_[seq] = 0;
    if (matrix_prefill_ && count >= kMatrixPrefillMinTokens && matrix_prefill_supported()) {
        // long prompts: blocks of rows through the MFMA kernels (one pass over the weights per block)
        if (count > c_.max_seq) return fail(ESP_ERR_OUT_OF_RANGE, "runtime position %d exceeds context %d", c_.max_seq, c_.max_seq);
        for (int i = 0; i < count; i++)
            if (tokens[i] >= (uint32_t)c_.vocab) return fail(ESP_ERR_OUT_OF_RANGE, "token %u is outside vocab %d", tokens[i], c_.vocab);
        int rc = ESP_OK;
        for (int base = 0; base < count && rc == ESP_OK; base += kPrefillBlockRows) {
            const int rows = count - base < kPrefillBlockRows ? count - base : kPrefillBlockRows;
            rc = prefill_block(seq, tokens + base, rows, base);
            if (rc == ESP_OK && base + rows == count) rc = keep_row(rows - 1, seq);
        }
        if (rc != ESP_OK) return rc;
        ESP_HIP_TRY(hipStreamSynchronize(context().stream));
        visible_[seq] = count;
        return ESP_OK;
    }
    for (int i = 0; i < count; i++) {
        int rc = advance(seq, tokens[i]);
        if (rc != ESP_OK) return rc;
    }
    return ESP_OK;
}

bool LlamaRuntime::matrix_prefill_supported() const {
    auto ok = [](const DeviceMatrix &m) { return m.format != FMT_F32 && m.cols % 64 == 0; };
    for (const Layer &L : layers_)
        if (!ok(L.wqkv) || !ok(L.wo) || !ok(L.w13) || !ok(L.w2)) return false;
    return true;
}

// `rows` prompt tokens at positions base.. of one sequence: the layer loop of forwardToken (:6221-6347) over
// a block of rows, every projection as one dequant-fused MFMA GEMM.  Rows of the block see each other's
// keys and values causally because the whole block's K/V is written before its attention runs.
int LlamaRuntime::prefill_block(int seq, const uint32_t *tokens, int rows, int base) {
    hipStream_t s = context().stream;
    const int d = c_.d_model, ad = c_.attention_dim(), kd = c_.kv_dim(), hd = c_.hidden_dim;
    const bool kv16 = c_.kv_format == FMT_F16;
    std::vector<int> h_tok(rows), h_pos(rows), h_seq(rows, seq);
    for (int i = 0; i < rows; i++) { h_tok[i] = (int)tokens[i]; h_pos[i] = base + i; }
    ESP_HIP_TRY(hipMemcpyAsync(d_tokens_, h_tok.data(), sizeof(int) * rows, hipMemcpyHostToDevice, s));
    ESP_HIP_TRY(hipMemcpyAsync(d_pos_, h_pos.data(), sizeof(int) * rows, hipMemcpyHostToDevice, s));
    ESP_HIP_TRY(hipMemcpyAsync(d_seq_, h_seq.data(), sizeof(int) * rows, hipMemcpyHostToDevice, s));
    ESP_HIP_TRY(hipStreamSynchronize(s));   // the host vectors go out of scope
    ESP_HIP_TRY(launch_embed(embedding_, embedding_f16_, d_tokens_, rows, d, hidden_, s));
    (void)ad; (void)kd; (void)hd; (void)kv16;
    return enqueue_layers_matrix(rows, true);
}

// The layer loop over `rows` rows whose embeddings sit in hidden_ and whose (position, sequence) sit in
// d_pos_/d_seq_, every projection as one dequant-fused MFMA GEMM.  Rows that are one sequence at consecutive positions
// (a prompt block) take the matrix-core attention kernel, others the single-query one.
// Prompt blocks of Q4_K models: every projection with exact weights and split activations (launch_gemm_split), queries and softmax
// weights split in the attention: the block then stays as close to the fp32 CPU walk as the decode steps do.
bool LlamaRuntime::split_blocks_supported() const {
    if (!split_activations_ || !xn_lo_ || !prompt_attention_ || c_.kv_format != FMT_F16 || c_.d_model > 8192) return false;
    for (const Layer &L : layers_)
        if (L.q_norm || !gemm_split_supported(L.wqkv) || !gemm_split_supported(L.wo) || !gemm_split_supported(L.w13) || !gemm_split_supported(L.w2)) return false;
    return true;
}

int LlamaRuntime::enqueue_layers_split(int rows) {
    hipStream_t s = context().stream;
    const int d = c_.d_model, ad = c_.attention_dim(), kd = c_.kv_dim(), hd = c_.hidden_dim;
    const size_t cache_seq_stride = (size_t)kd * c_.max_seq;
    SplitRowsView xn{xn_, xn_lo_, xn_sums_}, ctx{ctx_, ctx_lo_, ctx_sums_}, act{act_, act_lo_, act_sums_};
    // RMSNorm of hidden_ (or of the split-K planes a projection left, added to hidden_ first) into split rows
    auto norm = [&](const float *w, int splits) -> hipError_t {
        SplitRowsParams p;
        p.rows = rows; p.cols = d; p.norm_w = w; p.norm_eps = c_.norm_eps; p.out = xn;
        if (splits > 1) { p.x = gemm_workspace_; p.splits = splits; p.plane = (size_t)rows * d; p.residual = hidden_; p.y = hidden_; }
        else p.x = hidden_;
        return launch_split_rows(p, s);
    };
    ESP_HIP_TRY(norm(layers_.front().rms_att, 1));
    for (size_t li = 0; li < layers_.size(); li++) {
        Layer &L = layers_[li];
        GemmSplitParams g;
        g.rows = rows; g.workspace = gemm_workspace_; g.workspace_floats = kGemmWorkspaceFloats;
        int splits = 1;
        g.w = L.wqkv; g.x = xn; g.y = qkv_; g.deferred_splits = &splits;
        ESP_HIP_TRY(launch_gemm_split(g, s));
        QkvPostArgs qa{};
        qa.qkv = splits > 1 ? gemm_workspace_ : qkv_; qa.splits = splits; qa.plane = (size_t)rows * (ad + 2 * kd);
        qa.q_norm = nullptr; qa.k_norm = nullptr; qa.norm_eps = c_.norm_eps;
        qa.n_head = c_.n_head; qa.n_kv_head = c_.n_kv_head; qa.head_dim = c_.head_dim; qa.max_seq = c_.max_seq;
        qa.rope_cos = rope_cos_; qa.rope_sin = rope_sin_; qa.pos = d_pos_; qa.seq = d_seq_;
        qa.q_out = q_; qa.k_cache = L.k_cache; qa.v_cache = L.v_cache; qa.cache_seq_stride = cache_seq_stride;
        ESP_HIP_TRY(launch_qkv_post(qa, rows, true, s));
        AttentionArgs aa{};
        aa.q = q_; aa.k_cache = L.k_cache; aa.v_cache = L.v_cache; aa.cache_seq_stride = cache_seq_stride;
        aa.n_head = c_.n_head; aa.n_kv_head = c_.n_kv_head; aa.head_dim = c_.head_dim; aa.max_seq = c_.max_seq;
        aa.pos = d_pos_; aa.seq = d_seq_; aa.ctx_hi = ctx.hi; aa.ctx_lo = ctx.lo; aa.ctx_sums = ctx.sums;
        ESP_HIP_TRY(launch_attention_prompt(aa, rows, true, s));
        g.w = L.wo; g.x = ctx; g.y = hidden_; g.residual = hidden_; splits = 1;
        ESP_HIP_TRY(launch_gemm_split(g, s));
        ESP_HIP_TRY(norm(L.rms_ffn, splits));
        g.w = L.w13; g.x = xn; g.y = nullptr; g.residual = nullptr; g.swiglu = act; g.deferred_splits = nullptr;
        g.shared_k = &gemm_shared_k_;
        ESP_HIP_TRY(launch_gemm_split(g, s));
        g.swiglu = SplitRowsView{}; g.shared_k = nullptr;
        const bool last = li + 1 == layers_.size();
        g.w = L.w2; g.x = act; g.y = hidden_; g.residual = hidden_; splits = 1; g.deferred_splits = last ? nullptr : &splits;
        ESP_HIP_TRY(launch_gemm_split(g, s));
        if (!last) ESP_HIP_TRY(norm(layers_[li + 1].rms_att, splits));
    }
    return ESP_OK;
}

int LlamaRuntime::enqueue_layers_matrix(int rows, bool one_sequence_consecutive) {
    if (one_sequence_consecutive && split_blocks_supported()) return enqueue_layers_split(rows);
    hipStream_t s = context().stream;
    const int d = c_.d_model, ad = c_.attention_dim(), kd = c_.kv_dim(), hd = c_.hidden_dim;
    const bool kv16 = c_.kv_format == FMT_F16;
    const size_t cache_seq_stride = (size_t)kd * c_.max_seq;
    GemmParams g;
    g.rows = rows; g.workspace = gemm_workspace_; g.workspace_floats = kGemmWorkspaceFloats;
    // The RMSNorm that follows a projection with a residual reads that projection's result; when the GEMM ran split-K the
    // norm kernel adds the partial sums itself (one launch instead of reduce + norm).
    const bool fuse_norm = rmsnorm_reduce_supported(d);
    auto project_and_norm = [&](const float *norm_w) -> int {   // g is set up for a GEMM into hidden_ with hidden_ as residual
        int splits = 1;
        g.deferred_splits = norm_w && fuse_norm ? &splits : nullptr;
        ESP_HIP_TRY(launch_gemm(g, s));
        g.deferred_splits = nullptr;
        if (!norm_w) return ESP_OK;
        if (splits > 1) ESP_HIP_TRY(launch_rmsnorm_reduce(gemm_workspace_, splits, (size_t)rows * d, hidden_, hidden_, norm_w, c_.norm_eps, rows, d, xn_, s));
        else ESP_HIP_TRY(launch_rmsnorm(hidden_, norm_w, c_.norm_eps, rows, d, xn_, nullptr, s));
        return ESP_OK;
    };
    ESP_HIP_TRY(launch_rmsnorm(hidden_, layers_.front().rms_att, c_.norm_eps, rows, d, xn_, nullptr, s));
    for (size_t li = 0; li < layers_.size(); li++) {
        Layer &L = layers_[li];
        int qkv_splits = 1;   // split-K partial sums of q|k|v are added by the kernel that applies norm / RoPE and writes the caches
        g.w = L.wqkv; g.x = xn_; g.y = qkv_; g.residual = nullptr; g.deferred_splits = &qkv_splits;
        ESP_HIP_TRY(launch_gemm(g, s));
        g.deferred_splits = nullptr;
        QkvPostArgs qa{};
        qa.qkv = qkv_splits > 1 ? gemm_workspace_ : qkv_; qa.splits = qkv_splits; qa.plane = (size_t)rows * (ad + 2 * kd);
        qa.q_norm = L.q_norm; qa.k_norm = L.k_norm; qa.norm_eps = c_.norm_eps;
        qa.n_head = c_.n_head; qa.n_kv_head = c_.n_kv_head; qa.head_dim = c_.head_dim; qa.max_seq = c_.max_seq;
        qa.rope_cos = rope_cos_; qa.rope_sin = rope_sin_; qa.pos = d_pos_; qa.seq = d_seq_;
        qa.q_out = q_; qa.k_cache = L.k_cache; qa.v_cache = L.v_cache; qa.cache_seq_stride = cache_seq_stride;
        ESP_HIP_TRY(launch_qkv_post(qa, rows, kv16, s));
        AttentionArgs aa{};
        aa.q = q_; aa.k_cache = L.k_cache; aa.v_cache = L.v_cache; aa.cache_seq_stride = cache_seq_stride;
        aa.n_head = c_.n_head; aa.n_kv_head = c_.n_kv_head; aa.head_dim = c_.head_dim; aa.max_seq = c_.max_seq;
        aa.pos = d_pos_; aa.seq = d_seq_; aa.ctx_f16 = ctx_; aa.split_scratch = attn_scratch_;
        if (one_sequence_consecutive && prompt_attention_) ESP_HIP_TRY(launch_attention_prompt(aa, rows, kv16, s));
        else ESP_HIP_TRY(launch_attention(aa, rows, kv16, s));
        g.w = L.wo; g.x = ctx_; g.y = hidden_; g.residual = hidden_;
        { int rc = project_and_norm(L.rms_ffn); if (rc != ESP_OK) return rc; }
        g.w = L.w13; g.x = xn_; g.y = gu_; g.residual = nullptr; g.swiglu_out = act_;   // SwiGLU in the GEMM's epilogue where it can be
        ESP_HIP_TRY(launch_gemm(g, s));
        g.swiglu_out = nullptr;
        g.w = L.w2; g.x = act_; g.y = hidden_; g.residual = hidden_;
        { int rc = project_and_norm(li + 1 < layers_.size() ? layers_[li + 1].rms_att : nullptr); if (rc != ESP_OK) return rc; }
    }
    (void)ad;
    return ESP_OK;
}

int LlamaRuntime::run_head(const float *hidden_rows, int count, bool want_logits) {
    hipStream_t s = context().stream;
    if (count <= 2 && !want_logits && head_fuses_argmax()) {
        // final RMSNorm in the staging, first-max arg-max in the epilogue: no logits are written (:8219-8275)
        GemvParams g;
        int blocks = 0;
        g.w = lm_head_; g.norm_x = hidden_rows; g.norm_w = final_norm_; g.norm_eps = c_.norm_eps; g.batch = count; g.epilogue = EPI_ARGMAX;
        g.argmax_value = argmax_scratch_.part_value; g.argmax_index = argmax_scratch_.part_index; g.argmax_capacity = head_partial_capacity_;
        g.argmax_blocks = &blocks;
        int rc;
        if ((rc = time_begin(K_HEAD)) != ESP_OK) return rc;
        ESP_HIP_TRY(launch_gemv(g, s));
        if ((rc = time_end()) != ESP_OK) return rc;
        ESP_HIP_TRY(launch_argmax_final(argmax_scratch_, blocks, count, d_out_tokens_, s));
        return ESP_OK;
    }
    if (count > 2 && matrix_prefill_ && lm_head_.format != FMT_F32 && lm_head_.cols % 64 == 0) {
        // batched rows: final RMSNorm, then the head as one MFMA GEMM
        ESP_HIP_TRY(launch_rmsnorm(hidden_rows, final_norm_, c_.norm_eps, count, c_.d_model, xn_, nullptr, s));
        GemmParams m;
        m.w = lm_head_; m.x = xn_; m.y = logits_; m.rows = count; m.workspace = gemm_workspace_; m.workspace_floats = kGemmWorkspaceFloats;
        ESP_HIP_TRY(launch_gemm(m, s));
        ESP_HIP_TRY(launch_argmax(logits_, count, c_.vocab, d_out_tokens_, nullptr, argmax_scratch_, s));
        return ESP_OK;
    }
    GemvParams g;   // final RMSNorm fused into the head GEMV's staging
    g.w = lm_head_; g.norm_x = hidden_rows; g.norm_w = final_norm_; g.norm_eps = c_.norm_eps;
    g.y = logits_; g.batch = count; g.epilogue = EPI_STORE_F32;
    int rc;
    if ((rc = time_begin(K_HEAD)) != ESP_OK) return rc;
    ESP_HIP_TRY(launch_gemv(g, s));
    if ((rc = time_end()) != ESP_OK) return rc;
    ESP_HIP_TRY(launch_argmax(logits_, count, c_.vocab, d_out_tokens_, nullptr, argmax_scratch_, s));
    return ESP_OK;
}

int LlamaRuntime::select_greedy(int seq, uint32_t *token) {
    if (!finalized_) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    if (seq < 0 || seq >= c_.max_sequences || !token) return fail(ESP_ERR_OUT_OF_RANGE, "select_greedy(seq %d)", seq);
    int rc = run_head(last_hidden_ + (size_t)seq * c_.d_model, 1);
    if (rc != ESP_OK) return rc;
    int t = 0;
    ESP_HIP_TRY(hipMemcpyAsync(&t, d_out_tokens_, sizeof(int), hipMemcpyDeviceToHost, context().stream));
    ESP_HIP_TRY(hipStreamSynchronize(context().stream));
    *token = (uint32_t)t;
    return ESP_OK;
}

int LlamaRuntime::head_rows(int count, uint32_t *tokens) {
    if (!finalized_) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    if (count < 1 || count > kMaxStepRows || !tokens) return fail(ESP_ERR_INVALID_ARGUMENT, "head_rows(%d)", count);
    int rc = run_head(hidden_, count);
    if (rc != ESP_OK) return rc;
    int t[kMaxStepRows];
    ESP_HIP_TRY(hipMemcpyAsync(t, d_out_tokens_, sizeof(int) * count, hipMemcpyDeviceToHost, context().stream));
    ESP_HIP_TRY(hipStreamSynchronize(context().stream));
    for (int i = 0; i < count; i++) tokens[i] = (uint32_t)t[i];
    return ESP_OK;
}

// head(last hidden of seq) -> argmax -> feed row 0 -> trunk -> keep row 0, captured once per sequence.
// Both step graphs of a sequence, at its first replayed step (a one-off of a few milliseconds per runtime, outside any later call).
int LlamaRuntime::capture_step_graph(int seq) {
    const int rc = capture_steps(seq, 1, &step_graphs_[seq]);
    return rc != ESP_OK ? rc : capture_steps(seq, kStepsPerGraph, &multi_graphs_[seq]);
}

// Replays `steps` greedy steps: graphs of kStepsPerGraph steps while that many are left, single steps for the rest.  Every boundary between two graph launches costs about 3.5 us on the device, whatever the graphs hold
// (6-layer model: 8.1 k tok/s with one step per graph, 8.35 k with four, 8.45 k with sixteen; 8B: 736 / 738.5 / 738.5).
int LlamaRuntime::replay_steps(int seq, int steps) {
    hipStream_t s = context().stream;
    int i = 0;
    if (multi_graphs_[seq])
        for (; i + kStepsPerGraph <= steps; i += kStepsPerGraph) ESP_HIP_TRY(hipGraphLaunch(multi_graphs_[seq], s));
    for (; i < steps; i++) ESP_HIP_TRY(hipGraphLaunch(step_graphs_[seq], s));
    return ESP_OK;
}

int LlamaRuntime::capture_steps(int seq, int count, hipGraphExec_t *out) {
    hipStream_t s = context().stream;
    hipGraph_t graph = nullptr;
    ESP_HIP_TRY(hipStreamSynchronize(s));
    ESP_HIP_TRY(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    int rc = ESP_OK;
    float *kept = last_hidden_ + (size_t)seq * c_.d_model;
    for (int step = 0; step < count && rc == ESP_OK; step++) {
        // head GEMV with the arg-max in its epilogue, then one launch that picks the token among the workgroups' candidates,
        // feeds it and fetches its embedding; the last layer writes the new hidden state where the next step's head reads
        // it: 2 + 5 per layer launches (3 + 5 per layer when the head has to store its logits)
        GemvParams g;
        g.w = lm_head_; g.norm_x = kept; g.norm_w = final_norm_; g.norm_eps = c_.norm_eps; g.batch = 1;
        hipError_t e;
        if (head_fuses_argmax()) {
            int blocks = 0;
            g.epilogue = EPI_ARGMAX;
            g.argmax_value = argmax_scratch_.part_value; g.argmax_index = argmax_scratch_.part_index; g.argmax_capacity = head_partial_capacity_;
            g.argmax_blocks = &blocks;
            e = launch_gemv(g, s);
            if (e == hipSuccess)
                e = launch_greedy_tail(argmax_scratch_, blocks, d_out_tokens_, seq, d_visible_, d_tokens_, d_pos_, d_seq_, d_log_, d_log_count_,
                                       c_.max_seq, embedding_, embedding_f16_, c_.d_model, hidden_, c_.eos_token, s);
        } else {
            g.y = logits_; g.epilogue = EPI_STORE_F32;
            e = launch_gemv(g, s);
            if (e == hipSuccess)
                e = launch_greedy_step_tail(logits_, c_.vocab, d_out_tokens_, argmax_scratch_, seq, d_visible_, d_tokens_, d_pos_, d_seq_, d_log_,
                                            d_log_count_, c_.max_seq, embedding_, embedding_f16_, c_.d_model, hidden_, c_.eos_token, s);
        }
        if (e != hipSuccess) rc = fail_hip(e, "greedy step head");
        if (rc == ESP_OK) rc = enqueue_trunk(1, true, kept);
    }
    hipError_t e = hipStreamEndCapture(s, &graph);
    if (rc != ESP_OK) { if (graph) (void)hipGraphDestroy(graph); return rc; }
    if (e != hipSuccess) return fail_hip(e, "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return fail_hip(e, "hipGraphInstantiate");
    *out = exec;
    return ESP_OK;
}

int LlamaRuntime::continue_greedy(int seq, int steps, uint32_t *out_tokens) {
    if (!finalized_) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    sync_tuning();
    if (seq < 0 || seq >= c_.max_sequences) return fail(ESP_ERR_OUT_OF_RANGE, "sequence %d of %d", seq, c_.max_sequences);
    if (steps < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "steps must be >= 0");
    if (visible_[seq] + steps > c_.max_seq)
        return fail(ESP_ERR_OUT_OF_RANGE, "runtime position %d + %d steps exceeds context %d", visible_[seq], steps, c_.max_seq);
    if (steps == 0) return ESP_OK;
    hipStream_t s = context().stream;
    int rc;
    if (!use_graph_ || timing_enabled_) {
        for (int i = 0; i < steps; i++) {
            uint32_t t = 0;
            if ((rc = select_greedy(seq, &t)) != ESP_OK) return rc;
            if (out_tokens) out_tokens[i] = t;
            if ((rc = advance(seq, t)) != ESP_OK) return rc;
        }
        return ESP_OK;
    }
    if (!step_graphs_[seq]) {
        // one eager step first: it configures every kernel's LDS limit outside the capture
        uint32_t t = 0;
        if ((rc = select_greedy(seq, &t)) != ESP_OK) return rc;
        if (out_tokens) out_tokens[0] = t;
        if ((rc = advance(seq, t)) != ESP_OK) return rc;
        if ((rc = capture_step_graph(seq)) != ESP_OK) return rc;
        if (out_tokens) out_tokens += 1;
        steps -= 1;
        if (steps == 0) return ESP_OK;
    }
    ESP_HIP_TRY(launch_set_ints(d_visible_ + seq, visible_[seq], d_log_count_, 0, s));
    ESP_HIP_TRY(launch_set_ints(d_log_count_ + 1, 0, d_log_count_ + 2, 0, s));   // not stopped, and no stop at the stop token
    if ((rc = replay_steps(seq, steps)) != ESP_OK) return rc;
    std::vector<int> log(steps);
    ESP_HIP_TRY(hipMemcpyAsync(log.data(), d_log_, sizeof(int) * steps, hipMemcpyDeviceToHost, s));
    ESP_HIP_TRY(hipStreamSynchronize(s));
    visible_[seq] += steps;
    if (out_tokens) for (int i = 0; i < steps; i++) out_tokens[i] = (uint32_t)log[i];
    return ESP_OK;
}

// continue_greedy that ends with the stop token: the token is emitted and not consumed, as in the reference loop (:6385-6388).  The
// replays run in chunks; the step graph itself notices the stop token, and replays after it change nothing.
int LlamaRuntime::continue_greedy_until_stop(int seq, int steps, uint32_t *out_tokens, int *produced) {
    if (!finalized_) return fail(ESP_ERR_INVALID_ARGUMENT, "runtime is not finalized");
    if (seq < 0 || seq >= c_.max_sequences || !out_tokens || !produced) return fail(ESP_ERR_OUT_OF_RANGE, "continue_greedy_until_stop(seq %d)", seq);
    *produced = 0;
    sync_tuning();
    if (steps < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "steps must be >= 0");
    if (visible_[seq] + steps > c_.max_seq)
        return fail(ESP_ERR_OUT_OF_RANGE, "runtime position %d + %d steps exceeds context %d", visible_[seq], steps, c_.max_seq);
    const int eos = c_.eos_token;
    hipStream_t s = context().stream;
    int rc;
    auto eager_step = [&](bool *stopped) {
        uint32_t t = 0;
        int r = select_greedy(seq, &t);
        if (r != ESP_OK) return r;
        out_tokens[(*produced)++] = t;
        *stopped = eos >= 0 && t == (uint32_t)eos;
        return *stopped ? ESP_OK : advance(seq, t);
    };
    bool stopped = false;
    if (!use_graph_ || timing_enabled_) {
        while (*produced < steps && !stopped)
            if ((rc = eager_step(&stopped)) != ESP_OK) return rc;
        return ESP_OK;
    }
    if (steps > 0) {
        // The first step always runs from the host.  A replay that finds the stop token re-embeds the row that sits in
        // d_tokens_/d_pos_/d_seq_[0] and lets the trunk recompute it, which changes nothing only when that row is the one this
        // sequence consumed last; after a prompt block or another sequence's pass those arrays hold something else.  advance()
        // leaves exactly that row there (and the eager step configures every kernel's LDS limit outside a capture).
        if ((rc = eager_step(&stopped)) != ESP_OK) return rc;
        if (stopped) return ESP_OK;
        if (!step_graphs_[seq] && (rc = capture_step_graph(seq)) != ESP_OK) return rc;
    }
    if (*produced >= steps) return ESP_OK;
    const int first = *produced, want = steps - first;
    ESP_HIP_TRY(launch_set_ints(d_visible_ + seq, visible_[seq], d_log_count_, 0, s));
    ESP_HIP_TRY(launch_set_ints(d_log_count_ + 1, 0, d_log_count_ + 2, 1, s));
    int state[2] = {0, 0};   // tokens logged, stopped
    for (int launched = 0; launched < want && !state[1];) {
        const int chunk = want - launched < 32 ? want - launched : 32;
        if ((rc = replay_steps(seq, chunk)) != ESP_OK) return rc;
        launched += chunk;
        ESP_HIP_TRY(hipMemcpyAsync(state, d_log_count_, sizeof(state), hipMemcpyDeviceToHost, s));
        ESP_HIP_TRY(hipStreamSynchronize(s));
    }
    const int logged = state[0] < want ? state[0] : want;
    std::vector<int> log(logged > 0 ? logged : 1);
    if (logged > 0) {
        ESP_HIP_TRY(hipMemcpyAsync(log.data(), d_log_, sizeof(int) * logged, hipMemcpyDeviceToHost, s));
        ESP_HIP_TRY(hipStreamSynchronize(s));
    }
    for (int i = 0; i < logged; i++) out_tokens[first + i] = (uint32_t)log[i];
    *produced = first + logged;
    visible_[seq] += logged - (state[1] ? 1 : 0);   // every logged token was consumed, except a stop token
    return ESP_OK;
}

int LlamaRuntime::read_last_hidden(int seq, float *out) {
    if (!finalized_ || seq < 0 || seq >= c_.max_sequences || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "read_last_hidden");
    ESP_HIP_TRY(hipMemcpyAsync(out, last_hidden_ + (size_t)seq * c_.d_model, (size_t)c_.d_model * 4, hipMemcpyDeviceToHost,
                               context().stream));
    ESP_HIP_TRY(hipStreamSynchronize(context().stream));
    return ESP_OK;
}

int LlamaRuntime::read_logits(int seq, float *out) {
    if (!finalized_ || seq < 0 || seq >= c_.max_sequences || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "read_logits");
    int rc = run_head(last_hidden_ + (size_t)seq * c_.d_model, 1, true);
    if (rc != ESP_OK) return rc;
    ESP_HIP_TRY(hipMemcpyAsync(out, logits_, (size_t)c_.vocab * 4, hipMemcpyDeviceToHost, context().stream));
    ESP_HIP_TRY(hipStreamSynchronize(context().stream));
    return ESP_OK;
}

}  // namespace esp
