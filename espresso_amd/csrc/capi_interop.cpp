// C ABI: kernel handles and surfaces in the call shape of the reference's ANEInterop module
// (Sources/ANEInterop/include/ane_interop.h).  See the header for the contract of every function.
#include <atomic>
#include <cmath>
#include <cstring>
#include <initializer_list>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "context.h"
#include "host/model_support.h"
#include "kernels/decode_ops.h"
#include "kernels/surface_ops.h"

using namespace esp;

// A surface: HBM buffer + host shadow; `host_valid` / `device_valid` say which copy is current.
struct ESPSurface {
    std::atomic<int> refs{1};
    size_t bytes = 0;
    std::vector<uint8_t> host;
    uint8_t *device = nullptr;
    bool host_valid = true, device_valid = false;
    int write_locks = 0, read_locks = 0;
};

namespace {

std::atomic<int> g_compile_count{0}, g_live_handles{0};
std::atomic<int> g_last_compile_error{ESP_INTEROP_COMPILE_ERROR_NONE};
std::atomic<bool> g_force_eval_failure{false};

bool surface_to_host(ESPSurface *s) {
    if (s->host_valid) return true;
    if (!s->device) return false;
    if (hipMemcpy(s->host.data(), s->device, s->bytes, hipMemcpyDeviceToHost) != hipSuccess) return false;
    s->host_valid = true;
    return true;
}

bool surface_to_device(ESPSurface *s) {
    if (ensure_init() != ESP_OK) return false;
    if (!s->device) {
        void *p = nullptr;
        if (hipMalloc(&p, s->bytes ? s->bytes : 16) != hipSuccess) return false;
        s->device = static_cast<uint8_t *>(p);
        s->device_valid = false;
    }
    if (s->device_valid) return true;
    if (!s->host_valid) return false;
    if (hipMemcpy(s->device, s->host.data(), s->bytes, hipMemcpyHostToDevice) != hipSuccess) return false;
    s->device_valid = true;
    return true;
}

// fp16 view of the shadow for reading / writing [channels, spatial] regions
uint16_t *shadow_for_write(ESPSurface *s) {
    if (!s || !surface_to_host(s)) return nullptr;
    s->device_valid = false;
    return reinterpret_cast<uint16_t *>(s->host.data());
}
const uint16_t *shadow_for_read(ESPSurface *s) {
    if (!s || !surface_to_host(s)) return nullptr;
    return reinterpret_cast<const uint16_t *>(s->host.data());
}
bool region_ok(const ESPSurface *s, int ch_off, int channels, int spatial) {
    if (!s || ch_off < 0 || channels < 0 || spatial <= 0) return false;
    return ((size_t)ch_off + (size_t)channels) * (size_t)spatial * 2 <= s->bytes;
}
bool slice_ok(const ESPSurface *s, int ch_off, int channels, int spatial, int index) {
    return region_ok(s, ch_off, channels, spatial) && index >= 0 && index < spatial;
}

enum KernelKind { KIND_GEMV, KIND_CLASSIFIER, KIND_FFN, KIND_QKV, KIND_PROJECTION };

std::string trim(const std::string &s) {
    size_t a = s.find_first_not_of(" \t\r"), b = s.find_last_not_of(" \t\r");
    return a == std::string::npos ? "" : s.substr(a, b - a + 1);
}

// "key: value" pairs; several pairs may share a line
std::map<std::string, std::string> parse_program(const std::string &text) {
    std::map<std::string, std::string> kv;
    std::stringstream lines(text);
    std::string line;
    while (std::getline(lines, line)) {
        std::stringstream words(line);
        std::string tok, key;
        while (words >> tok) {
            if (!tok.empty() && tok.back() == ':') key = tok.substr(0, tok.size() - 1);
            else if (!key.empty()) { kv[key] = trim(tok); key.clear(); }
        }
    }
    return kv;
}

int format_by_name(const std::string &n) {
    if (n == "f32") return FMT_F32;
    if (n == "f16") return FMT_F16;
    if (n == "q4_0") return FMT_Q4_0;
    if (n == "q8_0") return FMT_Q8_0;
    if (n == "q4_k") return FMT_Q4_K;
    return -1;
}

std::string weight_stem(const char *path) {
    std::string p = path ? path : "";
    size_t slash = p.find_last_of('/');
    if (slash != std::string::npos) p = p.substr(slash + 1);
    if (p.size() > 4 && p.compare(p.size() - 4, 4, ".bin") == 0) p = p.substr(0, p.size() - 4);
    return p;
}

struct WeightBytes { const uint8_t *data; size_t len; };

// fp16 payload of a BLOBFILE, or the bytes themselves when they carry no BLOBFILE header
WeightBytes payload_of(WeightBytes w) {
    BlobWeightLoader::Header h;
    if (w.len >= 128 && BlobWeightLoader::parseHeader(w.data, w.len, &h) == BlobWeightLoaderError::none && 128 + (size_t)h.dataSize == w.len)
        return {w.data + 128, (size_t)h.dataSize};
    return w;
}

}  // namespace

struct ESPHandle {
    int kind = KIND_GEMV;
    int lanes = 1, spatial = 1, rows = 0, cols = 0, dim = 0, hidden = 0, vocab = 0, q_dim = 0, kv_dim = 0;
    float norm_eps = 1e-5f;
    DeviceMatrix w, w13, w2, classifier;
    float *norm = nullptr;
    std::vector<ESPSurface *> inputs, outputs;
    // scratch
    uint16_t *x16 = nullptr, *act16 = nullptr;
    float *x32 = nullptr, *y32 = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    uint64_t last_ns = 0;
};

namespace {

void destroy_handle(ESPHandle *h) {
    if (!h) return;
    matrix_release(&h->w); matrix_release(&h->w13); matrix_release(&h->w2); matrix_release(&h->classifier);
    if (h->norm) (void)hipFree(h->norm);
    if (h->x16) (void)hipFree(h->x16);
    if (h->act16) (void)hipFree(h->act16);
    if (h->x32) (void)hipFree(h->x32);
    if (h->y32) (void)hipFree(h->y32);
    if (h->ev0) (void)hipEventDestroy(h->ev0);
    if (h->ev1) (void)hipEventDestroy(h->ev1);
    for (ESPSurface *s : h->inputs) esp_surface_release(s);
    for (ESPSurface *s : h->outputs) esp_surface_release(s);
    delete h;
}

ESPHandle *compile_fail(ESPHandle *h, int code, const char *fmt, const char *arg = "") {
    g_last_compile_error = code;
    fail(ESP_ERR_INVALID_ARGUMENT, fmt, arg);
    destroy_handle(h);
    return nullptr;
}

int upload_norm(WeightBytes raw, int count, float **out) {
    WeightBytes p = payload_of(raw);
    if (p.len != (size_t)count * 2) return fail(ESP_ERR_INVALID_ARGUMENT, "norm weight holds %zu bytes, expected %d fp16 values", p.len, count);
    std::vector<float> v(count);
    for (int i = 0; i < count; i++) v[i] = half_to_float((uint16_t)(p.data[2 * i] | (p.data[2 * i + 1] << 8)));
    int rc = device_alloc(out, (size_t)count);
    if (rc != ESP_OK) return rc;
    ESP_HIP_TRY(hipMemcpy(*out, v.data(), (size_t)count * 4, hipMemcpyHostToDevice));
    return ESP_OK;
}

int upload_matrix(WeightBytes raw, int format, int rows, int cols, DeviceMatrix *out) {
    WeightBytes p = format == FMT_F16 ? payload_of(raw) : raw;
    const size_t want = format_bytes(format, (size_t)rows * cols);
    if (p.len != want) return fail(ESP_ERR_INVALID_ARGUMENT, "weight matrix holds %zu bytes, format needs %zu for %dx%d", p.len, want, rows, cols);
    return matrix_upload(format, p.data, rows, cols, out);
}

}  // namespace

extern "C" {

void esp_interop_init(void) { (void)ensure_init(); }

ESPSurfaceRef esp_interop_create_surface(size_t bytes) {
    ESPSurface *s = new ESPSurface();
    s->bytes = bytes;
    s->host.assign(bytes, 0);
    return s;
}

ESPSurfaceRef esp_surface_retain(ESPSurfaceRef s) {
    if (s) s->refs.fetch_add(1);
    return s;
}

void esp_surface_release(ESPSurfaceRef s) {
    if (!s) return;
    if (s->refs.fetch_sub(1) == 1) {
        if (s->device) (void)hipFree(s->device);
        delete s;
    }
}

size_t esp_surface_bytes(ESPSurfaceRef s) { return s ? s->bytes : 0; }

ESPHandle *esp_interop_compile(const uint8_t *program, size_t program_len, const char **weight_paths,
                               const uint8_t **weight_datas, const size_t *weight_lens, int weight_count,
                               int n_inputs, const size_t *input_sizes, int n_outputs, const size_t *output_sizes) {
    g_last_compile_error = ESP_INTEROP_COMPILE_ERROR_NONE;
    if (!program || program_len == 0 || weight_count < 0 || n_inputs < 0 || n_outputs < 0 ||
        (weight_count > 0 && (!weight_paths || !weight_datas || !weight_lens)) || (n_inputs > 0 && !input_sizes) ||
        (n_outputs > 0 && !output_sizes))
        return compile_fail(nullptr, ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS, "compile: invalid arguments%s");
    std::map<std::string, WeightBytes> weights;
    for (int i = 0; i < weight_count; i++) {
        if (!weight_paths[i]) return compile_fail(nullptr, ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS, "compile: null weight path%s");
        // a weight path never leaves the model directory (ane_interop.m rejects ".." components)
        const std::string raw_path = weight_paths[i];
        if (raw_path == ".." || raw_path.rfind("../", 0) == 0 || raw_path.find("/../") != std::string::npos ||
            (raw_path.size() >= 3 && raw_path.compare(raw_path.size() - 3, 3, "/..") == 0))
            return compile_fail(nullptr, ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS, "compile: weight path %s leaves the model directory", weight_paths[i]);
        const std::string stem = weight_stem(weight_paths[i]);
        if (weights.count(stem)) return compile_fail(nullptr, ESP_INTEROP_COMPILE_ERROR_DUPLICATE_WEIGHT_PATH, "compile: duplicate weight path %s", weight_paths[i]);
        weights[stem] = {weight_datas[i], weight_datas[i] ? weight_lens[i] : 0};
    }
    if (ensure_init() != ESP_OK) { g_last_compile_error = ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE; return nullptr; }

    const auto kv = parse_program(std::string(reinterpret_cast<const char *>(program), program_len));
    auto get_int = [&](const char *k, int dflt) { auto it = kv.find(k); return it == kv.end() ? dflt : std::atoi(it->second.c_str()); };
    auto get_str = [&](const char *k) { auto it = kv.find(k); return it == kv.end() ? std::string() : it->second; };
    ESPHandle *h = new ESPHandle();
    const std::string kind = get_str("kernel");
    const int format = format_by_name(get_str("format"));
    h->spatial = get_int("spatial", 1);
    h->lanes = get_int("lanes", 1);
    if (!get_str("norm_eps").empty()) h->norm_eps = (float)std::atof(get_str("norm_eps").c_str());
    if (get_str("program") != "espresso.hip/1") return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: program header must be espresso.hip/1%s");
    if (h->spatial < 1 || h->lanes < 1 || h->lanes > 16 || h->lanes > h->spatial)
        return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: spatial/lanes out of range%s");
    auto need = [&](const char *name) -> WeightBytes * { auto it = weights.find(name); return it == weights.end() || !it->second.data ? nullptr : &it->second; };
    std::vector<size_t> want_in, want_out;
    int rc = ESP_OK;
    if (kind == "gemv") {
        h->kind = KIND_GEMV;
        h->rows = get_int("rows", 0); h->cols = get_int("cols", 0);
        WeightBytes *w = need("w");
        if (format < 0 || h->rows <= 0 || h->cols <= 0 || !w) return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: gemv needs format, rows, cols and weight w%s");
        rc = upload_matrix(*w, format, h->rows, h->cols, &h->w);
        want_in = {(size_t)h->cols * h->spatial * 2};
        want_out = {(size_t)h->rows * h->spatial * 2};
    } else if (kind == "rmsnorm_classifier") {
        h->kind = KIND_CLASSIFIER;
        h->dim = get_int("dim", 0); h->vocab = get_int("vocab", 0);
        WeightBytes *g = need("rms_final"), *c = need("classifier");
        if (format < 0 || h->dim <= 0 || h->vocab <= 0 || !g || !c) return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: rmsnorm_classifier needs format, dim, vocab, rms_final and classifier%s");
        rc = upload_norm(*g, h->dim, &h->norm);
        if (rc == ESP_OK) rc = upload_matrix(*c, format, h->vocab, h->dim, &h->classifier);
        want_in = {(size_t)h->dim * h->spatial * 2};
        want_out = {(size_t)h->vocab * h->spatial * 2, (size_t)h->spatial * 2};
        h->rows = h->vocab; h->cols = h->dim;
    } else if (kind == "decode_ffn") {
        h->kind = KIND_FFN;
        h->dim = get_int("dim", 0); h->hidden = get_int("hidden", 0);
        WeightBytes *g = need("rms_ffn"), *w1 = need("w1"), *w3 = need("w3"), *w2 = need("w2");
        if (format < 0 || h->dim <= 0 || h->hidden <= 0 || !g || !w1 || !w3 || !w2) return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: decode_ffn needs format, dim, hidden, rms_ffn, w1, w3 and w2%s");
        rc = upload_norm(*g, h->dim, &h->norm);
        const size_t rb = format_bytes(format, (size_t)h->dim);
        if (rc == ESP_OK && (w1->len != rb * h->hidden || w3->len != rb * h->hidden) && format != FMT_F16)
            rc = fail(ESP_ERR_INVALID_ARGUMENT, "w1/w3 byte counts do not match %dx%d", h->hidden, h->dim);
        if (rc == ESP_OK) {
            // gate and up rows interleaved (g0, u0, g1, u1, ...) so that one GEMV feeds the SwiGLU epilogue
            WeightBytes p1 = format == FMT_F16 ? payload_of(*w1) : *w1, p3 = format == FMT_F16 ? payload_of(*w3) : *w3;
            if (p1.len != rb * h->hidden || p3.len != rb * h->hidden) rc = fail(ESP_ERR_INVALID_ARGUMENT, "w1/w3 byte counts do not match %dx%d", h->hidden, h->dim);
            else {
                std::vector<uint8_t> fused(2 * rb * h->hidden);
                for (int i = 0; i < h->hidden; i++) {
                    std::memcpy(&fused[(size_t)(2 * i) * rb], p1.data + (size_t)i * rb, rb);
                    std::memcpy(&fused[(size_t)(2 * i + 1) * rb], p3.data + (size_t)i * rb, rb);
                }
                rc = matrix_upload(format, fused.data(), 2 * h->hidden, h->dim, &h->w13);
            }
        }
        if (rc == ESP_OK) rc = upload_matrix(*w2, format, h->dim, h->hidden, &h->w2);
        want_in = {(size_t)h->dim * h->spatial * 2};
        want_out = {(size_t)h->dim * h->spatial * 2};
        h->rows = h->dim; h->cols = h->dim;
    } else if (kind == "decode_qkv") {
        // decodeQKVOnly (DecodeAttentionQKVGenerator.swift:86-131; outputs k @ 0, q @ 1, v @ 2, DecodeForwardPass.swift:374-377):
        // rmsnorm, then the three projections; RoPE, the KV-cache update and attention are separate calls, as in the reference
        h->kind = KIND_QKV;
        h->dim = get_int("dim", 0); h->q_dim = get_int("q_dim", h->dim); h->kv_dim = get_int("kv_dim", h->dim);
        WeightBytes *g = need("rms_att"), *wq = need("wq"), *wk = need("wk"), *wv = need("wv");
        if (format < 0 || h->dim <= 0 || h->q_dim <= 0 || h->kv_dim <= 0 || !g || !wq || !wk || !wv)
            return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: decode_qkv needs format, dim, rms_att, wq, wk and wv%s");
        rc = upload_norm(*g, h->dim, &h->norm);
        if (rc == ESP_OK) {
            const size_t rb = format_bytes(format, (size_t)h->dim);
            WeightBytes pq = format == FMT_F16 ? payload_of(*wq) : *wq, pk = format == FMT_F16 ? payload_of(*wk) : *wk, pv = format == FMT_F16 ? payload_of(*wv) : *wv;
            if (pq.len != rb * h->q_dim || pk.len != rb * h->kv_dim || pv.len != rb * h->kv_dim) rc = fail(ESP_ERR_INVALID_ARGUMENT, "wq/wk/wv byte counts do not match their shapes");
            else {
                std::vector<uint8_t> fused(rb * (size_t)(h->q_dim + 2 * h->kv_dim));   // rows: q, then k, then v
                std::memcpy(fused.data(), pq.data, pq.len);
                std::memcpy(fused.data() + pq.len, pk.data, pk.len);
                std::memcpy(fused.data() + pq.len + pk.len, pv.data, pv.len);
                rc = matrix_upload(format, fused.data(), h->q_dim + 2 * h->kv_dim, h->dim, &h->w);
            }
        }
        want_in = {(size_t)h->dim * h->spatial * 2};
        want_out = {(size_t)h->kv_dim * h->spatial * 2, (size_t)h->q_dim * h->spatial * 2, (size_t)h->kv_dim * h->spatial * 2};
        h->rows = h->q_dim + 2 * h->kv_dim; h->cols = h->dim;
    } else if (kind == "decode_projection") {
        // decodeProjection: out = residual + Wo * context; input 0 = the attention context, input 1 = the residual, which the
        // reference rebinds to the layer's input surface (DecodeForwardPass.swift:383,396)
        h->kind = KIND_PROJECTION;
        h->dim = get_int("dim", 0); h->q_dim = get_int("q_dim", h->dim);
        WeightBytes *wo = need("wo");
        if (format < 0 || h->dim <= 0 || h->q_dim <= 0 || !wo)
            return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: decode_projection needs format, dim and wo%s");
        rc = upload_matrix(*wo, format, h->dim, h->q_dim, &h->w);
        want_in = {(size_t)h->q_dim * h->spatial * 2, (size_t)h->dim * h->spatial * 2};
        want_out = {(size_t)h->dim * h->spatial * 2};
        h->rows = h->dim; h->cols = h->q_dim;
    } else {
        return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE, "compile: unknown kernel kind %s", kind.c_str());
    }
    if (rc != ESP_OK) { g_last_compile_error = ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE; destroy_handle(h); return nullptr; }
    if ((size_t)n_inputs != want_in.size() || (size_t)n_outputs != want_out.size())
        return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS, "compile: surface counts do not match the kernel%s");
    for (size_t i = 0; i < want_in.size(); i++)
        if (input_sizes[i] != want_in[i]) return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS, "compile: input surface size does not match channels x spatial x 2%s");
    for (size_t i = 0; i < want_out.size(); i++)
        if (output_sizes[i] != want_out[i]) return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS, "compile: output surface size does not match channels x spatial x 2%s");
    for (size_t b : want_in) h->inputs.push_back(esp_interop_create_surface(b));
    for (size_t b : want_out) h->outputs.push_back(esp_interop_create_surface(b));
    const size_t widest = (size_t)std::max(std::max(std::max(h->rows, h->cols), std::max(h->hidden, h->vocab)), std::max(h->dim, h->q_dim));
    bool ok = device_alloc(&h->x16, (size_t)h->lanes * widest) == ESP_OK && device_alloc(&h->act16, (size_t)h->lanes * widest) == ESP_OK &&
              device_alloc(&h->x32, (size_t)h->lanes * widest) == ESP_OK && device_alloc(&h->y32, (size_t)h->lanes * widest) == ESP_OK &&
              hipEventCreate(&h->ev0) == hipSuccess && hipEventCreate(&h->ev1) == hipSuccess;
    for (ESPSurface *s : h->inputs) ok = ok && surface_to_device(s);
    for (ESPSurface *s : h->outputs) ok = ok && surface_to_device(s);
    if (!ok) return compile_fail(h, ESP_INTEROP_COMPILE_ERROR_SURFACE_ALLOCATION_FAILED, "compile: surface allocation failed%s");
    g_live_handles.fetch_add(1);
    g_compile_count.fetch_add(1);  // successful compiles only
    clear_error();
    return h;
}

bool esp_interop_eval(ESPHandle *h) {
    if (!h) return false;
    if (g_force_eval_failure.load()) { fail(ESP_ERR_FORCED_FAILURE, "eval failure forced by esp_interop_set_force_eval_failure"); return false; }
    hipStream_t s = context().stream;
    for (ESPSurface *in : h->inputs) if (!surface_to_device(in)) { fail(ESP_ERR_LAUNCH_FAILED, "eval: input surface upload failed"); return false; }
    for (ESPSurface *out : h->outputs) if (!surface_to_device(out)) { fail(ESP_ERR_LAUNCH_FAILED, "eval: output surface upload failed"); return false; }
    const uint16_t *in0 = reinterpret_cast<const uint16_t *>(h->inputs[0]->device);
    uint16_t *out0 = reinterpret_cast<uint16_t *>(h->outputs[0]->device);
    hipError_t e = hipEventRecord(h->ev0, s);
    GemvParams g;
    g.batch = h->lanes;
    if (e == hipSuccess && h->kind == KIND_GEMV) {
        e = launch_gather_columns(in0, h->cols, h->spatial, h->lanes, h->x16, nullptr, s);
        g.w = h->w; g.x = h->x16; g.y = h->y32; g.epilogue = EPI_STORE_F32;
        if (e == hipSuccess) e = launch_gemv(g, s);
        if (e == hipSuccess) e = launch_scatter_columns(h->y32, h->rows, h->spatial, h->lanes, out0, s);
    } else if (e == hipSuccess && h->kind == KIND_CLASSIFIER) {
        e = launch_gather_columns(in0, h->dim, h->spatial, h->lanes, nullptr, h->x32, s);
        // RMSNorm runs inside the GEMV's staging
        g.w = h->classifier; g.norm_x = h->x32; g.norm_w = h->norm; g.norm_eps = h->norm_eps; g.y = h->y32; g.epilogue = EPI_STORE_F32;
        if (e == hipSuccess) e = launch_gemv(g, s);
        if (e == hipSuccess) e = launch_scatter_columns(h->y32, h->vocab, h->spatial, h->lanes, out0, s);
        if (e == hipSuccess) e = launch_row_max(h->y32, h->vocab, h->spatial, h->lanes, reinterpret_cast<uint16_t *>(h->outputs[1]->device), s);
    } else if (e == hipSuccess && h->kind == KIND_QKV) {
        e = launch_gather_columns(in0, h->dim, h->spatial, h->lanes, nullptr, h->x32, s);
        g.w = h->w; g.norm_x = h->x32; g.norm_w = h->norm; g.norm_eps = h->norm_eps; g.y = h->y32; g.epilogue = EPI_STORE_F32;
        if (e == hipSuccess) e = launch_gemv(g, s);
        const int stride = h->q_dim + 2 * h->kv_dim;
        if (e == hipSuccess) e = launch_scatter_columns_strided(h->y32 + h->q_dim, stride, h->kv_dim, h->spatial, h->lanes, out0, s);                         // k @ 0
        if (e == hipSuccess) e = launch_scatter_columns_strided(h->y32, stride, h->q_dim, h->spatial, h->lanes, reinterpret_cast<uint16_t *>(h->outputs[1]->device), s);   // q @ 1
        if (e == hipSuccess) e = launch_scatter_columns_strided(h->y32 + h->q_dim + h->kv_dim, stride, h->kv_dim, h->spatial, h->lanes, reinterpret_cast<uint16_t *>(h->outputs[2]->device), s);   // v @ 2
    } else if (e == hipSuccess && h->kind == KIND_PROJECTION) {
        e = launch_gather_columns(in0, h->q_dim, h->spatial, h->lanes, h->x16, nullptr, s);
        if (e == hipSuccess) e = launch_gather_columns(reinterpret_cast<const uint16_t *>(h->inputs[1]->device), h->dim, h->spatial, h->lanes, nullptr, h->x32, s);
        g.w = h->w; g.x = h->x16; g.y = h->y32; g.residual = h->x32; g.epilogue = EPI_ADD_RESIDUAL;
        if (e == hipSuccess) e = launch_gemv(g, s);
        if (e == hipSuccess) e = launch_scatter_columns(h->y32, h->dim, h->spatial, h->lanes, out0, s);
    } else if (e == hipSuccess) {
        e = launch_gather_columns(in0, h->dim, h->spatial, h->lanes, nullptr, h->x32, s);
        g.w = h->w13; g.norm_x = h->x32; g.norm_w = h->norm; g.norm_eps = h->norm_eps; g.out_f16 = h->act16; g.epilogue = EPI_SWIGLU_F16;
        if (e == hipSuccess) e = launch_gemv(g, s);
        g.w = h->w2; g.x = h->act16; g.norm_x = nullptr; g.norm_w = nullptr; g.out_f16 = nullptr; g.y = h->y32; g.residual = h->x32; g.epilogue = EPI_ADD_RESIDUAL;
        if (e == hipSuccess) e = launch_gemv(g, s);
        if (e == hipSuccess) e = launch_scatter_columns(h->y32, h->dim, h->spatial, h->lanes, out0, s);
    }
    if (e == hipSuccess) e = hipEventRecord(h->ev1, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) { fail_hip(e, "eval"); return false; }
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, h->ev0, h->ev1) == hipSuccess) h->last_ns = (uint64_t)((double)ms * 1e6);
    for (ESPSurface *out : h->outputs) { out->device_valid = true; out->host_valid = false; }
    return true;
}

ESPSurfaceRef esp_interop_get_input(ESPHandle *h, int i) { return h && i >= 0 && i < (int)h->inputs.size() ? h->inputs[i] : nullptr; }
ESPSurfaceRef esp_interop_get_output(ESPHandle *h, int i) { return h && i >= 0 && i < (int)h->outputs.size() ? h->outputs[i] : nullptr; }
ESPSurfaceRef esp_interop_copy_input(ESPHandle *h, int i) { return esp_surface_retain(esp_interop_get_input(h, i)); }
ESPSurfaceRef esp_interop_copy_output(ESPHandle *h, int i) { return esp_surface_retain(esp_interop_get_output(h, i)); }

void esp_interop_free(ESPHandle *h) {
    if (!h) return;
    g_live_handles.fetch_sub(1);
    destroy_handle(h);
}

int esp_interop_compile_count(void) { return g_compile_count.load(); }
void esp_interop_set_compile_count(int v) { g_compile_count = v; }
int esp_interop_last_compile_error(void) { return g_last_compile_error.load(); }
void esp_interop_set_force_eval_failure(bool v) { g_force_eval_failure = v; }
int esp_interop_live_handle_count(void) { return g_live_handles.load(); }
uint64_t esp_interop_last_hw_execution_time_ns(ESPHandle *h) { return h ? h->last_ns : 0; }
bool esp_interop_has_perf_stats(ESPHandle *h) { return h != nullptr; }

bool esp_interop_rebind_input(ESPHandle *h, int index, ESPSurfaceRef s) {
    if (!h || !s || index < 0 || index >= (int)h->inputs.size() || s->bytes != h->inputs[index]->bytes) return false;
    esp_surface_retain(s);
    esp_surface_release(h->inputs[index]);
    h->inputs[index] = s;
    return true;
}

void esp_interop_cvt_f32_to_f16(void *dst, const float *src, int count) {
    uint16_t *d = static_cast<uint16_t *>(dst);
    for (int i = 0; i < count; i++) d[i] = float_to_half_rne(src[i]);
}
void esp_interop_cvt_f16_to_f32(float *dst, const void *src, int count) {
    const uint16_t *s = static_cast<const uint16_t *>(src);
    for (int i = 0; i < count; i++) dst[i] = half_to_float(s[i]);
}
void esp_interop_argmax_f16_strided(const void *src, int count, int stride, int *out_index, float *out_value) {
    const uint16_t *s = static_cast<const uint16_t *>(src);
    int best = 0;
    float bv = count > 0 ? half_to_float(s[0]) : 0.0f;
    for (int i = 1; i < count; i++) {
        const float v = half_to_float(s[(size_t)i * stride]);
        if (v > bv) { bv = v; best = i; }
    }
    if (out_index) *out_index = best;
    if (out_value) *out_value = bv;
}
void esp_interop_argmax_f16(const void *src, int count, int *out_index, float *out_value) {
    esp_interop_argmax_f16_strided(src, count, 1, out_index, out_value);
}

bool esp_interop_io_copy(ESPSurfaceRef dst, int dst_ch_off, ESPSurfaceRef src, int src_ch_off, int channels, int spatial) {
    if (!region_ok(dst, dst_ch_off, channels, spatial) || !region_ok(src, src_ch_off, channels, spatial)) return false;
    const uint16_t *s = shadow_for_read(src);
    uint16_t *d = shadow_for_write(dst);
    if (!s || !d) return false;
    std::memmove(d + (size_t)dst_ch_off * spatial, s + (size_t)src_ch_off * spatial, (size_t)channels * spatial * 2);
    return true;
}

bool esp_interop_io_copy_fp16_spatial_slice(ESPSurfaceRef dst, int dst_ch_off, int dst_index, int dst_spatial, ESPSurfaceRef src,
                                            int src_ch_off, int src_index, int src_spatial, int channels) {
    if (!slice_ok(dst, dst_ch_off, channels, dst_spatial, dst_index) || !slice_ok(src, src_ch_off, channels, src_spatial, src_index)) return false;
    const uint16_t *s = shadow_for_read(src);
    uint16_t *d = shadow_for_write(dst);
    if (!s || !d) return false;
    for (int c = 0; c < channels; c++) d[(size_t)(dst_ch_off + c) * dst_spatial + dst_index] = s[(size_t)(src_ch_off + c) * src_spatial + src_index];
    return true;
}

bool esp_interop_io_write_fp16_spatial_slice(ESPSurfaceRef surface, int ch_off, int index, int spatial, const float *data, int channels) {
    if (!data || !slice_ok(surface, ch_off, channels, spatial, index)) return false;
    uint16_t *d = shadow_for_write(surface);
    if (!d) return false;
    for (int c = 0; c < channels; c++) d[(size_t)(ch_off + c) * spatial + index] = float_to_half_rne(data[c]);
    return true;
}

bool esp_interop_io_read_fp16_spatial_slice(ESPSurfaceRef surface, int ch_off, int index, int spatial, float *data, int channels) {
    if (!data || !slice_ok(surface, ch_off, channels, spatial, index)) return false;
    const uint16_t *s = shadow_for_read(surface);
    if (!s) return false;
    for (int c = 0; c < channels; c++) data[c] = half_to_float(s[(size_t)(ch_off + c) * spatial + index]);
    return true;
}

bool esp_interop_io_argmax_fp16_spatial_slice(ESPSurfaceRef surface, int ch_off, int index, int spatial, int channels, int *out_index,
                                              float *out_value) {
    if (channels <= 0 || !slice_ok(surface, ch_off, channels, spatial, index)) return false;
    const uint16_t *s = shadow_for_read(surface);
    if (!s) return false;
    esp_interop_argmax_f16_strided(s + (size_t)ch_off * spatial + index, channels, spatial, out_index, out_value);
    return true;
}

bool esp_interop_io_write_fp16_at(ESPSurfaceRef surface, int ch_off, const float *data, int channels, int spatial) {
    if (!data || !region_ok(surface, ch_off, channels, spatial)) return false;
    uint16_t *d = shadow_for_write(surface);
    if (!d) return false;
    esp_interop_cvt_f32_to_f16(d + (size_t)ch_off * spatial, data, channels * spatial);
    return true;
}
bool esp_interop_io_write_fp16(ESPSurfaceRef surface, const float *data, int channels, int spatial) {
    return esp_interop_io_write_fp16_at(surface, 0, data, channels, spatial);
}
bool esp_interop_io_read_fp16(ESPSurfaceRef surface, int ch_off, float *data, int channels, int spatial) {
    if (!data || !region_ok(surface, ch_off, channels, spatial)) return false;
    const uint16_t *s = shadow_for_read(surface);
    if (!s) return false;
    esp_interop_cvt_f16_to_f32(data, s + (size_t)ch_off * spatial, channels * spatial);
    return true;
}
bool esp_interop_io_read_fp16_batched(ESPSurfaceRef surface, int spatial, float *const *destinations, const int *channel_offsets,
                                      const int *channels, int region_count) {
    if (!destinations || !channel_offsets || !channels || region_count < 0) return false;
    for (int r = 0; r < region_count; r++) if (!region_ok(surface, channel_offsets[r], channels[r], spatial) || !destinations[r]) return false;
    for (int r = 0; r < region_count; r++) if (!esp_interop_io_read_fp16(surface, channel_offsets[r], destinations[r], channels[r], spatial)) return false;
    return true;
}

bool esp_interop_io_write_embedding_batch_fp16(ESPSurfaceRef surface, int ch_off, int spatial, const float *table, int vocab_size, int dim,
                                               const uint16_t *token_ids, int stream_count) {
    if (!table || !token_ids || stream_count < 0 || stream_count > spatial || !region_ok(surface, ch_off, dim, spatial)) return false;
    for (int s = 0; s < stream_count; s++) if (token_ids[s] >= vocab_size) return false;
    uint16_t *d = shadow_for_write(surface);
    if (!d) return false;
    for (int s = 0; s < stream_count; s++)
        for (int c = 0; c < dim; c++) d[(size_t)(ch_off + c) * spatial + s] = float_to_half_rne(table[(size_t)token_ids[s] * dim + c]);
    return true;
}

bool esp_interop_io_argmax_batch_fp16_spatial(ESPSurfaceRef surface, int ch_off, int spatial, int channels, int stream_count, int *out_indices,
                                              float *out_values) {
    if (!out_indices || !out_values || stream_count < 0 || stream_count > spatial || channels <= 0 || !region_ok(surface, ch_off, channels, spatial)) return false;
    const uint16_t *s = shadow_for_read(surface);
    if (!s) return false;
    for (int i = 0; i < stream_count; i++) esp_interop_argmax_f16_strided(s + (size_t)ch_off * spatial + i, channels, spatial, &out_indices[i], &out_values[i]);
    return true;
}

// ---- what the reference's hybrid decode does between its kernel evaluations, on surfaces resident in HBM ----
namespace {
bool surfaces_on_device(std::initializer_list<ESPSurface *> list) {
    for (ESPSurface *s : list) if (!s || !surface_to_device(s)) return false;
    return true;
}
void written_on_device(ESPSurface *s) { s->device_valid = true; s->host_valid = false; }
bool finish(hipError_t e, const char *what) {
    if (e == hipSuccess) e = hipStreamSynchronize(context().stream);
    if (e != hipSuccess) { fail_hip(e, what); return false; }
    return true;
}
}  // namespace

bool esp_interop_rope_decode(ESPSurfaceRef q, ESPSurfaceRef k, int n_heads, int n_kv_heads, int head_dim, int position, float theta, int lane_spatial) {
    if (n_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || head_dim % 2 != 0 || position < 0 || lane_spatial <= 0 ||
        !region_ok(q, 0, n_heads * head_dim, lane_spatial) || !region_ok(k, 0, n_kv_heads * head_dim, lane_spatial) || !surfaces_on_device({q, k}))
        return false;
    const hipError_t e = launch_surface_rope(reinterpret_cast<uint16_t *>(q->device), reinterpret_cast<uint16_t *>(k->device), n_heads, n_kv_heads, head_dim,
                                             position, theta, lane_spatial, context().stream);
    if (!finish(e, "rope_decode")) return false;   // a launch that failed wrote nothing: the surfaces keep their valid copies
    written_on_device(q); written_on_device(k);
    return true;
}

bool esp_interop_kv_cache_scatter(ESPSurfaceRef k_src, ESPSurfaceRef v_src, ESPSurfaceRef k_cache, ESPSurfaceRef v_cache, int kv_dim, int token_index,
                                  int cache_stride, int lane_spatial) {
    if (kv_dim <= 0 || lane_spatial <= 0 || !slice_ok(k_cache, 0, kv_dim, cache_stride, token_index) || !slice_ok(v_cache, 0, kv_dim, cache_stride, token_index) ||
        !region_ok(k_src, 0, kv_dim, lane_spatial) || !region_ok(v_src, 0, kv_dim, lane_spatial) || !surfaces_on_device({k_src, v_src, k_cache, v_cache}))
        return false;
    const hipError_t e = launch_surface_kv_scatter(reinterpret_cast<const uint16_t *>(k_src->device), reinterpret_cast<const uint16_t *>(v_src->device),
                                                   reinterpret_cast<uint16_t *>(k_cache->device), reinterpret_cast<uint16_t *>(v_cache->device), kv_dim,
                                                   token_index, cache_stride, lane_spatial, context().stream);
    if (!finish(e, "kv_cache_scatter")) return false;
    written_on_device(k_cache); written_on_device(v_cache);
    return true;
}

bool esp_interop_decode_sdpa(ESPSurfaceRef q, ESPSurfaceRef k_cache, ESPSurfaceRef v_cache, ESPSurfaceRef context_surface, int heads, int kv_heads, int head_dim,
                             int visible_tokens, int token_base, int cache_stride, int lane_spatial) {
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0 || visible_tokens <= 0 || token_base < 0 || lane_spatial <= 0 ||
        token_base + visible_tokens > cache_stride || !region_ok(q, 0, heads * head_dim, lane_spatial) ||
        !region_ok(context_surface, 0, heads * head_dim, lane_spatial) || !region_ok(k_cache, 0, kv_heads * head_dim, cache_stride) ||
        !region_ok(v_cache, 0, kv_heads * head_dim, cache_stride) || !surfaces_on_device({q, k_cache, v_cache, context_surface}))
        return false;
    const hipError_t e = launch_surface_sdpa(reinterpret_cast<const uint16_t *>(q->device), reinterpret_cast<const uint16_t *>(k_cache->device),
                                             reinterpret_cast<const uint16_t *>(v_cache->device), reinterpret_cast<uint16_t *>(context_surface->device), heads,
                                             kv_heads, head_dim, visible_tokens, token_base, cache_stride, lane_spatial, context().stream);
    if (!finish(e, "decode_sdpa")) return false;
    written_on_device(context_surface);
    return true;
}

// ---- the remaining surface I/O variants of ane_interop.h ----
void esp_interop_gather_f16_to_f32(float *dst, const void *src, int count, int stride) {
    const uint16_t *s = static_cast<const uint16_t *>(src);
    for (int i = 0; i < count; i++) dst[i] = half_to_float(s[(size_t)i * stride]);
}
void esp_interop_scatter_f32_to_f16(void *dst, const float *src, int count, int stride) {
    uint16_t *d = static_cast<uint16_t *>(dst);
    for (int i = 0; i < count; i++) d[(size_t)i * stride] = float_to_half_rne(src[i]);
}

bool esp_interop_io_copy_two_fp16_spatial_slices(ESPSurfaceRef dst0, int dst0_ch_off, int dst0_index, int dst0_spatial, ESPSurfaceRef src0, int src0_ch_off,
                                                 int src0_index, int src0_spatial, ESPSurfaceRef dst1, int dst1_ch_off, int dst1_index, int dst1_spatial,
                                                 ESPSurfaceRef src1, int src1_ch_off, int src1_index, int src1_spatial, int channels) {
    // both pairs are checked before either is touched
    if (!slice_ok(dst0, dst0_ch_off, channels, dst0_spatial, dst0_index) || !slice_ok(src0, src0_ch_off, channels, src0_spatial, src0_index) ||
        !slice_ok(dst1, dst1_ch_off, channels, dst1_spatial, dst1_index) || !slice_ok(src1, src1_ch_off, channels, src1_spatial, src1_index))
        return false;
    return esp_interop_io_copy_fp16_spatial_slice(dst0, dst0_ch_off, dst0_index, dst0_spatial, src0, src0_ch_off, src0_index, src0_spatial, channels) &&
           esp_interop_io_copy_fp16_spatial_slice(dst1, dst1_ch_off, dst1_index, dst1_spatial, src1, src1_ch_off, src1_index, src1_spatial, channels);
}

bool esp_interop_io_argmax_fp16_spatial_slice_with_hint(ESPSurfaceRef surface, int ch_off, int index, int spatial, int channels, ESPSurfaceRef hint_surface,
                                                        int hint_index, int hint_spatial, int *out_index, float *out_value) {
    if (channels <= 0 || !slice_ok(surface, ch_off, channels, spatial, index) || !slice_ok(hint_surface, 0, 1, hint_spatial, hint_index)) return false;
    const uint16_t *s = shadow_for_read(surface), *hint = shadow_for_read(hint_surface);
    if (!s || !hint) return false;
    // the hint is the column's maximum (the classifier kernel's reduce_max output): the first channel that equals it is the
    // first maximum; a hint that matches nothing falls back to the full scan
    const uint16_t want = hint[hint_index];
    for (int c = 0; c < channels; c++)
        if (s[(size_t)(ch_off + c) * spatial + index] == want) {
            if (out_index) *out_index = c;
            if (out_value) *out_value = half_to_float(want);
            return true;
        }
    esp_interop_argmax_f16_strided(s + (size_t)ch_off * spatial + index, channels, spatial, out_index, out_value);
    return true;
}

bool esp_interop_io_write_fp16_at_batched(ESPSurfaceRef surface, const int *channel_offsets, const float *const *sources, const int *channels, int region_count,
                                          int spatial) {
    if (!channel_offsets || !sources || !channels || region_count < 0) return false;
    for (int r = 0; r < region_count; r++) if (!sources[r] || !region_ok(surface, channel_offsets[r], channels[r], spatial)) return false;
    for (int r = 0; r < region_count; r++) if (!esp_interop_io_write_fp16_at(surface, channel_offsets[r], sources[r], channels[r], spatial)) return false;
    return true;
}

bool esp_interop_io_copy_batched(ESPSurfaceRef dst, ESPSurfaceRef src, const int *dst_channel_offsets, const int *src_channel_offsets, const int *channels,
                                 int region_count, int spatial) {
    if (!dst_channel_offsets || !src_channel_offsets || !channels || region_count < 0) return false;
    for (int r = 0; r < region_count; r++)
        if (!region_ok(dst, dst_channel_offsets[r], channels[r], spatial) || !region_ok(src, src_channel_offsets[r], channels[r], spatial)) return false;
    for (int r = 0; r < region_count; r++) if (!esp_interop_io_copy(dst, dst_channel_offsets[r], src, src_channel_offsets[r], channels[r], spatial)) return false;
    return true;
}

bool esp_interop_io_copy_multi_src(ESPSurfaceRef dst, const ESPSurfaceRef *sources, const int *dst_channel_offsets, const int *src_channel_offsets,
                                   const int *channels, int region_count, int spatial) {
    if (!sources || !dst_channel_offsets || !src_channel_offsets || !channels || region_count < 0) return false;
    for (int r = 0; r < region_count; r++)
        if (!region_ok(dst, dst_channel_offsets[r], channels[r], spatial) || !region_ok(sources[r], src_channel_offsets[r], channels[r], spatial)) return false;
    for (int r = 0; r < region_count; r++)
        if (!esp_interop_io_copy(dst, dst_channel_offsets[r], sources[r], src_channel_offsets[r], channels[r], spatial)) return false;
    return true;
}

// The channel range is split into n_blocks parts that are scanned independently and merged in channel order, so the result
// is the serial scan's: lowest index on ties (surface_io.c:689-700).  (The reference runs the parts on separate cores.)
bool esp_interop_io_argmax_batch_fp16_spatial_parallel(ESPSurfaceRef surface, int ch_off, int spatial, int channels, int stream_count, int *out_indices,
                                                       float *out_values, int n_blocks) {
    if (!out_indices || !out_values || stream_count < 0 || stream_count > spatial || channels <= 0 || !region_ok(surface, ch_off, channels, spatial)) return false;
    const uint16_t *s = shadow_for_read(surface);
    if (!s) return false;
    if (n_blocks < 1) n_blocks = 1;
    if (n_blocks > channels) n_blocks = channels;
    const int per = (channels + n_blocks - 1) / n_blocks;
    for (int i = 0; i < stream_count; i++) {
        int best = 0;
        float bv = -INFINITY;
        bool any = false;
        for (int b = 0; b < n_blocks; b++) {
            const int lo = b * per, hi = lo + per < channels ? lo + per : channels;
            if (lo >= hi) break;
            int bi = 0;
            float v = 0.0f;
            esp_interop_argmax_f16_strided(s + (size_t)(ch_off + lo) * spatial + i, hi - lo, spatial, &bi, &v);
            if (!any || v > bv) { bv = v; best = lo + bi; any = true; }   // strict >: an earlier block keeps a tie
        }
        out_indices[i] = best;
        out_values[i] = bv;
    }
    return true;
}
bool esp_interop_io_argmax_batch_fp16_spatial_nolock(ESPSurfaceRef surface, int ch_off, int spatial, int channels, int stream_count, int *out_indices,
                                                     float *out_values, int n_blocks) {
    // "assumes the surface is already coherent": the host shadow is read as it is when it is current, else it is fetched
    return esp_interop_io_argmax_batch_fp16_spatial_parallel(surface, ch_off, spatial, channels, stream_count, out_indices, out_values, n_blocks);
}

// ane_interop_fused_expansion_argmax_fp16 (surface_io.c:1438-1520, :1521-1700): logit[c][s] = sum_k proj[g * cpg + k][s] * w[c][k] with
// g = c / (vocab / groups), accumulated in fp16 with a fused multiply-add per term as the NEON code does, strict > across
// channels.  The same argument checks: vocab <= 65535, spatial a multiple of 8, bottleneck and vocab multiples of groups.
bool esp_interop_fused_expansion_argmax_fp16(ESPSurfaceRef proj_surface, int proj_ch_off, int spatial, int bottleneck, int groups,
                                             const void *expansion_weights_fp16, int vocab_size, int stream_count, int *out_indices, float *out_values,
                                             int n_blocks) {
    (void)n_blocks;   // the partition only spreads work over cores in the reference; the result does not depend on it
    if (!proj_surface || !expansion_weights_fp16 || !out_indices || !out_values) return false;
    if (proj_ch_off < 0 || spatial <= 0 || bottleneck <= 0 || groups <= 0 || vocab_size <= 0) return false;
    if (stream_count <= 0 || stream_count > spatial || vocab_size > 65535) return false;
    if (spatial > 32768 || spatial % 8 != 0 || bottleneck % groups != 0 || vocab_size % groups != 0) return false;
    if (!region_ok(proj_surface, proj_ch_off, bottleneck, spatial)) return false;
    const uint16_t *proj = shadow_for_read(proj_surface);
    if (!proj) return false;
    const _Float16 *w = static_cast<const _Float16 *>(expansion_weights_fp16);
    const int cpg = bottleneck / groups, ch_per_group = vocab_size / groups;
    for (int s = 0; s < stream_count; s++) {
        _Float16 best = (_Float16)(-65504.0f);
        int best_i = 0;
        for (int c = 0; c < vocab_size; c++) {
            const int g = c / ch_per_group;
            _Float16 acc = (_Float16)0.0f;
            for (int k = 0; k < cpg; k++) {
                const _Float16 p = __builtin_bit_cast(_Float16, proj[(size_t)(proj_ch_off + g * cpg + k) * spatial + s]);
                acc = (_Float16)((double)w[(size_t)c * cpg + k] * (double)p + (double)acc);   // one rounding per term: fp16 fused multiply-add
            }
            if (acc > best) { best = acc; best_i = c; }
        }
        out_indices[s] = best_i;
        out_values[s] = (float)best;
    }
    return true;
}

// The factored head resident in HBM (MetalExpansionArgmax.swift:966-1088): weights uploaded once, candidates and results in buffers the
// object keeps, one kernel over (vocab, lane) and a final pick per lane.
struct ESPExpansionHead {
    uint16_t *w = nullptr;
    int bottleneck = 0, groups = 0, vocab = 0, blocks = 0, lanes = 0;
    float *cand_v = nullptr, *out_v = nullptr;
    int *cand_i = nullptr, *out_i = nullptr;
};

namespace {
void release_expansion_buffers(ESPExpansionHead *h) {
    for (void *p : {(void *)h->cand_v, (void *)h->out_v, (void *)h->cand_i, (void *)h->out_i}) if (p) (void)hipFree(p);
    h->cand_v = h->out_v = nullptr;
    h->cand_i = h->out_i = nullptr;
    h->lanes = 0;
}
bool reserve_expansion_lanes(ESPExpansionHead *h, int lanes) {
    if (lanes <= h->lanes) return true;
    release_expansion_buffers(h);
    const size_t cand = (size_t)lanes * h->blocks;
    if (hipMalloc((void **)&h->cand_v, cand * sizeof(float)) != hipSuccess || hipMalloc((void **)&h->cand_i, cand * sizeof(int)) != hipSuccess ||
        hipMalloc((void **)&h->out_v, (size_t)lanes * sizeof(float)) != hipSuccess || hipMalloc((void **)&h->out_i, (size_t)lanes * sizeof(int)) != hipSuccess) {
        release_expansion_buffers(h);
        return false;
    }
    h->lanes = lanes;
    return true;
}
}  // namespace

ESPExpansionHeadRef esp_interop_expansion_head_create(const void *expansion_weights_fp16, int bottleneck, int groups, int vocab_size) {
    if (!expansion_weights_fp16 || bottleneck <= 0 || groups <= 0 || vocab_size <= 0 || vocab_size > 65535 || bottleneck % groups != 0 ||
        vocab_size % groups != 0 || bottleneck > 24 * 1024) {
        fail(ESP_ERR_INVALID_ARGUMENT, "expansion_head_create: vocab <= 65535, bottleneck and vocab multiples of groups");
        return nullptr;
    }
    if (ensure_init() != ESP_OK) return nullptr;
    ESPExpansionHead *h = new ESPExpansionHead();
    h->bottleneck = bottleneck; h->groups = groups; h->vocab = vocab_size;
    h->blocks = (vocab_size + 255) / 256 < 256 ? (vocab_size + 255) / 256 : 256;
    const size_t bytes = (size_t)vocab_size * (bottleneck / groups) * 2;
    hipError_t e = hipMalloc((void **)&h->w, bytes);
    if (e == hipSuccess) e = hipMemcpy(h->w, expansion_weights_fp16, bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        fail_hip(e, "expansion_head_create");
        if (h->w) (void)hipFree(h->w);
        delete h;
        return nullptr;
    }
    return h;
}

bool esp_interop_expansion_head_argmax(ESPExpansionHeadRef head, ESPSurfaceRef proj_surface, int proj_ch_off, int spatial, int stream_count, int fp32_sums,
                                       int *out_indices, float *out_values) {
    if (!head || !proj_surface || !out_indices || !out_values) return false;
    if (proj_ch_off < 0 || spatial <= 0 || stream_count <= 0 || stream_count > spatial || spatial > 32768 || spatial % 8 != 0) return false;
    if (!region_ok(proj_surface, proj_ch_off, head->bottleneck, spatial) || !surfaces_on_device({proj_surface})) return false;
    if (!reserve_expansion_lanes(head, stream_count)) { fail(ESP_ERR_OUT_OF_MEMORY, "expansion_head_argmax: candidate buffers"); return false; }
    const uint16_t *proj = reinterpret_cast<const uint16_t *>(proj_surface->device) + (size_t)proj_ch_off * spatial;
    hipError_t e = launch_expansion_argmax(proj, spatial, stream_count, head->w, head->bottleneck, head->groups, head->vocab, fp32_sums != 0, head->blocks,
                                           head->cand_v, head->cand_i, head->out_i, head->out_v, context().stream);
    if (e == hipSuccess) e = hipMemcpyAsync(out_indices, head->out_i, (size_t)stream_count * sizeof(int), hipMemcpyDeviceToHost, context().stream);
    if (e == hipSuccess) e = hipMemcpyAsync(out_values, head->out_v, (size_t)stream_count * sizeof(float), hipMemcpyDeviceToHost, context().stream);
    return finish(e, "expansion_head_argmax");
}

void esp_interop_expansion_head_free(ESPExpansionHeadRef head) {
    if (!head) return;
    release_expansion_buffers(head);
    if (head->w) (void)hipFree(head->w);
    delete head;
}

bool esp_interop_io_lock_write(ESPSurfaceRef s) { if (!s || !surface_to_host(s)) return false; s->write_locks++; return true; }
bool esp_interop_io_unlock_write(ESPSurfaceRef s) { if (!s || s->write_locks <= 0) return false; s->write_locks--; s->device_valid = false; return true; }
bool esp_interop_io_lock_read(ESPSurfaceRef s) { if (!s || !surface_to_host(s)) return false; s->read_locks++; return true; }
bool esp_interop_io_unlock_read(ESPSurfaceRef s) { if (!s || s->read_locks <= 0) return false; s->read_locks--; return true; }
bool esp_interop_io_write_fp16_unlocked(ESPSurfaceRef s, const float *data, int channels, int spatial) {
    if (!s || s->write_locks <= 0) return false;
    return esp_interop_io_write_fp16_at(s, 0, data, channels, spatial);
}
bool esp_interop_io_read_fp16_unlocked(ESPSurfaceRef s, int ch_off, float *data, int channels, int spatial) {
    if (!s || s->read_locks <= 0) return false;
    return esp_interop_io_read_fp16(s, ch_off, data, channels, spatial);
}

}  // extern "C"
