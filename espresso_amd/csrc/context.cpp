#include "context.h"

#include <cstdarg>
#include <cstdio>
#include <mutex>

namespace esp {
namespace {
thread_local std::string t_last_error;
std::mutex g_init_mutex;
Context g_context;
}  // namespace

Context &context() { return g_context; }

void clear_error() { t_last_error.clear(); }

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    t_last_error = buf;
    return code;
}

int fail_hip(hipError_t e, const char *what) {
    int code = e == hipErrorOutOfMemory ? ESP_ERR_OUT_OF_MEMORY
               : (e == hipErrorNoDevice || e == hipErrorInvalidDevice) ? ESP_ERR_NO_DEVICE
                                                                        : ESP_ERR_LAUNCH_FAILED;
    return fail(code, "%s: %s", what, hipGetErrorString(e));
}

const char *last_error_text() { return t_last_error.c_str(); }

int ensure_init() {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_context.ready) return ESP_OK;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(ESP_ERR_NO_DEVICE, "no HIP device available (%s); this library has no CPU fallback",
                    e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    }
    ESP_HIP_TRY(hipSetDevice(0));
    ESP_HIP_TRY(hipGetDeviceProperties(&g_context.props, 0));
    ESP_HIP_TRY(hipStreamCreateWithFlags(&g_context.stream, hipStreamNonBlocking));
    g_context.device = 0;
    {
        const int rc = noalloc_setup(0);
        if (rc != ESP_OK) return rc;
    }
    g_context.ready = true;
    return ESP_OK;
}

int matrix_upload(int format, const void *gguf_blocks, int rows, int cols, DeviceMatrix *out) {
    *out = DeviceMatrix{};
    if (!gguf_blocks || rows <= 0 || cols <= 0) return fail(ESP_ERR_INVALID_ARGUMENT, "matrix: null data or empty shape");
    if (!(format == FMT_F32 || format == FMT_F16 || format == FMT_Q4_0 || format == FMT_Q8_0 || format == FMT_Q4_K))
        return fail(ESP_ERR_UNSUPPORTED, "matrix: format %d has no GEMV kernel", format);
    const int block = format == FMT_F16 ? 8 : format == FMT_F32 ? 4 : format_block_elems(format);
    if (cols % block != 0) return fail(ESP_ERR_INVALID_ARGUMENT, "matrix: cols %d is not a multiple of %d", cols, block);
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const size_t elems = (size_t)rows * cols;
    const size_t src_bytes = format_bytes(format, elems);

    DeviceMatrix m;
    m.format = format; m.rows = rows; m.cols = cols;
    switch (format) {
    case FMT_Q8_0: m.qs_row_bytes = (size_t)cols; break;
    case FMT_Q4_0: m.qs_row_bytes = (size_t)cols / 2; break;
    case FMT_Q4_K: m.qs_row_bytes = (size_t)cols / 256 * 144; break;
    case FMT_F32: m.qs_row_bytes = (size_t)cols * 4; break;
    default: m.qs_row_bytes = (size_t)cols * 2; break;
    }
    if (m.qs_row_bytes % 16 != 0) return fail(ESP_ERR_INVALID_ARGUMENT, "matrix: row of %zu bytes is not 16-byte aligned", m.qs_row_bytes);
    if ((rc = device_alloc(&m.qs, (size_t)rows * m.qs_row_bytes)) != ESP_OK) return rc;
    const bool planes = format == FMT_Q8_0 || format == FMT_Q4_0;
    if (planes && (rc = device_alloc(&m.scales, elems / 32)) != ESP_OK) { matrix_release(&m); return rc; }

    hipError_t e;
    if (planes) {
        uint8_t *staging = nullptr;
        if ((rc = device_alloc(&staging, src_bytes)) != ESP_OK) { matrix_release(&m); return rc; }
        e = hipMemcpyAsync(staging, gguf_blocks, src_bytes, hipMemcpyHostToDevice, c.stream);
        if (e == hipSuccess) e = launch_repack(format, staging, rows, cols, m, c.stream);
        // Q4_0 matrices of the widths the matrix-core GEMV is built for also get the tiled copy it reads
        if (e == hipSuccess && format == FMT_Q4_0 && gemv_wants_tiled_copy(format, cols)) {
            const size_t tiled_bytes = (size_t)((rows + 15) / 16) * (cols / 512) * 4608;
            if ((rc = device_alloc(&m.tiled, tiled_bytes)) != ESP_OK) { (void)hipFree(staging); matrix_release(&m); return rc; }
            e = launch_q40_tile(m.qs, m.scales, rows, cols, m.tiled, c.stream);
        }
        if (e == hipSuccess && format == FMT_Q8_0 && gemv_wants_tiled_copy(format, cols)) {
            const size_t tiled_bytes = (size_t)((rows + 15) / 16) * (cols / 256) * 4352;
            if ((rc = device_alloc(&m.tiled, tiled_bytes)) != ESP_OK) { (void)hipFree(staging); matrix_release(&m); return rc; }
            e = launch_q80_tile(m.qs, m.scales, rows, cols, m.tiled, c.stream);
        }
        if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
        (void)hipFree(staging);
    } else {
        e = hipMemcpyAsync(m.qs, gguf_blocks, src_bytes, hipMemcpyHostToDevice, c.stream);
        // Q4_K matrices of the widths the matrix-core GEMV is built for also get the tiled copy it reads
        if (e == hipSuccess && format == FMT_Q4_K && gemv_wants_tiled_copy(format, cols)) {
            const size_t tiled_bytes = (size_t)((rows + 15) / 16) * (cols / 256) * 2304;
            if ((rc = device_alloc(&m.tiled, tiled_bytes)) != ESP_OK) { matrix_release(&m); return rc; }
            e = launch_q4k_tile(m.qs, rows, cols, m.tiled, c.stream);
        }
        if (e == hipSuccess && format == FMT_F16 && gemv_wants_tiled_copy(format, cols)) {
            const size_t tiled_bytes = (size_t)((rows + 15) / 16) * (cols / 256) * 8192;
            if ((rc = device_alloc(&m.tiled, tiled_bytes)) != ESP_OK) { matrix_release(&m); return rc; }
            e = launch_f16_tile(m.qs, rows, cols, m.tiled, c.stream);
        }
        if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    }
    if (e != hipSuccess) { matrix_release(&m); return fail_hip(e, "matrix upload"); }
    *out = m;
    return ESP_OK;
}

void matrix_release(DeviceMatrix *m) {
    if (m->qs) (void)hipFree(m->qs);
    if (m->scales) (void)hipFree(m->scales);
    if (m->tiled) (void)hipFree(m->tiled);
    *m = DeviceMatrix{};
}

}  // namespace esp

extern "C" const char *esp_last_error(void) { return esp::last_error_text(); }
