// Library-wide state behind the C ABI: the device, the stream and per-thread error text.
#pragma once

#include <string>

#include "../../include/espresso_hip.h"
#include "../../include/espresso_hip_bench.h"
#include "common.h"

namespace esp {

struct Context {
    bool ready = false;
    int device = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t props{};
};

// Initialises on first use.  Returns ESP_OK or ESP_ERR_NO_DEVICE (with the error text set).
int ensure_init();
Context &context();

// Records `message` for the calling thread and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t e, const char *what);
void clear_error();

#define ESP_HIP_TRY(expr)                                         \
    do {                                                          \
        hipError_t esp_hip_try_e = (expr);                        \
        if (esp_hip_try_e != hipSuccess) return ::esp::fail_hip(esp_hip_try_e, #expr); \
    } while (0)

// Device allocation that fails with a code instead of throwing.
template <typename T>
int device_alloc(T **out, size_t count) {
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, count * sizeof(T) ? count * sizeof(T) : 16);
    if (e != hipSuccess) {
        *out = nullptr;
        return fail(ESP_ERR_OUT_OF_MEMORY, "hipMalloc(%zu bytes): %s", count * sizeof(T), hipGetErrorString(e));
    }
    *out = static_cast<T *>(p);
    return ESP_OK;
}

// Looks up the device address of the fixed scratch array of esp_gemv_device_noalloc for `device`, which must be the
// current device (capi_ops.cpp; called once from ensure_init).
int noalloc_setup(int device);

// Uploads GGUF-layout blocks (host memory) into a DeviceMatrix laid out for the GEMV kernels.
int matrix_upload(int format, const void *gguf_blocks, int rows, int cols, DeviceMatrix *out);
void matrix_release(DeviceMatrix *m);

}  // namespace esp

// opaque handle behind ESPMatrix
struct ESPMatrix {
    esp::DeviceMatrix m;
};
