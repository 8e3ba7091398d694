// Library identity, error text and the plain copy entry point.
#include "common.h"

static thread_local char g_err[512];

char *infllm_err_buf() { return g_err; }

int infllm_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" int infllm_version(void) { return INFLLM_ABI_VERSION; }

extern "C" const char *infllm_last_error(void) { return g_err; }

extern "C" int infllm_copy_async(void *dst, const void *src, int64_t nbytes, int32_t kind, void *stream) {
    INFLLM_REQUIRE(dst && src && nbytes >= 0, "copy_async: null pointer or negative size");
    hipMemcpyKind k;
    switch (kind) {
        case 1: k = hipMemcpyHostToDevice; break;
        case 2: k = hipMemcpyDeviceToHost; break;
        case 3: k = hipMemcpyDeviceToDevice; break;
        default: return infllm_fail(-1, "copy_async: kind %d is not 1 (h2d), 2 (d2h) or 3 (d2d)", kind);
    }
    if (nbytes == 0) return 0;
    hipError_t e = hipMemcpyAsync(dst, src, (size_t)nbytes, k, (hipStream_t)stream);
    if (e != hipSuccess) return infllm_fail(-2, "copy_async: %s", hipGetErrorString(e));
    return 0;
}
