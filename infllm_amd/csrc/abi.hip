// Library identity, error text and the plain copy entry point.
#include <stdlib.h>

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

extern "C" int infllm_cache_copy_async(void *dst, const void *src, int64_t nbytes, int32_t kind, void *stream) {
    return infllm_copy_async(dst, src, nbytes, kind, stream);
}

// ---------------------------------------------------------------------------
// Unit fetch: pinned host memory -> device slots in ONE launch.
// The sources of a block's cache misses are scattered over the host arena, and a
// hipMemcpyAsync per unit costs more to issue than the 512 KiB take to move; here the
// kernel reads the (device-mapped) pinned memory directly over PCIe.
namespace {

constexpr int kFetchMax = 64;          // units per launch

struct FetchList {
    const uint4 *src[kFetchMax];
    uint4 *dst[kFetchMax];
};

// A fixed number of workgroups walks all (unit, piece) pairs.  Reads that cross PCIe stay outstanding for
// microseconds and slow down whatever else runs on the chip in proportion to how many are in flight, so the
// launch is shaped for just enough of them to keep the link busy: 128 single-wave workgroups with one 16-byte
// load per lane (128 KiB in flight) measured best for the whole stream.  U independent loads per thread.
template <int U>
__global__ __launch_bounds__(256) void unit_fetch_kernel(FetchList list, int n_units, int64_t nbytes) {
    const int piece = (int)blockDim.x * U * 16;              // bytes moved by one workgroup iteration
    const int pieces_per_unit = (int)((nbytes + piece - 1) / piece);
    const int total = n_units * pieces_per_unit;
    const int64_t end = nbytes / 16;
    for (int w = blockIdx.x; w < total; w += gridDim.x) {
        const int unit = w / pieces_per_unit;
        const int64_t begin = (int64_t)(w % pieces_per_unit) * (piece / 16);
        const uint4 *src = list.src[unit];
        uint4 *dst = list.dst[unit];
        uint4 v[U];
#pragma unroll
        for (int i = 0; i < U; ++i)
            if (begin + threadIdx.x + blockDim.x * i < end) v[i] = src[begin + threadIdx.x + blockDim.x * i];
#pragma unroll
        for (int i = 0; i < U; ++i)
            if (begin + threadIdx.x + blockDim.x * i < end) dst[begin + threadIdx.x + blockDim.x * i] = v[i];
    }
}

// launch shape of the zero-copy fetch (see the kernel's comment)
constexpr int kFetchWorkgroups = 128, kFetchThreads = 64;

}  // namespace

extern "C" int infllm_fetch_units(const void *const *h_src, void *const *d_dst, int32_t n, int64_t nbytes, void *stream) {
    INFLLM_REQUIRE(n >= 0 && nbytes >= 0 && nbytes % 16 == 0, "fetch_units: bad sizes n=%d nbytes=%lld", n, (long long)nbytes);
    INFLLM_REQUIRE(n == 0 || (h_src && d_dst), "fetch_units: null list");
    if (nbytes == 0) return 0;
    for (int first = 0; first < n; first += kFetchMax) {
        const int m = n - first < kFetchMax ? n - first : kFetchMax;
        FetchList list;
        for (int i = 0; i < m; ++i) {
            INFLLM_REQUIRE(h_src[first + i] && d_dst[first + i], "fetch_units: null entry %d", first + i);
            INFLLM_REQUIRE(((uintptr_t)h_src[first + i] | (uintptr_t)d_dst[first + i]) % 16 == 0, "fetch_units: entry %d is not 16-byte aligned",
                           first + i);
            list.src[i] = (const uint4 *)h_src[first + i];
            list.dst[i] = (uint4 *)d_dst[first + i];
        }
        const int64_t piece = (int64_t)kFetchThreads * 16;
        const int64_t work = (int64_t)m * ((nbytes + piece - 1) / piece);
        const int wgs = work < kFetchWorkgroups ? (int)work : kFetchWorkgroups;
        hipLaunchKernelGGL(unit_fetch_kernel<1>, dim3(wgs), dim3(kFetchThreads), 0, (hipStream_t)stream, list, m, nbytes);
        INFLLM_CHECK_LAUNCH("unit_fetch");
    }
    return 0;
}

// library-internal: the same for sources in device memory (units that are still in a carve staging slot): one launch
// for all of them, shaped for HBM rather than for PCIe (as many workgroups as there are 4 KiB pieces)
int infllm_copy_units(const void *const *d_src, void *const *d_dst, int32_t n, int64_t nbytes, void *stream) {
    INFLLM_REQUIRE(n >= 0 && nbytes > 0 && nbytes % 16 == 0, "copy_units: bad sizes n=%d nbytes=%lld", n, (long long)nbytes);
    INFLLM_REQUIRE(n == 0 || (d_src && d_dst), "copy_units: null list");
    for (int first = 0; first < n; first += kFetchMax) {
        const int m = n - first < kFetchMax ? n - first : kFetchMax;
        FetchList list;
        for (int i = 0; i < m; ++i) {
            INFLLM_REQUIRE(d_src[first + i] && d_dst[first + i], "copy_units: null entry %d", first + i);
            INFLLM_REQUIRE(((uintptr_t)d_src[first + i] | (uintptr_t)d_dst[first + i]) % 16 == 0, "copy_units: entry %d is not 16-byte aligned",
                           first + i);
            list.src[i] = (const uint4 *)d_src[first + i];
            list.dst[i] = (uint4 *)d_dst[first + i];
        }
        const int64_t piece = 256 * 1 * 16;             // 4 KiB per workgroup: one round trip each, 128 workgroups per 512 KiB unit
        const int64_t work = (int64_t)m * ((nbytes + piece - 1) / piece);
        hipLaunchKernelGGL(unit_fetch_kernel<1>, dim3((unsigned)(work < 4096 ? work : 4096)), dim3(256), 0, (hipStream_t)stream, list, m, nbytes);
        INFLLM_CHECK_LAUNCH("copy_units");
    }
    return 0;
}

extern "C" void *infllm_host_device_pointer(void *h_pinned) {
    void *d = nullptr;
    if (!h_pinned || hipHostGetDevicePointer(&d, h_pinned, 0) != hipSuccess) {
        infllm_fail(-2, "host_device_pointer: %p is not device-mapped pinned memory", h_pinned);
        return nullptr;
    }
    return d;
}
