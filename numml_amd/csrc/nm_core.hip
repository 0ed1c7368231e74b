// Error reporting and version of libnumml_hip.so.
#include "nm_common.hpp"

#include <cstdarg>
#include <cstdio>

namespace {
thread_local char g_last_error[512] = "";
}

namespace nm {
int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}
}  // namespace nm

namespace {
typedef float F4 __attribute__((ext_vector_type(4)));

// Reads n_read 16-byte words, writes the first n_write of them back out: plain streaming, four
// requests per lane in flight, nontemporal both ways like the SpMV kernels' streams.
__global__ __launch_bounds__(256) void stream_probe_kernel(const F4 *__restrict__ src, int64_t n_read,
                                                           F4 *__restrict__ dst, int64_t n_write) {
    constexpr int U = 4;
    F4 acc = {0, 0, 0, 0};
    const int64_t stride = (int64_t)gridDim.x * 256 * U;
    for (int64_t i = (int64_t)blockIdx.x * 256 * U + threadIdx.x; i < n_read; i += stride) {
        F4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t k = i + u * 256 < n_read ? i + u * 256 : n_read - 1;
            v[u] = __builtin_nontemporal_load(src + k);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (i + u * 256 < n_write) __builtin_nontemporal_store(v[u], dst + i + u * 256);
            else if (i + u * 256 < n_read) acc += v[u];
        }
    }
    // (keeps the loads that are not written back alive; never true for finite data)
    if (acc[0] + acc[1] + acc[2] + acc[3] == 1.2345678e38f && n_write > 0) dst[0] = acc;
}
}  // namespace

extern "C" int nm_stream_probe(const void *src, size_t read_bytes, void *dst, size_t write_bytes, nm_stream stream) {
    NM_REQUIRE(src != nullptr && read_bytes >= 16 && read_bytes % 16 == 0 && write_bytes % 16 == 0 &&
                   write_bytes <= read_bytes && (write_bytes == 0 || dst != nullptr),
               "nm_stream_probe: sizes must be multiples of 16 with write_bytes <= read_bytes");
    const int64_t n_read = (int64_t)(read_bytes / 16), n_write = (int64_t)(write_bytes / 16);
    int64_t grid = nm::ceil_div(n_read, 256 * 4);
    if (grid > 16384) grid = 16384;
    hipLaunchKernelGGL(stream_probe_kernel, dim3((unsigned)grid), dim3(256), 0, nm::as_stream(stream),
                       (const F4 *)src, n_read, (F4 *)dst, n_write);
    NM_LAUNCH_CHECK("stream_probe_kernel");
    return NM_OK;
}

extern "C" int nm_version(void) { return 1001; }

extern "C" const char *nm_last_error(void) { return g_last_error; }
