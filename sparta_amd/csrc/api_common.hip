// Error text, version and the streaming-rate probe.
#include "common.hpp"
#include <string.h>

namespace spx {
char* last_error_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}

// Plain streaming kernels with the access shape the memory-bound kernels of this library
// use (16 bytes per lane, four independent accesses in flight per thread, non-temporal):
// a read-only pass and a copy.  They give the rates this machine sustains, to hold the
// bandwidth of those kernels against.
typedef uint32_t probe_vec __attribute__((ext_vector_type(4)));
template <bool COPY>
__global__ __launch_bounds__(256) void stream_probe_kernel(const probe_vec* __restrict__ src, probe_vec* __restrict__ dst, size_t n_vec) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    probe_vec acc = {0u, 0u, 0u, 0u};
    for (; i + 3 * stride < n_vec; i += 4 * stride) {
        probe_vec v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (COPY) __builtin_nontemporal_store(v[u], dst + i + u * stride);
            else acc ^= v[u];
        }
    }
    for (; i < n_vec; i += stride) {
        const probe_vec v = __builtin_nontemporal_load(src + i);
        if (COPY) __builtin_nontemporal_store(v, dst + i);
        else acc ^= v;
    }
    // the read-only pass keeps its loads alive through a store that practically never happens
    if (!COPY && (acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && dst) dst[0] = acc;
}
}  // namespace spx

extern "C" const char* spx_last_error(void) { return spx::last_error_buf(); }
extern "C" int spx_version(void) { return SPX_VERSION; }

extern "C" int spx_stream_probe(int mode, const void* src, void* dst, size_t bytes, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(mode == 0 || mode == 1, SPX_E_CONFIG, "mode must be 0 (read) or 1 (copy)");
    SPX_REQUIRE(src && (mode == 0 || dst), SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(bytes % 16 == 0 && aligned(src, 16) && (!dst || aligned(dst, 16)), SPX_E_ALIGN, "buffers and size must be multiples of 16 bytes");
    if (bytes == 0) return 0;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const size_t n_vec = bytes / 16;
    const unsigned blocks = (unsigned)(n_vec / 1024 < 8192 ? (n_vec / 1024 > 0 ? n_vec / 1024 : 1) : 8192);
    if (mode == 1)
        hipLaunchKernelGGL((stream_probe_kernel<true>), dim3(blocks), dim3(256), 0, st, reinterpret_cast<const probe_vec*>(src),
                           reinterpret_cast<probe_vec*>(dst), n_vec);
    else
        hipLaunchKernelGGL((stream_probe_kernel<false>), dim3(blocks), dim3(256), 0, st, reinterpret_cast<const probe_vec*>(src),
                           reinterpret_cast<probe_vec*>(dst), n_vec);
    SPX_LAUNCH_CHECK("stream_probe_kernel");
    return 0;
}
