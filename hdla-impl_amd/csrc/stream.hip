// Streaming kernel of known traffic: a measurement aid, not part of the operator.  It reads `n_read` buffers and
// writes `n_write` buffers of `bytes` bytes each, 16 bytes a lane, and does nothing else, so that (a) a hardware
// traffic counter can be scaled by what it reads for a launch whose traffic is known exactly, and (b) the rate it
// reaches is what HBM delivers for that mix of reads and writes, the yardstick for kernels that are bound by memory.
#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>
#include "../../include/hdla_hip.h"

namespace hdla {

typedef int i32x4 __attribute__((ext_vector_type(4)));
struct StreamArgs { const char* rd[3]; char* wr[2]; long long n; };

template <int R, int W>
__global__ __launch_bounds__(256) void stream_kernel(StreamArgs a) {
    constexpr int U = 2;                                      // independent 16-byte pieces per lane and buffer
    const long long stride = (long long)gridDim.x * blockDim.x * 16;
    for (long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 16; i < a.n; i += U * stride) {
        i32x4 x[U][R > 0 ? R : 1];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (i + u * stride < a.n) x[u][r] = *reinterpret_cast<const i32x4*>(a.rd[r] + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            i32x4 s = {1, 2, 3, 4};
#pragma unroll
            for (int r = 0; r < R; ++r) s += x[u][r];
            if (i + u * stride < a.n) {
#pragma unroll
                for (int w = 0; w < W; ++w) *reinterpret_cast<i32x4*>(a.wr[w] + i + u * stride) = s;
                // a read-only launch still has to consume what it loaded; this store never happens for buffers
                // holding anything but one particular pattern
                if (W == 0 && s[0] == 0x7ffffff1 && s[1] == 0x12345) *reinterpret_cast<volatile int*>(const_cast<char*>(a.rd[0])) = 0;
            }
        }
    }
}

template <int R, int W> static hipError_t launch(const StreamArgs& a, hipStream_t s) {
    hipLaunchKernelGGL((stream_kernel<R, W>), dim3(4096), dim3(256), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_stream(const StreamArgs& a, int R, int W, hipStream_t s) {
    switch (R * 4 + W) {
        case 1 * 4 + 0: return launch<1, 0>(a, s);
        case 0 * 4 + 1: return launch<0, 1>(a, s);
        case 1 * 4 + 1: return launch<1, 1>(a, s);
        case 2 * 4 + 1: return launch<2, 1>(a, s);
        case 3 * 4 + 1: return launch<3, 1>(a, s);
        case 1 * 4 + 2: return launch<1, 2>(a, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace hdla

extern "C" int hdla_calib_stream(const void* const* reads, int n_read, void* const* writes, int n_write, size_t bytes,
                                 void* stream) {
    if (n_read < 0 || n_read > 3 || n_write < 0 || n_write > 2 || n_read + n_write == 0) return HDLA_ERR_SHAPE;
    if (bytes == 0 || bytes % 16 != 0) return HDLA_ERR_SHAPE;
    hdla::StreamArgs a{};
    for (int i = 0; i < n_read; ++i) {
        if (!reads || !reads[i]) return HDLA_ERR_NULL;
        if (reinterpret_cast<uintptr_t>(reads[i]) % 16) return HDLA_ERR_ALIGN;
        a.rd[i] = static_cast<const char*>(reads[i]);
    }
    for (int i = 0; i < n_write; ++i) {
        if (!writes || !writes[i]) return HDLA_ERR_NULL;
        if (reinterpret_cast<uintptr_t>(writes[i]) % 16) return HDLA_ERR_ALIGN;
        a.wr[i] = static_cast<char*>(writes[i]);
    }
    a.n = (long long)bytes;
    const hipError_t e = hdla::launch_stream(a, n_read, n_write, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? HDLA_OK : (e == hipErrorInvalidValue ? HDLA_ERR_SHAPE : (int)e);
}
