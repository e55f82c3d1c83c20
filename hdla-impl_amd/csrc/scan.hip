// Host-side dispatch of the scan kernels by head shape (kernels: scan_impl.cuh, compiled in scan_*.hip).
#include "scan_shapes.h"

namespace hdla {

template <typename T>
static hipError_t launch_scan(const ChunkArgs<T>& a, int K, int V, ScanKind kind, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_scan_shape<T, 64, 64>(a, kind, stream);
    if (K == 128 && V == 128) return launch_scan_shape<T, 128, 128>(a, kind, stream);
    if (K == 64 && V == 128) return launch_scan_shape<T, 64, 128>(a, kind, stream);
    if (K == 128 && V == 64) return launch_scan_shape<T, 128, 64>(a, kind, stream);
    return hipErrorInvalidValue;
}

template <typename T>
hipError_t launch_scan_fwd(const ChunkArgs<T>& a, int K, int V, bool write_o, hipStream_t stream) {
    return launch_scan<T>(a, K, V, write_o ? SCAN_FWD_O : SCAN_FWD, stream);
}
template <typename T>
hipError_t launch_scan_bwd(const ChunkArgs<T>& a, int K, int V, hipStream_t stream) {
    return launch_scan<T>(a, K, V, SCAN_BWD, stream);
}
template <typename T>
hipError_t launch_scan_pair(const ChunkArgs<T>& a, int K, int V, hipStream_t stream) {
    return launch_scan<T>(a, K, V, SCAN_PAIR, stream);
}
template hipError_t launch_scan_fwd<bf16>(const ChunkArgs<bf16>&, int, int, bool, hipStream_t);
template hipError_t launch_scan_fwd<float>(const ChunkArgs<float>&, int, int, bool, hipStream_t);
template hipError_t launch_scan_bwd<bf16>(const ChunkArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_scan_bwd<float>(const ChunkArgs<float>&, int, int, hipStream_t);
template hipError_t launch_scan_pair<bf16>(const ChunkArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_scan_pair<float>(const ChunkArgs<float>&, int, int, hipStream_t);

}  // namespace hdla
