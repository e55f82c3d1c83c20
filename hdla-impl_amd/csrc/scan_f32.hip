// Scan kernels, fp32 inputs, head sizes K=64 V=64, K=64 V=128, K=128 V=64, K=128 V=128 (see scan_impl.cuh).
#include "scan_impl.cuh"

namespace hdla {
template hipError_t launch_scan_shape<float, 64, 64>(const ChunkArgs<float>&, ScanKind, hipStream_t);
template hipError_t launch_scan_shape<float, 64, 128>(const ChunkArgs<float>&, ScanKind, hipStream_t);
template hipError_t launch_scan_shape<float, 128, 64>(const ChunkArgs<float>&, ScanKind, hipStream_t);
template hipError_t launch_scan_shape<float, 128, 128>(const ChunkArgs<float>&, ScanKind, hipStream_t);
}  // namespace hdla
