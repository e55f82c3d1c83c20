// Scan kernels, bf16 inputs, head sizes K=128 V=64, K=128 V=128 (see scan_impl.cuh).
#include "scan_impl.cuh"

namespace hdla {
template hipError_t launch_scan_shape<bf16, 128, 64>(const ChunkArgs<bf16>&, ScanKind, hipStream_t);
template hipError_t launch_scan_shape<bf16, 128, 128>(const ChunkArgs<bf16>&, ScanKind, hipStream_t);
}  // namespace hdla
