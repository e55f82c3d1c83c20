// Entry points of the scan kernels per element type and head shape; each shape is compiled in its own
// translation unit (scan_*.hip) so that the build can run them in parallel.
#pragma once
#include "hdla_launch.h"

namespace hdla {

enum ScanKind { SCAN_FWD_O, SCAN_FWD, SCAN_BWD, SCAN_PAIR };   // forward scan with / without the output, reverse, both

template <typename T, int K, int V> hipError_t launch_scan_shape(const ChunkArgs<T>& a, ScanKind kind, hipStream_t stream);

}  // namespace hdla
