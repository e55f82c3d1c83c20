// Host-callable launchers of the HIP kernels (one per device stage); defined in the .hip files, used by api.hip.
#pragma once
#include <hip/hip_runtime.h>

#include "hdla_ws.h"

namespace hdla {

hipError_t launch_chunk_table(const int64_t* cu, int N, int T, int nch, int32_t* chunk_off, int32_t* chunk_seq, hipStream_t stream);

// K, V in {64, 128}; returns hipErrorInvalidValue for any other pair.
// mode: 0 = for the forward pass, 1 = for the backward pass, 2 = forward pass whose workspace the backward pass will use
template <typename T> hipError_t launch_prep(const ChunkArgs<T>& a, int K, int V, int mode, hipStream_t stream);
template <typename T> hipError_t launch_scan_fwd(const ChunkArgs<T>& a, int K, int V, bool write_o, hipStream_t stream);
template <typename T> hipError_t launch_scan_bwd(const ChunkArgs<T>& a, int K, int V, hipStream_t stream);
// both scans of the backward pass (scan_fwd without the output, scan_bwd) in one launch
template <typename T> hipError_t launch_scan_pair(const ChunkArgs<T>& a, int K, int V, hipStream_t stream);
template <typename T> hipError_t launch_chunk_grad(const ChunkArgs<T>& a, int K, int V, hipStream_t stream);
template <typename T> hipError_t launch_recurrent(const RecurrentArgs<T>& a, int K, int V, hipStream_t stream);

}  // namespace hdla
