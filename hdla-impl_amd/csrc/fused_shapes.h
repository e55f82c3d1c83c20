// Argument block and host entry points of the fused chunk kernels (fused_impl.cuh); each mode is compiled in its own
// translation unit (fused_*.hip) so that the build can run them in parallel.
#pragma once
#include "hdla_launch.h"

namespace hdla {

// FUSED_FWD: forward pass (o, or o_local and G for segments > 0; segment records).  FUSED_SUM: the segment records only
// (what a backward pass runs first when the forward pass left no boundary record).  FUSED_CKPT: the backward pass's
// forward half: state checkpoints, (I - A_ab)^-1, u, strong-decay flags, and the records the reverse half chains.
// FUSED_REV: the reverse scan of the state gradient: dS checkpoints, dv_new, dh0.
enum FusedMode { FUSED_FWD = 0, FUSED_SUM = 1, FUSED_CKPT = 2, FUSED_REV = 3 };

template <typename T>
struct FusedArgs {
    ChunkArgs<T> c;
    int nseg;              // time segments per sequence
    // records per (sequence, head, segment), fp32 tiles in fragment order (see fused_impl.cuh)
    float* sloc;           // [N][H][nseg][K*V]
    float* mseg;           // [N][H][nseg][K*K]
    float* rseg;           // [N][H][nseg][K*V]
    const float* sin;      // [N][H][nseg][K*V]  states entering the segments (read by FUSED_CKPT)
    float* sin_out;        // the same record, written by fixup_kernel (nullable)
    float* ol;             // [H][nch][16][V] fp32  local outputs of segments > 0 (forward pass)
    T* gw;                 // [H][nch][16][K]       G of segments > 0 (forward pass); null: fixup_kernel only chains
    int* err;              // set nonzero by a wave whose bounded wait ran out
};

// K = V = 64, 2-byte elements only; hipErrorInvalidValue otherwise
template <typename T> hipError_t launch_fused(const FusedArgs<T>& a, int K, int V, int mode, hipStream_t stream);
template <typename T> hipError_t launch_fixup(const FusedArgs<T>& a, int K, int V, hipStream_t stream);

// per-mode instantiations
template <typename T, int MODE> hipError_t launch_fused_mode(const FusedArgs<T>& a, hipStream_t stream);

}  // namespace hdla
