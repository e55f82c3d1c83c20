// Host-side dispatch of the fused chunk kernels (kernels: fused_impl.cuh, compiled per mode in fused_*.hip).
#include "fused_shapes.h"

namespace hdla {

template <typename T>
hipError_t launch_fused(const FusedArgs<T>& a, int K, int V, int mode, hipStream_t stream) {
    if constexpr (sizeof(T) == 2) {
        if (K != 64 || V != 64) return hipErrorInvalidValue;
        switch (mode) {
            case FUSED_FWD: return launch_fused_mode<T, FUSED_FWD>(a, stream);
            case FUSED_SUM: return launch_fused_mode<T, FUSED_SUM>(a, stream);
            case FUSED_CKPT: return launch_fused_mode<T, FUSED_CKPT>(a, stream);
            case FUSED_REV: return launch_fused_mode<T, FUSED_REV>(a, stream);
        }
    }
    return hipErrorInvalidValue;
}
template hipError_t launch_fused<bf16>(const FusedArgs<bf16>&, int, int, int, hipStream_t);
template hipError_t launch_fused<float>(const FusedArgs<float>&, int, int, int, hipStream_t);

}  // namespace hdla
