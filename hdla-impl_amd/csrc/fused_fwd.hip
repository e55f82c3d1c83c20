// Fused chunk kernels, mode fwd (see fused_impl.cuh).
#define FUSED_TU_MODE 0
#include "fused_mode.inc"
