// Fused chunk kernels, mode sum (see fused_impl.cuh).
#define FUSED_TU_MODE 1
#include "fused_mode.inc"
