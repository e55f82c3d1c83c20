// Fused chunk kernels, mode rev (see fused_impl.cuh).
#define FUSED_TU_MODE 3
#include "fused_mode.inc"
