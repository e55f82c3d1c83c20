// Fused chunk kernels, mode ckpt (see fused_impl.cuh).
#define FUSED_TU_MODE 2
#include "fused_mode.inc"
