// Tilings of the few-rows product (gemm_blocksplit_tiles.h): gated SiLU x up epilogue, 32-bit output.
#include "gemm_blocksplit_tiles.h"

int he_blocksplit_tiles_gated_f32(HE_BS_DISPATCH_ARGS) {
  HE_BS_ALL_TILINGS(true, float);
}
