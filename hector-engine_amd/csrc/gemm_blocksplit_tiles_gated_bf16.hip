// Tilings of the few-rows product (gemm_blocksplit_tiles.h): gated SiLU x up epilogue, bfloat16 output.
#include "gemm_blocksplit_tiles.h"

int he_blocksplit_tiles_gated_bf16(HE_BS_DISPATCH_ARGS) {
  HE_BS_ALL_TILINGS(true, bf16_t);
}
