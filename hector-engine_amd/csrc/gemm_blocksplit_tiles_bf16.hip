// Tilings of the few-rows product (gemm_blocksplit_tiles.h): plain, bias and residual epilogues, bfloat16 output.
#include "gemm_blocksplit_tiles.h"

int he_blocksplit_tiles_bf16(HE_BS_DISPATCH_ARGS) {
  HE_BS_ALL_TILINGS(false, bf16_t);
}
