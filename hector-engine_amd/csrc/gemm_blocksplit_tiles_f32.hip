// Tilings of the few-rows product (gemm_blocksplit_tiles.h): plain, bias and residual epilogues, 32-bit output.
#include "gemm_blocksplit_tiles.h"

int he_blocksplit_tiles_f32(HE_BS_DISPATCH_ARGS) {
  HE_BS_ALL_TILINGS(false, float);
}
