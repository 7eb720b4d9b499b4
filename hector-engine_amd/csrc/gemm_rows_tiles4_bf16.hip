// Tilings of the rows product (gemm_rows_tiles.h) with 4 row tiles: plain, bias and residual epilogues, bfloat16 output.
#include "gemm_rows_tiles.h"

int he_rows_tiles4_bf16(HE_ROWS_DISPATCH_ARGS) {
  HE_ROWS_TILING(4, 1, 4, false, bf16_t)
  HE_ROWS_TILING(4, 2, 4, false, bf16_t)
  HE_ROWS_TILING(4, 1, 8, false, bf16_t)
  HE_ROWS_TILING(4, 2, 8, false, bf16_t)
  HE_ROWS_TILING(4, 1, 16, false, bf16_t)
  HE_ROWS_NO_TILING;
}
