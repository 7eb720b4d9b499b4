// Tilings of the rows product (gemm_rows_tiles.h) with 4 row tiles: gated SiLU x up epilogue.
#include "gemm_rows_tiles.h"

int he_rows_tiles4_gated(HE_ROWS_DISPATCH_ARGS) {
  HE_ROWS_TILING(4, 1, 4, true, bf16_t)
  HE_ROWS_TILING(4, 2, 4, true, bf16_t)
  HE_ROWS_TILING(4, 1, 8, true, bf16_t)
  HE_ROWS_TILING(4, 2, 8, true, bf16_t)
  HE_ROWS_TILING(4, 1, 16, true, bf16_t)
  HE_ROWS_NO_TILING;
}
