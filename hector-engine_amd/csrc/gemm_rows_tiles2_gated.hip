// Tilings of the rows product (gemm_rows_tiles.h) with 2 row tiles: gated SiLU x up epilogue.
#include "gemm_rows_tiles.h"

int he_rows_tiles2_gated(HE_ROWS_DISPATCH_ARGS) {
  HE_ROWS_TILING(2, 1, 4, true, bf16_t)
  HE_ROWS_TILING(2, 1, 8, true, bf16_t)
  HE_ROWS_TILING(2, 2, 8, true, bf16_t)
  HE_ROWS_TILING(2, 1, 16, true, bf16_t)
  HE_ROWS_NO_TILING;
}
