// Tilings of the rows product (gemm_rows_tiles.h) with 2 row tiles: plain and bias epilogues, 32-bit output.
#include "gemm_rows_tiles.h"

int he_rows_tiles2_f32(HE_ROWS_DISPATCH_ARGS) {
  HE_ROWS_TILING(2, 1, 4, false, float)
  HE_ROWS_TILING(2, 1, 8, false, float)
  HE_ROWS_TILING(2, 2, 8, false, float)
  HE_ROWS_TILING(2, 1, 16, false, float)
  HE_ROWS_NO_TILING;
}
