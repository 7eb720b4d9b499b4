// Tilings of the rows product (gemm_rows_tiles.h) with 4 row tiles: plain and bias epilogues, 32-bit output.
#include "gemm_rows_tiles.h"

int he_rows_tiles4_f32(HE_ROWS_DISPATCH_ARGS) {
  HE_ROWS_TILING(4, 1, 4, false, float)
  HE_ROWS_TILING(4, 2, 4, false, float)
  HE_ROWS_TILING(4, 1, 8, false, float)
  HE_ROWS_TILING(4, 2, 8, false, float)
  HE_ROWS_TILING(4, 1, 16, false, float)
  HE_ROWS_NO_TILING;
}
