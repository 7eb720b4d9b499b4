// bf16 matrix product for few rows (M <= 32) with K cut inside the workgroup:
// C[M,N] = X[M,K] * W[N,K]^T (+ bias), or the gated activation of a gate||up
// weight. One workgroup owns up to 16*R weight rows (the rows are dealt out evenly over the
// compute units, see blocksplit_plan); its NW wavefronts take one K slice
// each (operands straight from global memory into the MFMA registers, in the operand
// layout gemm_rows.hip describes), leave their fp32
// tiles in LDS, and the workgroup adds the slices in wavefront order and writes
// the result. The sum is complete inside one launch: no partial sums in global
// memory, no second kernel, no atomics, and the order of the additions is fixed.
// With 16 wavefronts a product as small as 3584 x 3584 still puts 3584
// wavefronts on the chip.
//
// Gated epilogue: the weight alternates gate and up rows (gate i at row 2i, its up at
// 2i + 1), so the four neighbouring weight rows whose sums a thread holds are two
// (gate, up) pairs, and the output is silu(gate) * up, [M, N/2] (reference:
// kernels/activations.cu:183-198 as a kernel of its own).
//
// Two more epilogues carry an RMS norm across a pair of products without a kernel of
// its own (reference: kernels/fused_add_rmsnorm.cu:47-81 as a separate kernel):
//   residual: r[m][n] += acc (+ bias), stored fp32 in place; xg[m][n] = bf16(r * g[n]) with
//     the gain g of the norm that follows; and the sum of r^2 over the workgroup's columns
//     per row, one partial per workgroup: sq[m][block].
//   row scale: the consumer of xg adds the partials of a row in a fixed order,
//     s[m] = 1 / sqrt(sum / dim + eps), and multiplies its sums by s[m] before bias or
//     gate: W (r g s) = s W (r g). The norm's statistics stay fp32.
//
// Activations between two such products may lie piece-major instead of row-major: a [M, D]
// bf16 tensor as 16-byte pieces [D / 8][M][8], element (m, d) at ((d / 8) M + m) 8 + d % 8.
// The 16 lanes of an activation operand load then read 16 neighbouring pieces (two lines)
// instead of 16 rows (16 lines): the cost of the activation rows, which grows with their
// number (gate||up 48 us at 1 row, 50 at 8, 59 at 16), all but goes (49 and 55 us). The
// producing epilogue writes the layout, the consuming product reads it (x_pieces / out_pieces).
#include "common.h"
//
// The kernel is in gemm_blocksplit_tiles.h, its tilings are compiled in
// gemm_blocksplit_tiles_*.hip; this file has the rule that picks a tiling and the entry points.
#include "gemm_blocksplit_tiles.h"


// Tilings measured on MI355X (graph-timed sweeps over R, U and NW at the Qwen2.5-7B, Qwen2.5-32B
// and Qwen2-72B shapes). The rule depends on the sizes only, so a product always runs the same way.
// What counts is how many weight rows fall to a compute unit, so the bounds on N are written in
// rows a unit (on the MI355X's 256 units: 256 a unit = 65536 rows, the output head; 64 a unit =
// 16384, gate||up; 16 a unit = 4096); the bounds on K are lengths of a weight row.
static BlockSplitPlan blocksplit_plan(int M, int N, int K, int gated, int R, int U, int NW) {
  BlockSplitPlan p;
  const int cus = he_cus();
  p.MT = (M + 15) / 16;
  int r, u, nw;
  if (N >= 256 * cus) {             // 256 rows or more a unit: the output head
    if (M <= 8) r = 2, u = 1, nw = 8;
    else if (p.MT == 1) r = 4, u = 2, nw = 4;
    else r = 2, u = 2, nw = 4;
  } else if (K >= 8192) {           // long K
    const int groups = (N + 31) / 32, last_round = groups % cus;   // with two tiles a workgroup
    if (N < 16 * cus) {             // few weight rows: one tile a workgroup, or the chip is not filled
      r = 1, u = 1, nw = p.MT == 1 ? 8 : 4;
    } else if (p.MT == 2) {
      r = 2, u = 2, nw = 4;
    } else if (M > 8 && N >= 40 * cus) {
      r = 4, u = 2, nw = 4;         // the activation rows are read half as often
    } else if (groups < cus) {
      r = 2, u = 1, nw = 8;         // under one workgroup a compute unit: more wavefronts each
    } else if (groups < 4 * cus && last_round > 0 && last_round <= cus / 2) {
      r = 1, u = 1, nw = 8;         // the last round of whole tiles would fill under half of the chip:
                                    // the rows are dealt out below, 20 a workgroup for 10240
    } else if (K >= 16384) {
      r = 2, u = 2, nw = 8;         // 8192 x 29568 at 8 rows: 85.3 us against 89.2 us for the next line's tiling
    } else {
      r = 2, u = 4, nw = 4;
    }
  } else if (N >= 64 * cus) {       // wide N (gate||up)
    r = 2, u = 1, nw = 8;
    if (p.MT == 2 || K < 5120) u = 2, nw = 4;   // 37888 x 3584 at 8 rows: 47.7 us against 48.5 us
    else if (M > 8) r = 4;
  } else {                          // small products (q||k||v, o)
    r = N >= 16 * cus ? 2 : 1;
    u = p.MT == 1 && K < 5120 ? 4 : 1;   // 5120 x 5120 at 8 rows: 12.8 us unrolled once, 13.5 us four times
    nw = 8;
  }
  // Weight rows are dealt out evenly over the compute units (256 of them: or twice, three times ... 256
  // workgroups, at most 32 rows each) rather than in whole tiles of 16: 4608 rows as 256
  // workgroups of 18 rows instead of 144 of 32, the 37888 rows of gate||up as 1280 of 30
  // instead of 1184 of 32 (4.6 a compute unit). The last tile of such a workgroup is partly
  // empty. A workgroup's rows are an even number: a gate stays with its up, and outputs can be
  // stored in pairs. From two rows a unit on: the 896 rows of a small model's down projection as
  // 224 workgroups of 4 rather than 56 of 16 (896 x 4864 at 8 rows 9.5 -> 7.4 us, 1536 x 8960
  // 15.4 -> 12.5 us): a tile with four of its sixteen rows in use costs nothing that matters
  // there, a compute unit without work does.
  int rows = 0;
  if (R <= 0 && r <= 2 && N >= 2 * cus && N < 256 * cus) {
    const int rounds = (N + cus * 32 - 1) / (cus * 32);
    rows = ((N + cus * rounds - 1) / (cus * rounds) + 1) & ~1;
    r = rows > 16 ? 2 : 1;
  }
  p.R = R > 0 ? R : r;
  p.U = U > 0 ? U : u;
  if (NW <= 0) {
    NW = nw;
    while (NW > 1 && K / NW < 128) NW >>= 1;
  }
  if (NW > bs_max_waves(p.MT, p.R, p.U)) NW = bs_max_waves(p.MT, p.R, p.U);
  p.NW = NW;
  int ks = (K + NW - 1) / NW;
  p.kslice = (ks + 63) / 64 * 64;
  p.rows_per_block = rows > 0 ? rows : 16 * p.R;
  return p;
}

// Workgroups (= partial sums of squares per row) the residual epilogue of this product gives.
extern "C" int he_gemm_blocksplit_blocks(int M, int N, int K) {
  if (M <= 0 || M > HE_BLOCKSPLIT_MAX_M || N <= 0 || K <= 0) return 0;
  const BlockSplitPlan p = blocksplit_plan(M, N, K, 0, 0, 0, 0);
  return (N + p.rows_per_block - 1) / p.rows_per_block;
}

// R, U, NW <= 0 choose the heuristic tiling (NW wavefronts = K slices per workgroup).
// scale_partials: sums of squares of the input rows (the rows are then scaled before
// bias or gate); resid: the residual epilogue (C is not written; gain, xg, sq_out needed).
extern "C" int he_gemm_blocksplit_fused_bf16(void* C, const void* A, const void* W,
                                             const void* bias, int M, int N, int K, int out_dtype,
                                             int bias_dtype, int gated, int R, int U, int NW,
                                             const void* scale_partials, int scale_count,
                                             float scale_eps, void* resid, const void* gain,
                                             int gain_dtype, void* xg, void* sq_out,
                                             int sq_count, int x_pieces, int out_pieces,
                                             void* stream) {
  HE_REQUIRE(M > 0 && M <= HE_BLOCKSPLIT_MAX_M, "he_gemm_blocksplit_bf16: M=%d outside [1, %d]", M,
             HE_BLOCKSPLIT_MAX_M);
  HE_REQUIRE(N > 0 && K > 0, "he_gemm_blocksplit_bf16: bad sizes N=%d K=%d", N, K);
  HE_REQUIRE((K & 7) == 0, "he_gemm_blocksplit_bf16: K=%d must be a multiple of 8", K);
  HE_REQUIRE(out_dtype == HE_BF16 || out_dtype == HE_F32, "he_gemm_blocksplit_bf16: bad out dtype");
  HE_REQUIRE((((uintptr_t)A | (uintptr_t)W) & 15) == 0,
             "he_gemm_blocksplit_bf16: operands must be 16-byte aligned");
  HE_REQUIRE(!gated || ((N & 1) == 0 && bias == nullptr),
             "he_gemm_blocksplit_bf16: the gated epilogue needs an even N=%d and no bias", N);
  HE_REQUIRE(scale_partials == nullptr || scale_count > 0,
             "he_gemm_blocksplit_bf16: row scale without partial sums");
  HE_REQUIRE(!(x_pieces || out_pieces) || M <= 16,
             "he_gemm_blocksplit_bf16: piece-major activations are for up to 16 rows, not %d", M);
  HE_REQUIRE(!out_pieces || ((resid != nullptr || out_dtype == HE_BF16) && ((gated ? N / 2 : N) & 7) == 0),
             "he_gemm_blocksplit_bf16: a piece-major output is bf16 and a multiple of 8 wide");
  const BlockSplitPlan p = blocksplit_plan(M, N, K, gated, R, U, NW);
  HE_REQUIRE(p.NW >= 1 && p.NW <= 16, "he_gemm_blocksplit_bf16: %d wavefronts outside [1, 16]",
             p.NW);
  const int blocks = (N + p.rows_per_block - 1) / p.rows_per_block;
  if (resid != nullptr) {
    HE_REQUIRE(!gated && gain != nullptr && xg != nullptr && sq_out != nullptr,
               "he_gemm_blocksplit_bf16: the residual epilogue needs gain, xg and sq_out, and no gate");
    HE_REQUIRE(sq_count == blocks,
               "he_gemm_blocksplit_bf16: %d partial sums per row given, the product has %d workgroups",
               sq_count, blocks);
    HE_REQUIRE(gain_dtype == HE_F32 || gain_dtype == HE_BF16, "he_gemm_blocksplit_bf16: bad gain dtype");
  } else {
    HE_REQUIRE(C != nullptr, "he_gemm_blocksplit_bf16: no output");
  }
  BsFusion fu;
  fu.scale_partials = (const float*)scale_partials;
  fu.scale_count = scale_count;
  fu.scale_eps = scale_eps;
  fu.scale_dim = K;
  fu.resid = (float*)resid;
  fu.gain = gain;
  fu.gain_dtype = gain_dtype;
  fu.xg = (uint16_t*)xg;
  fu.sq_out = (float*)sq_out;
  fu.out_pieces = out_pieces;
  hipStream_t s = (hipStream_t)stream;
  int rc;
  static int (*const tiles[2][2])(HE_BS_DISPATCH_ARGS) = {
      {he_blocksplit_tiles_bf16, he_blocksplit_tiles_f32},
      {he_blocksplit_tiles_gated_bf16, he_blocksplit_tiles_gated_f32}};
  rc = tiles[gated != 0][out_dtype != HE_BF16](p, C, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s);
  if (rc) return rc;
  return he_check_launch("he_gemm_blocksplit_bf16");
}

extern "C" int he_gemm_blocksplit_bf16(void* C, const void* A, const void* W, const void* bias,
                                       int M, int N, int K, int out_dtype, int bias_dtype,
                                       int gated, int R, int U, int NW, void* stream) {
  return he_gemm_blocksplit_fused_bf16(C, A, W, bias, M, N, K, out_dtype, bias_dtype, gated, R, U,
                                       NW, nullptr, 0, 0.f, nullptr, nullptr, HE_F32, nullptr,
                                       nullptr, 0, 0, 0, stream);
}
