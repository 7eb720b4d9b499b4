// bf16 matrix product for 17 to 64 rows (one-token steps of larger batches):
// C[M,N] = X[M,K] * W[N,K]^T with the epilogues of gemm_blocksplit.hip (bias, gated
// SiLU x up, residual + rows for the next norm, owed row scale), where the reference calls
// its BLAS library (kernels/matmul_cublas.cu:240-277) and runs norm and activation as
// kernels of their own (kernels/fused_add_rmsnorm.cu, kernels/activations.cu:183-198).
//
// With more than 16 rows the activation rows cost as much to fetch as the weights when every
// wavefront fetches its own (gemm_blocksplit.hip). Here a workgroup's
// wavefronts all walk the same k range, each over 16 R weight rows of its own, so the
// activation rows of a k chunk are fetched once per workgroup: all threads copy the chunk
// [16 MT rows][128 k] into LDS, in the order of the MFMA's B operand (a wavefront's
// ds_read_b128 is one contiguous KiB), double-buffered with one barrier a chunk. The weights
// go straight from global memory into the A operand registers, the loads of the next chunk
// in flight while this one is multiplied. Operand layout of v_mfma_f32_16x16x32_bf16 as used here
// (the k slots of an instruction may hold any 8 k values as long as A and B agree):
//   A: lane l holds W[n0 + l % 16][k + 64 u + 16 (l / 16) + 8 h .. + 8]
//   B: lane l holds X[16 t + l % 16][the same k]
//   D: lane l holds D[n0 + 4 (l / 16) + i][16 t + l % 16], i = 0..3
//
// Products with few weight rows are also cut along K across workgroups (grid y): each slice
// leaves its fp32 sums [slices][M][N] and the reader adds them in slice order
// (he_splitk_reduce, he_splitk_reduce_residual): no atomics, a fixed order of additions.
//
// The kernel is in gemm_rows_tiles.h, its tilings are compiled in gemm_rows_tiles_*.hip; this
// file has the rule that picks a tiling, the entry points and the kernels that add the K slices.
#include "gemm_rows_tiles.h"

// Tilings measured on MI355X at the Qwen2.5-7B shapes; the rule depends on the sizes only, so a
// product always runs the same way. Wide products (gate||up, the output head) run in one K
// slice, their weight rows dealt out evenly over the workgroups the chip holds at once (two
// a compute unit: 37888 rows as 499 workgroups of 76, the last three of whose eight wavefronts
// only help to copy the activation rows; not 296 of 128, of which 40 would run after the
// others; above 32 rows one workgroup of sixteen wavefronts a compute unit); narrow ones are cut along K until the grid holds about a workgroup a compute unit.
static RowsPlan rows_plan(int M, int N, int K, int R, int NWV, int splits) {
  RowsPlan p;
  const int cus = he_cus();   // the bounds on N are weight rows a compute unit (256 units: 65536, 16384, 4096 rows)
  p.MT = M <= 32 ? 2 : 4;
  if (R <= 0 || NWV <= 0) {
    if (N >= 256 * cus) R = p.MT == 4 ? 1 : 2, NWV = p.MT == 4 ? 16 : 8;   // the output head (at 64 rows 223.6 -> 216.2 us)
    else if (N >= 64 * cus) R = 1, NWV = p.MT == 4 ? 16 : 8;  // gate||up: at 33 to 64 rows one workgroup a compute
                                                           // unit, so that the unit fetches the activation rows
                                                           // once, not twice (gate||up at 64 rows 61.1 -> 57.2 us;
                                                           // without that copying it takes 53.6)
    else R = 1, NWV = (K >= 8192 || N >= 16 * cus) ? 8 : 4;
  }
  p.R = R;
  p.NWV = NWV;
  const int cap = 16 * R * NWV;
  int rows = cap;
  if (N >= 64 * cus && splits <= 1) {
    // dealt out evenly over the workgroups the chip holds at once: one a compute unit where a workgroup
    // has 256 rows (the head; sixteen wavefronts), two otherwise
    const int slots = cus * ((R == 2 && NWV == 8) || NWV == 16 ? 1 : 2);
    const int rounds = (N + slots * cap - 1) / (slots * cap);
    rows = ((N + slots * rounds - 1) / (slots * rounds) + 3) & ~3;
    if (rows > cap) rows = cap;
  }
  p.rows_per_block = rows;
  p.groups = (N + p.rows_per_block - 1) / p.rows_per_block;
  int s = splits;
  if (s <= 0) {
    s = 1;
    // 192 workgroups on 256 units, slices of four chunks or more (q||k||v of 4608 x 3584 at 64 rows: 36 groups
    // in 7 slices of 512 take 15.9 us with their sum, in 4 slices of 896 17.8 us)
    while (p.groups * s < cus * 3 / 4 && K / (2 * s) >= 256 && s < 32) s *= 2;
  }
  int ks = (K + s - 1) / s;
  ks = (ks + ROWS_KC - 1) / ROWS_KC * ROWS_KC;
  p.kslice = ks;
  p.splits = (K + ks - 1) / ks;
  return p;
}

extern "C" int he_gemm_rows_plan(int M, int N, int K, int* groups, int* splits) {
  if (M <= 0 || M > HE_GEMM_ROWS_MAX_M || N <= 0 || K <= 0) return -1;
  const RowsPlan p = rows_plan(M, N, K, 0, 0, 0);
  if (groups) *groups = p.groups;
  if (splits) *splits = p.splits;
  return 0;
}

extern "C" int he_gemm_rows_bf16(void* C, void* partial_f32, int64_t partial_floats, const void* A,
                                 const void* W, const void* bias, int M, int N, int K, int out_dtype,
                                 int bias_dtype, int gated, int R, int NWV, int splits,
                                 const void* scale_partials, int scale_count, float scale_eps,
                                 void* resid, const void* gain, int gain_dtype, void* xg, void* sq_out,
                                 int sq_count, int x_pieces, int out_pieces, int* splits_used,
                                 void* stream) {
  HE_REQUIRE(M > 0 && M <= HE_GEMM_ROWS_MAX_M, "he_gemm_rows_bf16: M=%d outside [1, %d]", M,
             HE_GEMM_ROWS_MAX_M);
  HE_REQUIRE(N > 0 && K > 0, "he_gemm_rows_bf16: bad sizes N=%d K=%d", N, K);
  HE_REQUIRE((K & 7) == 0, "he_gemm_rows_bf16: K=%d must be a multiple of 8", K);
  HE_REQUIRE(out_dtype == HE_BF16 || out_dtype == HE_F32, "he_gemm_rows_bf16: bad out dtype");
  HE_REQUIRE((((uintptr_t)A | (uintptr_t)W) & 15) == 0, "he_gemm_rows_bf16: operands must be 16-byte aligned");
  HE_REQUIRE(!gated || ((N & 1) == 0 && bias == nullptr),
             "he_gemm_rows_bf16: the gated epilogue needs an even N=%d and no bias", N);
  HE_REQUIRE(scale_partials == nullptr || scale_count > 0, "he_gemm_rows_bf16: row scale without partial sums");
  HE_REQUIRE(!out_pieces || ((resid != nullptr || out_dtype == HE_BF16) && ((gated ? N / 2 : N) & 7) == 0),
             "he_gemm_rows_bf16: a piece-major output is bf16 and a multiple of 8 wide");
  HE_REQUIRE(R <= 0 || R == 1 || R == 2, "he_gemm_rows_bf16: R=%d is not 1 or 2", R);
  HE_REQUIRE(NWV <= 0 || NWV == 4 || NWV == 8 || NWV == 16, "he_gemm_rows_bf16: %d wavefronts, not 4, 8 or 16", NWV);
  HE_REQUIRE((R <= 0) == (NWV <= 0), "he_gemm_rows_bf16: give both R and NWV, or neither");
  HE_REQUIRE(!(R == 2 && NWV == 4) || M > 32,
             "he_gemm_rows_bf16: two tiles a wavefront in four wavefronts are for more than 32 rows");
  const RowsPlan p = rows_plan(M, N, K, R, NWV, splits);
  HE_REQUIRE(p.groups <= 0x7fffffff && p.splits >= 1 && p.splits <= 65535, "he_gemm_rows_bf16: grid too large");
  if (splits_used) *splits_used = p.splits;
  const bool epilogue = gated || resid != nullptr || out_pieces || bias != nullptr;
  if (p.splits > 1) {
    HE_REQUIRE(!epilogue, "he_gemm_rows_bf16: a product cut into %d K slices leaves plain partial sums; "
               "bias and the gated, residual and piece-major epilogues need one slice", p.splits);
    const int64_t need = (int64_t)p.splits * M * N;
    HE_REQUIRE(partial_f32 != nullptr && partial_floats >= need && (((uintptr_t)partial_f32) & 15) == 0,
               "he_gemm_rows_bf16: room for %lld partial sums, need %lld (16-byte aligned)",
               (long long)partial_floats, (long long)need);
  } else if (resid != nullptr) {
    HE_REQUIRE(!gated && gain != nullptr && xg != nullptr && sq_out != nullptr,
               "he_gemm_rows_bf16: the residual epilogue needs gain, xg and sq_out, and no gate");
    HE_REQUIRE(sq_count == p.groups, "he_gemm_rows_bf16: %d partial sums per row given, the product has %d workgroups",
               sq_count, p.groups);
    HE_REQUIRE(gain_dtype == HE_F32 || gain_dtype == HE_BF16, "he_gemm_rows_bf16: bad gain dtype");
  } else {
    HE_REQUIRE(C != nullptr, "he_gemm_rows_bf16: no output");
  }
  RowsFusion fu;
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
  float* partial = (float*)partial_f32;
  int rc;
  HE_REQUIRE(!gated || out_dtype == HE_BF16, "he_gemm_rows_bf16: the gated epilogue writes bfloat16");
  const int kind = gated ? 2 : out_dtype == HE_F32;
  static int (*const tiles[2][3])(HE_ROWS_DISPATCH_ARGS) = {
      {he_rows_tiles2_bf16, he_rows_tiles2_f32, he_rows_tiles2_gated},
      {he_rows_tiles4_bf16, he_rows_tiles4_f32, he_rows_tiles4_gated}};
  rc = tiles[p.MT == 4][kind](p, C, partial, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s);
  if (rc) return rc;
  return he_check_launch("he_gemm_rows_bf16");
}

// ---- the K slices of a product into a tensor -----------------------------------------
// out[m][n] = sum_s partial[s][m][n] (+ bias[n]), slices added in index order. Four neighbouring
// elements a thread where the width allows it; the loads of up to eight slices go out together
// before the first is added (a loop over the slices would wait for each in turn).
template <typename TC, int VEC>
__global__ void splitk_reduce_kernel(TC* __restrict__ C, const float* __restrict__ partial,
                                     const void* __restrict__ bias, int bias_dtype, int64_t total,
                                     int N, int splits) {
  const int64_t i = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * VEC;
  if (i >= total) return;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float v[8][VEC];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int sp = min(s0 + j, splits - 1);
      if (VEC == 4) {
        const float4 f = *reinterpret_cast<const float4*>(partial + sp * total + i);
        v[j][0] = f.x, v[j][1] = f.y, v[j][2] = f.z, v[j][3] = f.w;
      } else {
        v[j][0] = partial[sp * total + i];
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s0 + j < splits)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += v[j][e];
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e)
    if (bias != nullptr) acc[e] += load_param(bias, (i + e) % N, bias_dtype);
  if constexpr (VEC == 4) {
    rows_store4<TC>(C + i, acc, 4, 4);
  } else {
    C[i] = from_float<TC>(acc[0]);
  }
}

extern "C" int he_splitk_reduce(void* C, const void* partial_f32, const void* bias, int M, int N,
                                int splits, int out_dtype, int bias_dtype, void* stream) {
  HE_REQUIRE(M >= 0 && N > 0 && splits > 0, "he_splitk_reduce: bad sizes");
  HE_REQUIRE(out_dtype == HE_BF16 || out_dtype == HE_F32, "he_splitk_reduce: unknown dtype %d", out_dtype);
  if (M == 0) return 0;
  const int64_t total = (int64_t)M * N;
  const bool vec = (total & 3) == 0 && ((((uintptr_t)partial_f32) | ((uintptr_t)C)) & 15) == 0;
  const int64_t items = vec ? total / 4 : total;
  HE_REQUIRE((items + 255) / 256 <= 0x7fffffff, "he_splitk_reduce: too many elements for one launch");
  const unsigned blocks = (unsigned)((items + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
#define REDUCE(TC_, VEC_)                                                                        \
  splitk_reduce_kernel<TC_, VEC_><<<blocks, 256, 0, s>>>((TC_*)C, (const float*)partial_f32, bias, \
                                                         bias_dtype, total, N, splits)
  if (out_dtype == HE_BF16) {
    if (vec) REDUCE(bf16_t, 4); else REDUCE(bf16_t, 1);
  } else {
    if (vec) REDUCE(float, 4); else REDUCE(float, 1);
  }
#undef REDUCE
  return he_check_launch("he_splitk_reduce");
}

// ---- the K slices of a product into the residual stream -------------------------------
// resid[m][n] += sum_s partial[s][m][n] (+ bias[n]), slices in index order; xg[m][n] =
// bf16(resid * gain[n]) (row-major, or piece-major); sq[m][block] = the sum of resid^2 over the
// block's columns: what the residual epilogue of a one-slice product leaves (rows for the next
// norm, whose scale the next product applies). grid (column blocks of 1024, rows), 256 threads.
__global__ __launch_bounds__(256) void splitk_reduce_residual_kernel(
    float* __restrict__ resid, const float* __restrict__ partial, const void* __restrict__ bias,
    int bias_dtype, const void* __restrict__ gain, int gain_dtype, uint16_t* __restrict__ xg,
    float* __restrict__ sq_out, int M, int N, int splits, int out_pieces) {
  __shared__ float red[4];
  const int m = blockIdx.y;
  const int n = blockIdx.x * 1024 + 4 * threadIdx.x;
  float sq = 0.f;
  if (n < N) {
    const int valid = min(4, N - n);
    const int64_t at = (int64_t)m * N + n;
    const bool vec = valid == 4 && (N & 3) == 0;
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {
      const float4 r4 = *reinterpret_cast<const float4*>(resid + at);
      x[0] = r4.x, x[1] = r4.y, x[2] = r4.z, x[3] = r4.w;
    } else {
      for (int i = 0; i < valid; ++i) x[i] = resid[at + i];
    }
    float d[4] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {     // the loads of up to eight slices go out together, then they are added in order
      for (int s0 = 0; s0 < splits; s0 += 8) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          v[j] = *reinterpret_cast<const float4*>(partial + (int64_t)min(s0 + j, splits - 1) * M * N + at);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (s0 + j < splits) d[0] += v[j].x, d[1] += v[j].y, d[2] += v[j].z, d[3] += v[j].w;
      }
    } else {
      for (int s = 0; s < splits; ++s) {
        const float* p = partial + (int64_t)s * M * N + at;
        for (int i = 0; i < valid; ++i) d[i] += p[i];
      }
    }
    float g[4];
    for (int i = 0; i < 4; ++i) {
      const bool in = i < valid;
      if (in && bias != nullptr) d[i] += load_param(bias, n + i, bias_dtype);
      x[i] += d[i];
      g[i] = in ? x[i] * load_param(gain, n + i, gain_dtype) : 0.f;
      if (in) sq += x[i] * x[i];
    }
    if (vec) {
      *reinterpret_cast<float4*>(resid + at) = make_float4(x[0], x[1], x[2], x[3]);
    } else {
      for (int i = 0; i < valid; ++i) resid[at + i] = x[i];
    }
    if (out_pieces) {
      rows_store_pieces(xg, M, m, n, g, 4, valid);
    } else if (vec) {
      *reinterpret_cast<uint2*>(xg + at) = make_uint2(pack2_bf16(g[0], g[1]), pack2_bf16(g[2], g[3]));
    } else {
      for (int i = 0; i < valid; ++i) xg[at + i] = float_to_bf16_bits(g[i]);
    }
  }
  sq = wave_sum(sq);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sq;
  __syncthreads();
  if (threadIdx.x == 0) sq_out[(int64_t)m * gridDim.x + blockIdx.x] = ((red[0] + red[1]) + red[2]) + red[3];
}

extern "C" int he_splitk_reduce_residual_blocks(int N) { return N > 0 ? (N + 1023) / 1024 : 0; }

extern "C" int he_splitk_reduce_residual(void* resid_f32, const void* partial_f32, const void* bias,
                                         int bias_dtype, const void* gain, int gain_dtype, void* xg,
                                         void* sq_out, int sq_count, int M, int N, int splits,
                                         int out_pieces, void* stream) {
  HE_REQUIRE(M >= 0 && M <= 65535 && N > 0 && splits > 0, "he_splitk_reduce_residual: bad sizes");
  HE_REQUIRE(resid_f32 && partial_f32 && gain && xg && sq_out, "he_splitk_reduce_residual: missing buffers");
  HE_REQUIRE(sq_count == he_splitk_reduce_residual_blocks(N),
             "he_splitk_reduce_residual: %d partial sums per row given, %d column blocks", sq_count,
             he_splitk_reduce_residual_blocks(N));
  HE_REQUIRE(!out_pieces || (N & 7) == 0, "he_splitk_reduce_residual: a piece-major output is a multiple of 8 wide");
  HE_REQUIRE((((uintptr_t)resid_f32 | (uintptr_t)partial_f32) & 15) == 0 && (((uintptr_t)xg) & 7) == 0,
             "he_splitk_reduce_residual: buffers must be 16-byte aligned");
  if (M == 0) return 0;
  splitk_reduce_residual_kernel<<<dim3(sq_count, M), 256, 0, (hipStream_t)stream>>>(
      (float*)resid_f32, (const float*)partial_f32, bias, bias_dtype, gain, gain_dtype, (uint16_t*)xg,
      (float*)sq_out, M, N, splits, out_pieces);
  return he_check_launch("he_splitk_reduce_residual");
}
