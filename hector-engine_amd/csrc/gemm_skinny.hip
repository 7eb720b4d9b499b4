// bf16 matrix product for few rows (M <= 64): C[M,N] = X[M,K] * W[N,K]^T (+ bias),
// fp32 accumulation on the matrix cores, every weight element read from HBM
// exactly once for all M rows. It replaces the M = 1 BLAS call of the
// reference's decode step (kernels/linear.cu:24-30, kernels/matmul_cublas.cu:240-277).
//
// The product is computed transposed, D[n][m] = sum_k W[n][k] X[m][k], with
// v_mfma_f32_16x16x32_bf16: W supplies the A operand (16 rows n), X the B
// operand (16 columns m). One wavefront owns 16*R weight rows over one K slice
// and all M rows; it loads both operands straight from global memory into the
// operand registers (weights are used once, so there is nothing to stage;
// X is small and stays in L2). Operand layout of the instruction:
//   A: lane l holds A[l % 16][8 * (l / 16) .. +8)      (8 consecutive k)
//   B: lane l holds B[8 * (l / 16) .. +8)[l % 16]
//   D: lane l holds D[4 * (l / 16) + i][l % 16], i = 0..3
// The k slots of an instruction may hold any 8 k values as long as A and B
// agree, so a lane takes 16 consecutive k (32 contiguous bytes of a weight row)
// for two instructions: the four lanes of a row then read 128 contiguous bytes.
//
// K is cut into `splits` slices when there are too few row tiles to fill the
// chip. Every slice then writes its fp32 partial sums [splits][M][N]; they are
// added, in the order of the slice index, by whichever kernel reads the result
// next (the fused norm, the q/k/v kernel) or by he_splitk_reduce. No
// floating-point atomics and no device-wide fences: a fence that makes one
// XCD's writes visible to another costs more than the product itself.
//
// Epilogue: bias.
#include "common.h"
#include "hector_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

struct SkinnyPlan {
  int MT;       // 16-row tiles of M
  int R;        // 16-row tiles of N per wavefront
  int U;        // 64-wide k steps whose loads are issued together
  int ntiles;   // wavefront tiles along N
  int splits;   // K slices
  int kslice;   // K per slice, multiple of 64
};

static void finish_plan(SkinnyPlan& p, int N, int K, int splits_wanted) {
  p.ntiles = (N + 16 * p.R - 1) / (16 * p.R);
  int s = splits_wanted;
  if (s <= 0) {
    const int target_waves = 256 * 12;
    s = (target_waves + p.ntiles - 1) / p.ntiles;
    const int max_s = K / 512 > 0 ? K / 512 : 1;
    if (s > max_s) s = max_s;
  }
  if (s < 1) s = 1;
  if (s > 64) s = 64;
  int ks = (K + s - 1) / s;
  ks = (ks + 63) / 64 * 64;
  p.kslice = ks;
  p.splits = (K + ks - 1) / ks;
}

// Tilings measured on MI355X (graph-timed sweeps over R, U and the slice count at
// the Qwen2.5-7B shapes); the rule depends on the sizes only, so a product always
// runs the same way.
static SkinnyPlan skinny_plan(int M, int N, int K) {
  SkinnyPlan p;
  p.MT = (M + 15) / 16;
  if (p.MT >= 3) p.MT = 4;
  int splits;
  if (N >= 65536) {          // output head: plenty of row tiles, one slice
    p.R = p.MT == 4 ? 4 : 2;
    p.U = p.MT == 1 && M <= 8 ? 4 : (p.MT == 4 ? 1 : 2);
    splits = 1;
  } else if (K >= 8192) {           // long K (down projection)
    p.R = p.MT == 1 ? 2 : 4;
    p.U = p.MT == 1 ? 2 : 1;
    splits = p.MT == 1 ? 8 : 16;
  } else if (N >= 16384) {          // wide N (gate||up)
    p.R = p.MT == 1 ? (M <= 8 ? 1 : 2) : 4;
    p.U = p.MT == 1 && M <= 8 ? 2 : 1;
    splits = p.MT == 1 ? (M <= 8 ? 2 : 4) : 8;
  } else {                          // small products (q||k||v, o)
    p.R = p.MT == 1 ? (M <= 8 ? 1 : 2) : (p.MT == 2 ? 2 : 4);
    p.U = p.MT == 1 && M <= 8 ? 2 : 1;
    splits = K >= 2048 ? (p.MT == 1 ? 8 : 16) : (K >= 1024 ? 4 : (K >= 512 ? 2 : 1));
  }
  finish_plan(p, N, K, splits);
  return p;
}

__device__ __forceinline__ bf16x8 load8(const uint16_t* p, bool ok) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if (ok) v = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, v);
}

template <typename TC>
__device__ __forceinline__ void store4(TC* p, const float v[4], bool vec, int valid);
template <>
__device__ __forceinline__ void store4<float>(float* p, const float v[4], bool vec, int valid) {
  if (vec && valid == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    for (int i = 0; i < valid; ++i) p[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, const float v[4], bool vec, int valid) {
  if (vec && valid == 4) {
    uint2 w;
    w.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
    w.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = w;
  } else {
    for (int i = 0; i < valid; ++i) p[i].v = float_to_bf16_bits(v[i]);
  }
}

template <int MT, int R, int U, typename TC>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(
    TC* __restrict__ C, float* __restrict__ partial, const uint16_t* __restrict__ X, const uint16_t* __restrict__ W,
    const void* __restrict__ bias, int bias_dtype, int M, int N, int K, int ntiles, int splits,
    int kslice) {
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (gw >= ntiles * splits) return;
  const int tile = gw % ntiles;
  const int split = gw / ntiles;
  const int n0 = tile * 16 * R;
  const int k_begin = split * kslice;
  const int k_end = min(K, k_begin + kslice);
  const int lr = lane & 15, lg = lane >> 4;

  const uint16_t* wp[R];
  const uint16_t* xp[MT];
#pragma unroll
  for (int r = 0; r < R; ++r) wp[r] = W + (int64_t)min(n0 + 16 * r + lr, N - 1) * K + lg * 16;
#pragma unroll
  for (int t = 0; t < MT; ++t) xp[t] = X + (int64_t)min(16 * t + lr, M - 1) * K + lg * 16;

  floatx4 acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int k = k_begin; k < k_end; k += 64 * U) {
    bf16x8 a[U][R][2], b[U][MT][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k + 64 * u + lg * 16;   // this lane's 16 k values of the step
      const bool ok0 = kk + 8 <= k_end, ok1 = kk + 16 <= k_end;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        a[u][r][0] = load8(wp[r] + k + 64 * u, ok0);
        a[u][r][1] = load8(wp[r] + k + 64 * u + 8, ok1);
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        b[u][t][0] = load8(xp[t] + k + 64 * u, ok0);
        b[u][t][1] = load8(xp[t] + k + 64 * u + 8, ok1);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int t = 0; t < MT; ++t)
            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][r][h], b[u][t][h], acc[r][t],
                                                                0, 0, 0);
  }

  // acc[r][t][i] = D[n0 + 16r + 4lg + i][16t + lr]
  const bool vec = (N & 3) == 0;
  if (splits > 1) {
    // ---- this slice's partial sums; whoever reads the result adds the slices in order
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = n0 + 16 * r + 4 * lg;
      const int valid = min(4, N - n);
      if (valid <= 0) continue;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + lr;
        if (m >= M) continue;
        const float v[4] = {acc[r][t][0], acc[r][t][1], acc[r][t][2], acc[r][t][3]};
        store4<float>(partial + ((int64_t)split * M + m) * N + n, v, vec, valid);
      }
    }
    return;
  }

#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = n0 + 16 * r + 4 * lg;
    const int valid = min(4, N - n);
    if (valid <= 0) continue;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = 16 * t + lr;
      if (m >= M) continue;
      float v[4] = {acc[r][t][0], acc[r][t][1], acc[r][t][2], acc[r][t][3]};
      if (bias != nullptr)
        for (int i = 0; i < valid; ++i) v[i] += load_param(bias, n + i, bias_dtype);
      store4<TC>(C + (int64_t)m * N + n, v, vec, valid);
    }
  }
}

// out[m][n] = sum_s partial[s][m][n] (+ bias[n]), slices added in index order.
template <typename TC>
__global__ void splitk_reduce_kernel(TC* __restrict__ C, const float* __restrict__ partial,
                                     const void* __restrict__ bias, int bias_dtype, int64_t total,
                                     int N, int splits) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    float s = 0.f;
    for (int sp = 0; sp < splits; ++sp) s += partial[sp * total + i];
    if (bias != nullptr) s += load_param(bias, i % N, bias_dtype);
    C[i] = from_float<TC>(s);
  }
}

extern "C" int he_splitk_reduce(void* C, const void* partial_f32, const void* bias, int M, int N,
                                int splits, int out_dtype, int bias_dtype, void* stream) {
  HE_REQUIRE(M >= 0 && N > 0 && splits > 0, "he_splitk_reduce: bad sizes");
  if (M == 0) return 0;
  const int64_t total = (int64_t)M * N;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 4096) blocks = 4096;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == HE_BF16)
    splitk_reduce_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)C, (const float*)partial_f32, bias,
                                                        bias_dtype, total, N, splits);
  else if (out_dtype == HE_F32)
    splitk_reduce_kernel<float><<<blocks, 256, 0, s>>>((float*)C, (const float*)partial_f32, bias,
                                                       bias_dtype, total, N, splits);
  else
    HE_REQUIRE(false, "he_splitk_reduce: unknown dtype %d", out_dtype);
  return he_check_launch("he_splitk_reduce");
}

template <int MT, int R, int U, typename TC>
static void launch_skinny(const SkinnyPlan& p, void* C, float* partial, const void* X,
                          const void* W, const void* bias, int bias_dtype, int M, int N, int K,
                          hipStream_t s) {
  const int waves = p.ntiles * p.splits;
  gemm_skinny_kernel<MT, R, U, TC><<<(waves + 3) / 4, 256, 0, s>>>(
      (TC*)C, partial, (const uint16_t*)X, (const uint16_t*)W, bias, bias_dtype, M, N, K, p.ntiles,
      p.splits, p.kslice);
}

template <typename TC>
static int dispatch_skinny(const SkinnyPlan& p, void* C, float* partial, const void* X,
                           const void* W, const void* bias, int bias_dtype, int M, int N, int K,
                           hipStream_t s) {
#define SK(MT_, R_, U_)                                                                 \
  if (p.MT == MT_ && p.R == R_ && p.U == U_) {                                          \
    launch_skinny<MT_, R_, U_, TC>(p, C, partial, X, W, bias, bias_dtype, M, N, K, s); \
    return 0;                                                                           \
  }
  SK(1, 1, 1) SK(1, 1, 2) SK(1, 1, 4)
  SK(1, 2, 1) SK(1, 2, 2) SK(1, 2, 4) SK(2, 2, 1) SK(2, 2, 2) SK(4, 4, 1) SK(4, 2, 1) SK(4, 2, 2)
  SK(1, 4, 1) SK(1, 4, 2) SK(2, 4, 1) SK(2, 4, 2)
#undef SK
  he_set_error("he_gemm_skinny_bf16: no kernel for MT=%d R=%d U=%d", p.MT, p.R, p.U);
  return -1;
}

static int check_skinny(const void* A, const void* W, const void* bias, int M, int N, int K,
                        int out_dtype) {
  HE_REQUIRE(M > 0 && M <= HE_SKINNY_MAX_M, "he_gemm_skinny_bf16: M=%d outside [1, %d]", M,
             HE_SKINNY_MAX_M);
  HE_REQUIRE(N > 0 && K > 0, "he_gemm_skinny_bf16: bad sizes N=%d K=%d", N, K);
  HE_REQUIRE((K & 7) == 0, "he_gemm_skinny_bf16: K=%d must be a multiple of 8", K);
  HE_REQUIRE(out_dtype == HE_BF16 || out_dtype == HE_F32, "he_gemm_skinny_bf16: bad out dtype");
  HE_REQUIRE((((uintptr_t)A | (uintptr_t)W) & 15) == 0,
             "he_gemm_skinny_bf16: operands must be 16-byte aligned");
  return 0;
}

// Number of K slices the heuristic cuts this product into (1 = none).
extern "C" int he_gemm_skinny_splits(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 1;
  return skinny_plan(M, N, K).splits;
}

// R, U <= 0: the heuristic tiling. splits <= 0: the heuristic's slice count.
// With more than one slice, C is ignored and `partial_f32` receives
// [slices][M][N] fp32 sums; *splits_used tells how many slices were written.
extern "C" int he_gemm_skinny_bf16(void* C, void* partial_f32, int64_t partial_floats,
                                   const void* A, const void* W, const void* bias, int M, int N,
                                   int K, int out_dtype, int bias_dtype, int R, int U,
                                   int splits, int* splits_used, void* stream) {
  if (int rc = check_skinny(A, W, bias, M, N, K, out_dtype)) return rc;
  SkinnyPlan p = skinny_plan(M, N, K);
  if (R > 0) p.R = R;
  if (U > 0) p.U = U;
  if (R > 0 || U > 0 || splits > 0) finish_plan(p, N, K, splits);
  const int64_t need = p.splits > 1 ? (int64_t)p.splits * M * N : 0;
  HE_REQUIRE(partial_floats >= need && (need == 0 || partial_f32 != nullptr),
             "he_gemm_skinny_bf16: room for %lld partial sums, need %lld",
             (long long)partial_floats, (long long)need);
  HE_REQUIRE(need == 0 || (((uintptr_t)partial_f32) & 15) == 0,
             "he_gemm_skinny_bf16: the partial sums must be 16-byte aligned");
  if (splits_used) *splits_used = p.splits;
  hipStream_t s = (hipStream_t)stream;
  float* partial = (float*)partial_f32;
  int rc;
  rc = out_dtype == HE_BF16
           ? dispatch_skinny<bf16_t>(p, C, partial, A, W, bias, bias_dtype, M, N, K, s)
           : dispatch_skinny<float>(p, C, partial, A, W, bias, bias_dtype, M, N, K, s);
  if (rc) return rc;
  return he_check_launch("he_gemm_skinny_bf16");
}
