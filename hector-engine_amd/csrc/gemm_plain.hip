// Plain matrix product  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N])  with fp32 FMA accumulation
// in one fixed order per output element, whatever M and whichever rows share the launch, so
// a row's result never depends on the batch it is in or on how the step was cut. It is the
// true 32-bit path of every linear layer and the reference beside the MFMA kernels.
// Weight layout [N, K] row-major as in the reference (kernels/register_kernels.cpp:373-386).
//
// The order: K is cut into segments of GP_SEG (128) consecutive k. The sum of a segment is one
// chain of FMAs over its k in ascending order, begun at zero; the element is the segment
// sums added one after the other in segment order, begun at zero; then the bias.
// Three kernels keep this order and give the same bits:
//   tiles   64 x 64 outputs a workgroup, staged through LDS, every thread 4 x 4 outputs
//           (128 x 128 and 8 x 8 for fp32 steps of 128 rows or more);
//   rows    for up to GP_ROWS_MAX_M rows (the one-token steps): a thread owns one weight
//           row and one segment and walks it with all M activation rows at once, so a product
//           has N * ceil(K / GP_SEG) threads however few its rows are; the segment sums go
//           to a workspace and a second kernel adds them in order. (With few rows the tile
//           kernel is a grid of N / 64 workgroups walking all of K one after the other:
//           the Qwen2.5-7B shape's one-token step took 190 ms with it.)
// No multiply and add of this file is fused unless it is written as an fma: the same lines are
// compiled into several kernels that must give the same bits.
#pragma clang fp contract(off)
#include "common.h"
#include "hector_kernels.h"

#define GP_BM 64
#define GP_BN 64
#define GP_BK 16
#define GP_SEG 128          // a multiple of GP_BK
#define GP_ROWS_MAX_M 8

template <typename TA, typename TW, typename TC>
// (six wavefronts a SIMD, as without the segment totals: left alone the compiler takes registers for four)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(6, 8))) void gemm_plain_kernel(
    TC* __restrict__ C, const TA* __restrict__ A, const TW* __restrict__ W,
    const void* __restrict__ bias, int bias_dtype, int M, int N, int K, int64_t lda, int64_t ldw,
    int64_t ldc) {
  __shared__ float As[GP_BK][GP_BM + 1];
  __shared__ float Ws[GP_BK][GP_BN + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15;  // along N
  const int ty = tid >> 4;  // along M
  const int m0 = blockIdx.y * GP_BM;
  const int n0 = blockIdx.x * GP_BN;
  const int lrow = tid >> 2;       // 0..63
  const int lk = (tid & 3) * 4;    // 0,4,8,12
  float acc[4][4], total[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f, total[i][j] = 0.f;

  // a tile that lies inside both matrices is fetched four values a load
  const bool a_vec = sizeof(TA) == 4 && m0 + GP_BM <= M && (lda & 3) == 0 && (((uintptr_t)A) & 15) == 0;
  const bool w_vec = sizeof(TW) == 4 && n0 + GP_BN <= N && (ldw & 3) == 0 && (((uintptr_t)W) & 15) == 0;
  for (int k0 = 0; k0 < K; k0 += GP_BK) {
    const bool whole = k0 + GP_BK <= K;
    const int am = m0 + lrow, wn = n0 + lrow;
    if (a_vec && whole) {
      const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(A) + am * lda + k0 + lk);
      As[lk][lrow] = v.x, As[lk + 1][lrow] = v.y, As[lk + 2][lrow] = v.z, As[lk + 3][lrow] = v.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = k0 + lk + j;
        As[lk + j][lrow] = (am < M && k < K) ? to_float(A[am * lda + k]) : 0.f;
      }
    }
    if (w_vec && whole) {
      const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(W) + wn * ldw + k0 + lk);
      Ws[lk][lrow] = v.x, Ws[lk + 1][lrow] = v.y, Ws[lk + 2][lrow] = v.z, Ws[lk + 3][lrow] = v.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = k0 + lk + j;
        Ws[lk + j][lrow] = (wn < N && k < K) ? to_float(W[wn * ldw + k]) : 0.f;
      }
    }
    __syncthreads();
    // the chain of a segment holds its own k only: the last tile of K may be short
#define GP_TILE_STEP(kk)                                                     \
  {                                                                          \
    float a[4], b[4];                                                        \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i]; \
    _Pragma("unroll") for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j]; \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                            \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]); \
  }
    if (k0 + GP_BK <= K) {
#pragma unroll
      for (int kk = 0; kk < GP_BK; ++kk) GP_TILE_STEP(kk)
    } else {
      for (int kk = 0; kk < K - k0; ++kk) GP_TILE_STEP(kk)
    }
#undef GP_TILE_STEP
    __syncthreads();
    if ((k0 + GP_BK) % GP_SEG == 0 || k0 + GP_BK >= K) {   // the segment ends here
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) total[i][j] += acc[i][j], acc[i][j] = 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = total[i][j];
      if (bias != nullptr) v += load_param(bias, n, bias_dtype);
      C[m * ldc + n] = from_float<TC>(v);
    }
  }
}

// The same product and order in tiles of 128 x 128 outputs, every thread 8 x 8 of them (two
// groups of four rows by two groups of four columns, 64 apart, so that the operand reads from LDS
// are whole 16-byte reads of neighbouring lanes): four times the products per LDS read of the
// 64 x 64 kernel. For fp32 operands and steps of 128 rows or more (whole prompts).
#define GPW_BM 128
#define GPW_BN 128
__global__ __launch_bounds__(256) void gemm_plain_wide_kernel(
    float* __restrict__ C, const float* __restrict__ A, const float* __restrict__ W,
    const void* __restrict__ bias, int bias_dtype, int M, int N, int K, int64_t lda, int64_t ldw,
    int64_t ldc) {
  __shared__ __attribute__((aligned(16))) float As[GP_BK][GPW_BM + 4];
  __shared__ __attribute__((aligned(16))) float Ws[GP_BK][GPW_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15;  // along N
  const int ty = tid >> 4;  // along M
  const int m0 = blockIdx.y * GPW_BM;
  const int n0 = blockIdx.x * GPW_BN;
  const int lrow = tid >> 2;       // 0..63 (and + 64)
  const int lk = (tid & 3) * 4;    // 0,4,8,12
  float acc[8][8], total[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.f, total[i][j] = 0.f;
  const bool a_vec = m0 + GPW_BM <= M && (lda & 3) == 0 && (((uintptr_t)A) & 15) == 0;
  const bool w_vec = n0 + GPW_BN <= N && (ldw & 3) == 0 && (((uintptr_t)W) & 15) == 0;
  for (int k0 = 0; k0 < K; k0 += GP_BK) {
    const bool whole = k0 + GP_BK <= K;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int r = lrow + 64 * half;
      const int am = m0 + r, wn = n0 + r;
      if (a_vec && whole) {
        const float4 v = *reinterpret_cast<const float4*>(A + am * lda + k0 + lk);
        As[lk][r] = v.x, As[lk + 1][r] = v.y, As[lk + 2][r] = v.z, As[lk + 3][r] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int k = k0 + lk + j;
          As[lk + j][r] = (am < M && k < K) ? A[am * lda + k] : 0.f;
        }
      }
      if (w_vec && whole) {
        const float4 v = *reinterpret_cast<const float4*>(W + wn * ldw + k0 + lk);
        Ws[lk][r] = v.x, Ws[lk + 1][r] = v.y, Ws[lk + 2][r] = v.z, Ws[lk + 3][r] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int k = k0 + lk + j;
          Ws[lk + j][r] = (wn < N && k < K) ? W[wn * ldw + k] : 0.f;
        }
      }
    }
    __syncthreads();
#define GPW_STEP(kk)                                                                               \
  {                                                                                                \
    const float4 a0 = *reinterpret_cast<const float4*>(&As[kk][ty * 4]);                           \
    const float4 a1 = *reinterpret_cast<const float4*>(&As[kk][64 + ty * 4]);                      \
    const float4 b0 = *reinterpret_cast<const float4*>(&Ws[kk][tx * 4]);                           \
    const float4 b1 = *reinterpret_cast<const float4*>(&Ws[kk][64 + tx * 4]);                      \
    const float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};                           \
    const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};                           \
    _Pragma("unroll") for (int i = 0; i < 8; ++i)                                                  \
        _Pragma("unroll") for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);     \
  }
    if (whole) {
#pragma unroll
      for (int kk = 0; kk < GP_BK; ++kk) GPW_STEP(kk)
    } else {
      for (int kk = 0; kk < K - k0; ++kk) GPW_STEP(kk)
    }
#undef GPW_STEP
    __syncthreads();
    if ((k0 + GP_BK) % GP_SEG == 0 || k0 + GP_BK >= K) {   // the segment ends here
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) total[i][j] += acc[i][j], acc[i][j] = 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = m0 + (i >> 2) * 64 + ty * 4 + (i & 3);
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int n = n0 + (j >> 2) * 64 + tx * 4 + (j & 3);
      if (n >= N) continue;
      float v = total[i][j];
      if (bias != nullptr) v += load_param(bias, n, bias_dtype);
      C[m * ldc + n] = v;
    }
  }
}

// The sums of one segment for one weight row and MT activation rows. grid (ceil(N / 64),
// ceil(segments / 4)), block (64, 4): the lanes of a wavefront hold 64 neighbouring weight rows,
// its four wavefronts four segments. The activation values are the same for all lanes.
template <int MT, typename TA, typename TW>
__global__ __launch_bounds__(256) void gemm_plain_rows_kernel(
    float* __restrict__ partial, const TA* __restrict__ A, const TW* __restrict__ W, int M, int N, int K,
    int64_t lda, int64_t ldw, int segments) {
  const int n = blockIdx.x * 64 + threadIdx.x;
  const int seg = __builtin_amdgcn_readfirstlane(blockIdx.y * 4 + threadIdx.y);
  if (seg >= segments) return;
  const int k_begin = seg * GP_SEG, k_end = min(K, k_begin + GP_SEG);
  const TW* wrow = W + (int64_t)min(n, N - 1) * ldw;
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;
  const TA* arow[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) arow[m] = A + (int64_t)min(m, M - 1) * lda;
  int k = k_begin;
  const bool vec = sizeof(TW) == 4 && (ldw & 3) == 0 && (((uintptr_t)W) & 15) == 0;
  if (vec) {
    // 64 k of the row at a time: sixteen loads of 16 bytes on their way before the first product
    constexpr int UN = 16;
    for (; k + 4 * UN <= k_end; k += 4 * UN) {
      float4 wv[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) wv[u] = *reinterpret_cast<const float4*>(wrow + k + 4 * u);
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const float w[4] = {wv[u].x, wv[u].y, wv[u].z, wv[u].w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int m = 0; m < MT; ++m) acc[m] = fmaf(to_float(arow[m][k + 4 * u + e]), w[e], acc[m]);
      }
    }
    for (; k + 4 <= k_end; k += 4) {
      const float4 w4 = *reinterpret_cast<const float4*>(wrow + k);
      const float w[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = fmaf(to_float(arow[m][k + e]), w[e], acc[m]);
    }
  }
  for (; k < k_end; ++k) {
    const float w = to_float(wrow[k]);
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = fmaf(to_float(arow[m][k]), w, acc[m]);
  }
  if (n < N) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
      if (m < M) partial[((int64_t)seg * M + m) * N + n] = acc[m];
  }
}

// The same sums for 32-bit weights whose K is whole segments, with the weights fetched line by
// line: in the kernel above the 64 lanes of a load touch 64 cache lines (each lane its own row), and
// the rate at which a compute unit looks lines up bounds it (3.6 TB/s at the Qwen2.5-7B shape). Here
// eight neighbouring lanes fetch the 128 bytes of one row, a load touches eight lines, and the
// wavefront turns the tile round in LDS: 32 k of its 64 rows at a time (two such chunks on their
// way while one is multiplied), the values go into the wavefront's own LDS region as
// [16-byte piece][row, 65 to a piece][4], from which lane n reads the pieces of row n one after the
// other (a read of 64 lanes is one KiB on end) and extends its chain of FMAs in ascending k. The
// region is the wavefront's own: LDS runs a wavefront's writes and reads in program order, so no
// barrier is needed, and the compiler keeps stores and loads that may name the same address in
// order. (A wavefront-scope fence here kept the staging registers in scratch memory.) grid and
// block as above.
#define GP_TURN_ROWS 65
template <int MT>
__global__ __launch_bounds__(256) void gemm_plain_rows_turned_kernel(
    float* __restrict__ partial, const float* __restrict__ A, const float* __restrict__ W, int M, int N, int K,
    int64_t lda, int64_t ldw, int segments) {
  __shared__ float4 turned[4][8 * GP_TURN_ROWS];
  const int lane = threadIdx.x;
  const int n0 = blockIdx.x * 64;
  const int seg = __builtin_amdgcn_readfirstlane(blockIdx.y * 4 + threadIdx.y);
  if (seg >= segments) return;
  const int k_begin = seg * GP_SEG;
  // load i of a chunk of 32 k: row 8 i + lane / 8 of the tile, piece lane % 8 of its 128 bytes
  const int lrow = lane >> 3, piece = lane & 7;
  const float* src[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) src[i] = W + (int64_t)min(n0 + 8 * i + lrow, N - 1) * ldw + k_begin + 4 * piece;
  float4 w0[8], w1[8];   // two chunks of 32 k on their way while a third is multiplied
#pragma unroll
  for (int i = 0; i < 8; ++i) w0[i] = *reinterpret_cast<const float4*>(src[i]);
#pragma unroll
  for (int i = 0; i < 8; ++i) w1[i] = *reinterpret_cast<const float4*>(src[i] + 32);
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;
  const float* arow[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) arow[m] = A + (int64_t)min(m, M - 1) * lda + k_begin;
  float4* mine = turned[threadIdx.y];
#define GP_TURN(WV_, C_)                                                                          \
  {                                                                                               \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) mine[piece * GP_TURN_ROWS + 8 * i + lrow] = WV_[i]; \
    __builtin_amdgcn_wave_barrier();                                                              \
    _Pragma("unroll") for (int p = 0; p < 8; ++p) {                                               \
      const float4 w4 = mine[p * GP_TURN_ROWS + lane];                                            \
      const float w[4] = {w4.x, w4.y, w4.z, w4.w};                                                \
      _Pragma("unroll") for (int e = 0; e < 4; ++e)                                               \
        _Pragma("unroll") for (int m = 0; m < MT; ++m)                                            \
          acc[m] = fmaf(arow[m][32 * (C_) + 4 * p + e], w[e], acc[m]);                            \
    }                                                                                             \
    __builtin_amdgcn_wave_barrier();                                                              \
  }
  // (the scheduler would ask for all four chunks at once and then spill two of them: each
  // sched_barrier keeps a group of loads where it is written)
  __builtin_amdgcn_sched_barrier(0);
  GP_TURN(w0, 0)
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 8; ++i) w0[i] = *reinterpret_cast<const float4*>(src[i] + 64);
  __builtin_amdgcn_sched_barrier(0);
  GP_TURN(w1, 1)
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 8; ++i) w1[i] = *reinterpret_cast<const float4*>(src[i] + 96);
  __builtin_amdgcn_sched_barrier(0);
  GP_TURN(w0, 2)
  GP_TURN(w1, 3)
#undef GP_TURN
  const int n = n0 + lane;
  if (n < N) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
      if (m < M) partial[((int64_t)seg * M + m) * N + n] = acc[m];
  }
}

template <typename TC>
__global__ __launch_bounds__(256) void gemm_plain_rows_sum_kernel(
    TC* __restrict__ C, const float* __restrict__ partial, const void* __restrict__ bias, int bias_dtype,
    int M, int N, int64_t ldc, int segments) {
  const int n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (n >= N) return;
  float total = 0.f;
  int s = 0;
  for (; s + 8 <= segments; s += 8) {   // eight sums on their way at a time; added in segment order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = partial[((int64_t)(s + u) * M + m) * N + n];
#pragma unroll
    for (int u = 0; u < 8; ++u) total += v[u];
  }
  for (; s < segments; ++s) total += partial[((int64_t)s * M + m) * N + n];
  if (bias != nullptr) total += load_param(bias, n, bias_dtype);
  C[(int64_t)m * ldc + n] = from_float<TC>(total);
}

// Floats of workspace with which a product of M rows runs through the kernels for few rows (0: it
// runs through the tile kernel, which needs none).
extern "C" int64_t he_gemm_plain_workspace_floats(int M, int N, int K) {
  if (M <= 0 || M > GP_ROWS_MAX_M || N <= 0 || K <= 0) return 0;
  return (int64_t)((K + GP_SEG - 1) / GP_SEG) * M * N;
}

template <typename TA, typename TW, typename TC>
static int launch_rows(void* C, const void* A, const void* W, const void* bias, int bias_dtype, int M,
                       int N, int K, int64_t lda, int64_t ldw, int64_t ldc, float* ws, hipStream_t s) {
  const int segments = (K + GP_SEG - 1) / GP_SEG;
  dim3 grid((N + 63) / 64, (segments + 3) / 4), block(64, 4);
  HE_REQUIRE(grid.y <= 65535, "he_gemm_plain: K=%d too long for one launch", K);
  // 32-bit weights in whole segments, rows 16-byte aligned: fetched line by line and turned round in LDS
  constexpr bool f32 = sizeof(TA) == 4 && sizeof(TW) == 4;
  const bool turned = f32 && K % GP_SEG == 0 && (ldw & 3) == 0 && (((uintptr_t)W) & 15) == 0;
#define GP_ROWS(MT_)                                                                                  \
  if (turned)                                                                                         \
    gemm_plain_rows_turned_kernel<MT_><<<grid, block, 0, s>>>(ws, (const float*)A, (const float*)W, M, N, K, \
                                                              lda, ldw, segments);                    \
  else                                                                                                \
    gemm_plain_rows_kernel<MT_, TA, TW><<<grid, block, 0, s>>>(ws, (const TA*)A, (const TW*)W, M, N, K, \
                                                               lda, ldw, segments)
  if (M == 1) GP_ROWS(1);
  else if (M == 2) GP_ROWS(2);
  else if (M <= 4) GP_ROWS(4);
  else GP_ROWS(8);
#undef GP_ROWS
  int rc = he_check_launch("he_gemm_plain");
  if (rc) return rc;
  gemm_plain_rows_sum_kernel<TC><<<dim3((N + 255) / 256, M), 256, 0, s>>>((TC*)C, ws, bias, bias_dtype, M, N,
                                                                          ldc, segments);
  return he_check_launch("he_gemm_plain");
}

// workspace_f32 (may be null) of workspace_floats floats: with he_gemm_plain_workspace_floats(M, N, K)
// or more of them a product of few rows runs through the kernels made for it. The result is the
// same bit for bit either way.
extern "C" int he_gemm_plain(void* C, const void* A, const void* W, const void* bias, int M, int N,
                             int K, int64_t lda, int64_t ldw, int64_t ldc, int in_dtype,
                             int out_dtype, int bias_dtype, void* workspace_f32,
                             int64_t workspace_floats, void* stream) {
  HE_REQUIRE(M >= 0 && N > 0 && K > 0, "he_gemm_plain: bad sizes M=%d N=%d K=%d", M, N, K);
  HE_REQUIRE(lda >= K && ldw >= K && ldc >= N, "he_gemm_plain: bad leading dimensions");
  if (M == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int64_t need = he_gemm_plain_workspace_floats(M, N, K);
  if (need > 0 && workspace_f32 != nullptr && workspace_floats >= need) {
    float* ws = (float*)workspace_f32;
    if (in_dtype == HE_F32 && out_dtype == HE_F32)
      return launch_rows<float, float, float>(C, A, W, bias, bias_dtype, M, N, K, lda, ldw, ldc, ws, s);
    if (in_dtype == HE_BF16 && out_dtype == HE_BF16)
      return launch_rows<bf16_t, bf16_t, bf16_t>(C, A, W, bias, bias_dtype, M, N, K, lda, ldw, ldc, ws, s);
    if (in_dtype == HE_BF16 && out_dtype == HE_F32)
      return launch_rows<bf16_t, bf16_t, float>(C, A, W, bias, bias_dtype, M, N, K, lda, ldw, ldc, ws, s);
    HE_REQUIRE(false, "he_gemm_plain: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
  }
  dim3 grid((N + GP_BN - 1) / GP_BN, (M + GP_BM - 1) / GP_BM);
  HE_REQUIRE(grid.y <= 65535, "he_gemm_plain: M=%d too large for one launch", M);
  if (in_dtype == HE_F32 && out_dtype == HE_F32 && M >= GPW_BM) {
    dim3 wide((N + GPW_BN - 1) / GPW_BN, (M + GPW_BM - 1) / GPW_BM);
    gemm_plain_wide_kernel<<<wide, 256, 0, s>>>((float*)C, (const float*)A, (const float*)W, bias, bias_dtype, M, N,
                                                K, lda, ldw, ldc);
  } else if (in_dtype == HE_F32 && out_dtype == HE_F32)
    gemm_plain_kernel<float, float, float><<<grid, 256, 0, s>>>(
        (float*)C, (const float*)A, (const float*)W, bias, bias_dtype, M, N, K, lda, ldw, ldc);
  else if (in_dtype == HE_BF16 && out_dtype == HE_BF16)
    gemm_plain_kernel<bf16_t, bf16_t, bf16_t><<<grid, 256, 0, s>>>(
        (bf16_t*)C, (const bf16_t*)A, (const bf16_t*)W, bias, bias_dtype, M, N, K, lda, ldw, ldc);
  else if (in_dtype == HE_BF16 && out_dtype == HE_F32)
    gemm_plain_kernel<bf16_t, bf16_t, float><<<grid, 256, 0, s>>>(
        (float*)C, (const bf16_t*)A, (const bf16_t*)W, bias, bias_dtype, M, N, K, lda, ldw, ldc);
  else
    HE_REQUIRE(false, "he_gemm_plain: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
  return he_check_launch("he_gemm_plain");
}
