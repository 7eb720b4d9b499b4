// Plain tiled matrix product  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N])  with fp32
// FMA accumulation. Each output element is the sum over k = 0..K-1 in that
// order, whatever M and whichever rows share the launch, so a row's result
// never depends on the batch it is in. It is the true 32-bit path of every
// linear layer and the reference beside the MFMA kernels.
// Weight layout [N, K] row-major as in the reference (kernels/register_kernels.cpp:373-386).
#include "common.h"
#include "hector_kernels.h"

#define GP_BM 64
#define GP_BN 64
#define GP_BK 16

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_plain_kernel(
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
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GP_BK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const int am = m0 + lrow;
      const int wn = n0 + lrow;
      As[lk + j][lrow] = (am < M && k < K) ? to_float(A[am * lda + k]) : 0.f;
      Ws[lk + j][lrow] = (wn < N && k < K) ? to_float(W[wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GP_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias != nullptr) v += load_param(bias, n, bias_dtype);
      C[m * ldc + n] = from_float<TC>(v);
    }
  }
}

extern "C" int he_gemm_plain(void* C, const void* A, const void* W, const void* bias, int M, int N,
                             int K, int64_t lda, int64_t ldw, int64_t ldc, int in_dtype,
                             int out_dtype, int bias_dtype, void* stream) {
  HE_REQUIRE(M >= 0 && N > 0 && K > 0, "he_gemm_plain: bad sizes M=%d N=%d K=%d", M, N, K);
  HE_REQUIRE(lda >= K && ldw >= K && ldc >= N, "he_gemm_plain: bad leading dimensions");
  if (M == 0) return 0;
  dim3 grid((N + GP_BN - 1) / GP_BN, (M + GP_BM - 1) / GP_BM);
  HE_REQUIRE(grid.y <= 65535, "he_gemm_plain: M=%d too large for one launch", M);
  hipStream_t s = (hipStream_t)stream;
  if (in_dtype == HE_F32 && out_dtype == HE_F32)
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
