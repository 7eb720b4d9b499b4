// RMS normalisation. The residual stream is fp32 in both precisions; the fused
// kernel adds the pending branch output to it and normalises the sum in one
// pass over the row:
//   r = resid + delta          (fp32, stored back as the new residual)
//   y = r * (1/sqrt(mean(r^2) + eps)) * w
// Reference formulas: kernels/normalization.cu:36-63 (norm) and
// kernels/fused_add_rmsnorm.cu:47-81 (add + norm, two outputs).
#include "common.h"
#include "hector_kernels.h"

template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                   const void* __restrict__ w, int w_dtype, TO* __restrict__ out,
                                   int D, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float* r = resid + row * (int64_t)D;
  float ss = 0.f;
  if (delta != nullptr) {
    const TD* d = delta + row * (int64_t)D;
    for (int i = threadIdx.x; i < D; i += blockDim.x) {
      const float v = r[i] + to_float(d[i]);
      r[i] = v;
      ss += v * v;
    }
  } else {
    for (int i = threadIdx.x; i < D; i += blockDim.x) {
      const float v = r[i];
      ss += v * v;
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / (float)D + eps);
  if (out == nullptr) return;
  TO* o = out + row * (int64_t)D;
  // each thread re-reads exactly the elements it wrote above
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    o[i] = from_float<TO>(r[i] * inv * load_param(w, i, w_dtype));
  }
}

// The same with a row of at most NORM_EPT * blockDim.x elements kept in registers:
// every load of the row is issued before the reduction, nothing is read twice.
#define NORM_EPT 8
template <typename TD, typename TO>
__global__ void add_rmsnorm_reg_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                       const void* __restrict__ w, int w_dtype,
                                       TO* __restrict__ out, int D, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float* r = resid + row * (int64_t)D;
  const TD* d = delta ? delta + row * (int64_t)D : nullptr;
  float v[NORM_EPT], g[NORM_EPT];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < NORM_EPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    v[e] = 0.f;
    g[e] = 0.f;
    if (i < D) {
      v[e] = r[i];
      if (d) v[e] += to_float(d[i]);
      if (out) g[e] = load_param(w, i, w_dtype);
    }
  }
#pragma unroll
  for (int e = 0; e < NORM_EPT; ++e) ss += v[e] * v[e];
  if (d) {
#pragma unroll
    for (int e = 0; e < NORM_EPT; ++e) {
      const int i = threadIdx.x + e * blockDim.x;
      if (i < D) r[i] = v[e];
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / (float)D + eps);
  if (out == nullptr) return;
  TO* o = out + row * (int64_t)D;
#pragma unroll
  for (int e = 0; e < NORM_EPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    if (i < D) o[i] = from_float<TO>(v[e] * inv * g[e]);
  }
}

// The same with four neighbouring elements a thread and access (16 bytes of the fp32
// residual, 8 of a bf16 tensor): a row of at most 4 * NORM_VEC * blockDim.x elements, D a
// multiple of 4. Tall inputs (prompt steps) are bound by memory traffic; with one element an
// access the kernel reached 3.4 TB/s.
#define NORM_VEC 4
__device__ __forceinline__ void load4(const float* p, float* v) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float* v) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(x.x << 16), v[1] = __uint_as_float(x.x & 0xffff0000u);
  v[2] = __uint_as_float(x.y << 16), v[3] = __uint_as_float(x.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float* v) {
  uint2 x;
  x.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
  x.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = x;
}

template <typename TD, typename TO, typename TW>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                       const TW* __restrict__ w, TO* __restrict__ out, int D,
                                       float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float* r = resid + row * (int64_t)D;
  const TD* d = delta ? delta + row * (int64_t)D : nullptr;
  float v[NORM_VEC][4], g[NORM_VEC][4], a[NORM_VEC][4];
  float ss = 0.f;
  // the loads stand in no per-thread branch (a group beyond the row reads the row's last four
  // elements and counts as zeros), so they all go out before the first is waited for
#pragma unroll
  for (int e = 0; e < NORM_VEC; ++e) load4(r + min(4 * (int)(threadIdx.x + e * blockDim.x), D - 4), v[e]);
  if (d) {
#pragma unroll
    for (int e = 0; e < NORM_VEC; ++e) load4(d + min(4 * (int)(threadIdx.x + e * blockDim.x), D - 4), a[e]);
  }
  if (out) {
#pragma unroll
    for (int e = 0; e < NORM_VEC; ++e) load4(w + min(4 * (int)(threadIdx.x + e * blockDim.x), D - 4), g[e]);
  }
#pragma unroll
  for (int e = 0; e < NORM_VEC; ++e) {
    const bool in = 4 * (int)(threadIdx.x + e * blockDim.x) < D;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[e][j] = in ? v[e][j] + (d ? a[e][j] : 0.f) : 0.f;
      g[e][j] = (in && out) ? g[e][j] : 0.f;
    }
  }
#pragma unroll
  for (int e = 0; e < NORM_VEC; ++e)
#pragma unroll
    for (int j = 0; j < 4; ++j) ss += v[e][j] * v[e][j];
  if (d) {
#pragma unroll
    for (int e = 0; e < NORM_VEC; ++e) {
      const int i = 4 * (threadIdx.x + e * blockDim.x);
      if (i < D) store4(r + i, v[e]);
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / (float)D + eps);
  if (out == nullptr) return;
  TO* o = out + row * (int64_t)D;
#pragma unroll
  for (int e = 0; e < NORM_VEC; ++e) {
    const int i = 4 * (threadIdx.x + e * blockDim.x);
    if (i < D) {
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] = v[e][j] * inv * g[e][j];
      store4(o + i, y);
    }
  }
}

template <typename TD, typename TO>
static void launch_add_rmsnorm_vec(float* resid, const void* delta, const void* w, int w_dtype,
                                   void* out, int rows, int D, float eps, hipStream_t s) {
  int threads = 64;
  while (threads < 512 && 4 * NORM_VEC * threads < D) threads <<= 1;
  while (threads > 64 && 4 * (threads >> 1) >= D) threads >>= 1;
  if (w_dtype == HE_BF16)
    add_rmsnorm_vec_kernel<TD, TO, bf16_t><<<rows, threads, 0, s>>>(
        resid, (const TD*)delta, (const bf16_t*)w, (TO*)out, D, eps);
  else
    add_rmsnorm_vec_kernel<TD, TO, float><<<rows, threads, 0, s>>>(
        resid, (const TD*)delta, (const float*)w, (TO*)out, D, eps);
}

static int norm_threads(int D) { return D >= 2048 ? 512 : (D >= 512 ? 256 : (D >= 128 ? 128 : 64)); }

extern "C" int he_add_rmsnorm(void* resid_f32, const void* delta, const void* weight, void* out,
                              int rows, int D, float eps, int act_dtype, int w_dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && D > 0, "he_add_rmsnorm: bad sizes rows=%d D=%d", rows, D);
  HE_REQUIRE(w_dtype == HE_F32 || w_dtype == HE_BF16, "he_add_rmsnorm: bad weight dtype");
  HE_REQUIRE(act_dtype == HE_F32 || act_dtype == HE_BF16, "he_add_rmsnorm: unknown dtype %d",
             act_dtype);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = norm_threads(D);
  if ((D & 3) == 0 && D <= 4 * NORM_VEC * 512 &&
             ((((uintptr_t)resid_f32) | ((uintptr_t)delta) | ((uintptr_t)weight) | ((uintptr_t)out)) & 15) == 0) {
    if (act_dtype == HE_BF16)
      launch_add_rmsnorm_vec<bf16_t, bf16_t>((float*)resid_f32, delta, weight, w_dtype, out, rows, D, eps, s);
    else
      launch_add_rmsnorm_vec<float, float>((float*)resid_f32, delta, weight, w_dtype, out, rows, D, eps, s);
  } else if (D <= NORM_EPT * threads) {
    if (act_dtype == HE_BF16)
      add_rmsnorm_reg_kernel<bf16_t, bf16_t><<<rows, threads, 0, s>>>(
          (float*)resid_f32, (const bf16_t*)delta, weight, w_dtype, (bf16_t*)out, D, eps);
    else
      add_rmsnorm_reg_kernel<float, float><<<rows, threads, 0, s>>>(
          (float*)resid_f32, (const float*)delta, weight, w_dtype, (float*)out, D, eps);
  } else if (act_dtype == HE_BF16) {
    add_rmsnorm_kernel<bf16_t, bf16_t><<<rows, threads, 0, s>>>(
        (float*)resid_f32, (const bf16_t*)delta, weight, w_dtype, (bf16_t*)out, D, eps);
  } else {
    add_rmsnorm_kernel<float, float><<<rows, threads, 0, s>>>(
        (float*)resid_f32, (const float*)delta, weight, w_dtype, (float*)out, D, eps);
  }
  return he_check_launch("he_add_rmsnorm");
}

// Plain row-wise RMS norm of an activation tensor with a row stride (for
// normalising slices such as per-head vectors): x viewed as [rows, D].
template <typename T>
__global__ void rmsnorm_rows_kernel(T* __restrict__ out, const T* __restrict__ x,
                                    const void* __restrict__ w, int w_dtype, int D,
                                    int64_t x_stride, int64_t out_stride, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const T* xi = x + row * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    const float v = to_float(xi[i]);
    ss += v * v;
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / (float)D + eps);
  T* o = out + row * out_stride;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    const float g = w ? load_param(w, i, w_dtype) : 1.f;
    o[i] = from_float<T>(to_float(xi[i]) * inv * g);
  }
}

extern "C" int he_rmsnorm_rows(void* out, const void* x, const void* weight, int rows, int D,
                               int64_t x_stride, int64_t out_stride, float eps, int dtype,
                               int w_dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && D > 0 && x_stride >= D && out_stride >= D,
             "he_rmsnorm_rows: bad sizes rows=%d D=%d", rows, D);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = norm_threads(D);
  if (dtype == HE_BF16)
    rmsnorm_rows_kernel<bf16_t><<<rows, threads, 0, s>>>((bf16_t*)out, (const bf16_t*)x, weight,
                                                         w_dtype, D, x_stride, out_stride, eps);
  else if (dtype == HE_F32)
    rmsnorm_rows_kernel<float><<<rows, threads, 0, s>>>((float*)out, (const float*)x, weight,
                                                        w_dtype, D, x_stride, out_stride, eps);
  else
    HE_REQUIRE(false, "he_rmsnorm_rows: unknown dtype %d", dtype);
  return he_check_launch("he_rmsnorm_rows");
}

// Rows x = r * gain whose scale is still owed: out = x / sqrt(sum(partials of the row) / D + eps).
// The partial sums of squares (one per workgroup of the product that made the rows) are
// added as that product's consumers add them: lanes over strided partials, then the wavefront.
// x_pieces: x lies piece-major, 16-byte pieces [D / 8][rows][8]; out is row-major either way.
__global__ void scale_rows_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ x,
                                  const float* __restrict__ partials, int count, int D, float eps,
                                  int x_pieces) {
  __shared__ float inv_s;
  const int64_t row = blockIdx.x;
  if (threadIdx.x < 64) {
    float part = 0.f;
    for (int i = threadIdx.x; i < count; i += 64) part += partials[row * count + i];
    const float total = wave_sum(part);
    if (threadIdx.x == 0) inv_s = 1.0f / sqrtf(total / (float)D + eps);
  }
  __syncthreads();
  const float inv = inv_s;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    const int64_t at = x_pieces ? ((int64_t)(i >> 3) * gridDim.x + row) * 8 + (i & 7) : row * D + i;
    out[row * D + i] = float_to_bf16_bits(bf16_bits_to_float(x[at]) * inv);
  }
}

extern "C" int he_scale_rows_bf16(void* out, const void* x, const void* partials, int count,
                                  int rows, int D, float eps, int x_pieces, void* stream) {
  HE_REQUIRE(rows >= 0 && D > 0 && count > 0, "he_scale_rows_bf16: bad sizes rows=%d D=%d count=%d",
             rows, D, count);
  HE_REQUIRE(!x_pieces || D % 8 == 0, "he_scale_rows_bf16: piece-major rows of width %d, not a multiple of 8", D);
  if (rows == 0) return 0;
  scale_rows_kernel<<<rows, norm_threads(D), 0, (hipStream_t)stream>>>(
      (uint16_t*)out, (const uint16_t*)x, (const float*)partials, count, D, eps, x_pieces);
  return he_check_launch("he_scale_rows_bf16");
}
