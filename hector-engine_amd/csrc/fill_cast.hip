// Weight preparation on the device: seeded random tensors whose every element the host can
// reproduce (the reference has no such mode; its tests fill buffers from a host mt19937:
// tests/test_kernels.cu:19-35), and the dtype conversion of uploaded tensors.
//
// Random values are counter-based: element i of a tensor with key k takes 16 bits of
//   word(j) = mix64(k + (j + 1) * 0x9E3779B97F4A7C15),  j = i / 4,  bits 16 (i % 4) .. + 16,
// (mix64 = the splitmix64 finaliser) and looks them up in a table of 65536 quantiles of the
// standard normal distribution that the host computes once and hands over. The value is
// quantile * std + mean, each operation rounded to fp32 on its own, then rounded to bfloat16
// (nearest even) whatever the tensor's dtype: integers and one table lookup, so the host's
// numpy lines give the same bits. Integer tables take (word32 * high) >> 32.
#include "common.h"
#include "hector_kernels.h"

__host__ __device__ __forceinline__ uint64_t he_mix64(uint64_t z) {
  z ^= z >> 30;
  z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27;
  z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}

// four elements a thread: one word
template <typename T>
__global__ void fill_normal_kernel(T* __restrict__ out, int64_t n, uint64_t key,
                                   const float* __restrict__ quantiles, float mean, float std) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t i0 = 4 * j;
  if (i0 >= n) return;
  const uint64_t w = he_mix64(key + (uint64_t)(j + 1) * 0x9E3779B97F4A7C15ull);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (i0 + e >= n) break;
    const float z = quantiles[(w >> (16 * e)) & 0xffffu];
    const float v = __fadd_rn(__fmul_rn(z, std), mean);   // two roundings, never fused
    out[i0 + e] = from_float<T>(bf16_bits_to_float(float_to_bf16_bits(v)));
  }
}

__global__ void fill_integers_kernel(int32_t* __restrict__ out, int64_t n, uint64_t key, uint32_t high) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t w = he_mix64(key + (uint64_t)(i + 1) * 0x9E3779B97F4A7C15ull);
  out[i] = (int32_t)(((w >> 32) * (uint64_t)high) >> 32);
}

extern "C" int he_fill_random(void* out, int64_t n, int dtype, uint64_t key, const void* quantiles_f32,
                              float mean, float std, void* stream) {
  HE_REQUIRE(n >= 0 && n < ((int64_t)1 << 40), "he_fill_random: bad element count %lld", (long long)n);
  HE_REQUIRE(quantiles_f32 != nullptr, "he_fill_random: the quantile table is missing");
  if (n == 0) return 0;
  const int threads = 256;
  const int64_t blocks = ((n + 3) / 4 + threads - 1) / threads;
  HE_REQUIRE(blocks <= 0x7fffffff, "he_fill_random: %lld elements are too many for one launch", (long long)n);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    fill_normal_kernel<bf16_t><<<(unsigned)blocks, threads, 0, s>>>((bf16_t*)out, n, key, (const float*)quantiles_f32, mean, std);
  else if (dtype == HE_F32)
    fill_normal_kernel<float><<<(unsigned)blocks, threads, 0, s>>>((float*)out, n, key, (const float*)quantiles_f32, mean, std);
  else
    HE_REQUIRE(false, "he_fill_random: unknown dtype %d", dtype);
  return he_check_launch("he_fill_random");
}

extern "C" int he_fill_random_integers(void* out_i32, int64_t n, uint64_t key, int64_t high, void* stream) {
  HE_REQUIRE(n >= 0 && high > 0 && high <= 0xffffffffll, "he_fill_random_integers: bad sizes");
  if (n == 0) return 0;
  const int64_t blocks = (n + 255) / 256;
  HE_REQUIRE(blocks <= 0x7fffffff, "he_fill_random_integers: too many elements for one launch");
  fill_integers_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((int32_t*)out_i32, n, key, (uint32_t)high);
  return he_check_launch("he_fill_random_integers");
}

// ---- conversion of an uploaded tensor into the dtype it runs in ------------------------
__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
  if (exp == 0) {                       // zero or subnormal: man * 2^-24
    const float f = (float)man * 5.9604644775390625e-8f;
    return __uint_as_float(__float_as_uint(f) | sign);
  }
  if (exp == 31) return __uint_as_float(sign | 0x7f800000u | (man << 13));
  return __uint_as_float(sign | ((exp + 112u) << 23) | (man << 13));
}

template <int IN>
__device__ __forceinline__ float cast_load(const void* in, int64_t i) {
  if (IN == HE_F32) return ((const float*)in)[i];
  if (IN == HE_BF16) return bf16_bits_to_float(((const uint16_t*)in)[i]);
  return half_bits_to_float(((const uint16_t*)in)[i]);
}

template <int IN, typename TO>
__global__ void cast_kernel(TO* __restrict__ out, const void* __restrict__ in, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = from_float<TO>(cast_load<IN>(in, i));
}

extern "C" int he_cast(void* out, const void* in, int64_t n, int in_dtype, int out_dtype, void* stream) {
  HE_REQUIRE(n >= 0, "he_cast: bad element count");
  HE_REQUIRE(out_dtype == HE_F32 || out_dtype == HE_BF16, "he_cast: the output is float32 or bfloat16, not %d", out_dtype);
  if (n == 0) return 0;
  const int threads = 256;
  const unsigned blocks = (unsigned)((n + threads - 1) / threads < 65536 ? (n + threads - 1) / threads : 65536);
  hipStream_t s = (hipStream_t)stream;
#define CAST(IN_)                                                                          \
  case IN_:                                                                                \
    if (out_dtype == HE_F32) cast_kernel<IN_, float><<<blocks, threads, 0, s>>>((float*)out, in, n); \
    else cast_kernel<IN_, bf16_t><<<blocks, threads, 0, s>>>((bf16_t*)out, in, n);         \
    break;
  switch (in_dtype) {
    CAST(HE_F32) CAST(HE_BF16) CAST(HE_F16)
    default:
      HE_REQUIRE(false, "he_cast: unknown input dtype %d", in_dtype);
  }
#undef CAST
  return he_check_launch("he_cast");
}
