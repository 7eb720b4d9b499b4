// Row-wise kernels without reductions: embedding gather into the fp32 residual
// stream, row gather, gated activation (SiLU(gate) * up) and the materialising
// residual add.
#include "common.h"
#include "hector_kernels.h"

// out[t, :] = table[ids[t], :] as fp32; an id outside [0, V) gives a zero row
// (reference: kernels/linear.cu:36-69).
template <typename T>
__global__ void embedding_kernel(float* __restrict__ out, const T* __restrict__ table,
                                 const int32_t* __restrict__ ids, int D, int V) {
  const int64_t t = blockIdx.x;
  const int id = ids[t];
  float* o = out + t * (int64_t)D;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* row = table + (int64_t)id * D;
  if (sizeof(T) == 2 && (D & 7) == 0 && (((uintptr_t)table | (uintptr_t)out) & 15) == 0) {
    // eight elements a thread and turn: one 16-byte load, two 16-byte stores
    for (int i = 8 * threadIdx.x; i < D; i += 8 * blockDim.x) {
      const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(row) + i);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      float f[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f[2 * j] = __uint_as_float(w[j] << 16);
        f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
      *reinterpret_cast<float4*>(o + i) = make_float4(f[0], f[1], f[2], f[3]);
      *reinterpret_cast<float4*>(o + i + 4) = make_float4(f[4], f[5], f[6], f[7]);
    }
    return;
  }
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = to_float(row[i]);
}

extern "C" int he_embedding(void* out_f32, const void* table, const void* ids, int rows, int D,
                            int V, int table_dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && D > 0 && V > 0, "he_embedding: bad sizes rows=%d D=%d V=%d", rows, D, V);
  if (rows == 0) return 0;
  const int threads = D >= 1024 ? 256 : (D >= 256 ? 128 : 64);
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == HE_BF16)
    embedding_kernel<bf16_t><<<rows, threads, 0, s>>>((float*)out_f32, (const bf16_t*)table,
                                                      (const int32_t*)ids, D, V);
  else if (table_dtype == HE_F32)
    embedding_kernel<float><<<rows, threads, 0, s>>>((float*)out_f32, (const float*)table,
                                                     (const int32_t*)ids, D, V);
  else
    HE_REQUIRE(false, "he_embedding: unknown dtype %d", table_dtype);
  return he_check_launch("he_embedding");
}

// out[r, :] = src[rows[r], :]; a negative row index gives a zero row.
__global__ void gather_rows_f32_kernel(float* __restrict__ out, const float* __restrict__ src,
                                       const int32_t* __restrict__ rows, int D, int n_src) {
  const int64_t r = blockIdx.x;
  const int idx = rows[r];
  float* o = out + r * (int64_t)D;
  if (idx < 0 || idx >= n_src) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const float* in = src + (int64_t)idx * D;
  if ((D & 3) == 0 && (((uintptr_t)src | (uintptr_t)out) & 15) == 0) {
    for (int i = 4 * threadIdx.x; i < D; i += 4 * blockDim.x)
      *reinterpret_cast<float4*>(o + i) = *reinterpret_cast<const float4*>(in + i);
    return;
  }
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = in[i];
}

extern "C" int he_gather_rows_f32(void* out, const void* src, const void* rows, int n_out, int D,
                                  int n_src, void* stream) {
  HE_REQUIRE(n_out >= 0 && D > 0 && n_src >= 0, "he_gather_rows_f32: bad sizes");
  if (n_out == 0) return 0;
  gather_rows_f32_kernel<<<n_out, 256, 0, (hipStream_t)stream>>>(
      (float*)out, (const float*)src, (const int32_t*)rows, D, n_src);
  return he_check_launch("he_gather_rows_f32");
}

// resid[r, :] += delta[r, :], the residual sum in fp32.
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ resid, const T* __restrict__ delta,
                                    int64_t n) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) resid[i] += to_float(delta[i]);
}

extern "C" int he_residual_add(void* resid_f32, const void* delta, int64_t n, int delta_dtype,
                               void* stream) {
  HE_REQUIRE(n >= 0, "he_residual_add: bad size");
  if (n == 0) return 0;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipStream_t s = (hipStream_t)stream;
  if (delta_dtype == HE_BF16)
    residual_add_kernel<bf16_t><<<(int)blocks, 256, 0, s>>>((float*)resid_f32,
                                                            (const bf16_t*)delta, n);
  else if (delta_dtype == HE_F32)
    residual_add_kernel<float><<<(int)blocks, 256, 0, s>>>((float*)resid_f32, (const float*)delta,
                                                           n);
  else
    HE_REQUIRE(false, "he_residual_add: unknown dtype %d", delta_dtype);
  return he_check_launch("he_residual_add");
}

// out[r, i] = silu(gate[r, i]) * up[r, i] with x = [rows, 2I],
// silu(z) = z / (1 + exp(-z)) in fp32 (reference: kernels/activations.cu:19-21,183-198).
// Column layout of x: gate then up (x[r, i], x[r, I + i]); or interleaved, as the
// fused gate||up weight of the MFMA path lays its rows out: gate i at column 2i,
// its up at 2i + 1.
// With splits > 0, x is the fp32 K slices [splits][rows][2I] of the gate||up product,
// added here in the order of the slice index.
template <typename T, typename TI>
__global__ void silu_mul_kernel(T* __restrict__ out, const TI* __restrict__ x, int64_t rows,
                                int I, int interleaved, int splits) {
  const int64_t n = rows * (int64_t)I;
  const int64_t split_stride = rows * 2 * (int64_t)I;
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const int64_t r = i / I;
    const int c = (int)(i - r * I);
    const int gc = interleaved ? 2 * c : c;
    const int uc = interleaved ? gc + 1 : I + c;
    const TI* row = x + r * 2 * (int64_t)I;
    float g = to_float(row[gc]), u = to_float(row[uc]);
    for (int s = 1; s < splits; ++s) {
      g += to_float(row[s * split_stride + gc]);
      u += to_float(row[s * split_stride + uc]);
    }
    const float y = g / (1.f + expf(-g)) * u;
    out[i] = from_float<T>(y);
  }
}

// bf16, eight outputs per thread, I a multiple of 8: eight consecutive gates and their ups are
// two runs of 16 bytes, or, interleaved, one run of 32 bytes of (gate, up) pairs.
__global__ void silu_mul_vec_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ x,
                                    int64_t rows, int I, int interleaved) {
  const int64_t n8 = rows * (int64_t)(I >> 3);
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int per_row = I >> 3;
  for (; i < n8; i += stride) {
    const int64_t r = i / per_row;
    const int c = (int)(i - r * per_row) << 3;
    const uint16_t* row = x + r * 2 * (int64_t)I;
    uint32_t o[4];
    if (interleaved) {
      const uint4 a = *reinterpret_cast<const uint4*>(row + 2 * c);
      const uint4 b = *reinterpret_cast<const uint4*>(row + 2 * c + 8);
      const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};   // (gate, up) a word
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(w[2 * j] << 16), u0 = __uint_as_float(w[2 * j] & 0xffff0000u);
        const float g1 = __uint_as_float(w[2 * j + 1] << 16), u1 = __uint_as_float(w[2 * j + 1] & 0xffff0000u);
        o[j] = pack2_bf16(g0 / (1.f + expf(-g0)) * u0, g1 / (1.f + expf(-g1)) * u1);
      }
    } else {
      const uint4 g4 = *reinterpret_cast<const uint4*>(row + c);
      const uint4 u4 = *reinterpret_cast<const uint4*>(row + I + c);
      const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
        o[j] = pack2_bf16(g0 / (1.f + expf(-g0)) * u0, g1 / (1.f + expf(-g1)) * u1);
      }
    }
    *reinterpret_cast<uint4*>(out + r * (int64_t)I + c) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

extern "C" int he_silu_mul(void* out, const void* gate_up, int rows, int I, int interleaved,
                           int splits, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && I > 0, "he_silu_mul: bad sizes rows=%d I=%d", rows, I);
  HE_REQUIRE(splits >= 0 && splits <= 64, "he_silu_mul: bad slice count %d", splits);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_silu_mul: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  const int64_t n = (int64_t)rows * I;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65535 * 4) blocks = 65535 * 4;
  hipStream_t s = (hipStream_t)stream;
  if (splits == 0 && dtype == HE_BF16 && (I & 7) == 0 &&
      ((((uintptr_t)out) | ((uintptr_t)gate_up)) & 15) == 0) {
    const int64_t n8 = n >> 3;
    int64_t vb = (n8 + 255) / 256;
    if (vb > 65535 * 4) vb = 65535 * 4;
    silu_mul_vec_kernel<<<(int)vb, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)gate_up, rows, I,
                                                interleaved);
  } else if (splits > 0) {  // fp32 partial sums in
    if (dtype == HE_BF16)
      silu_mul_kernel<bf16_t, float><<<(int)blocks, 256, 0, s>>>(
          (bf16_t*)out, (const float*)gate_up, rows, I, interleaved, splits);
    else
      silu_mul_kernel<float, float><<<(int)blocks, 256, 0, s>>>(
          (float*)out, (const float*)gate_up, rows, I, interleaved, splits);
  } else if (dtype == HE_BF16) {
    silu_mul_kernel<bf16_t, bf16_t><<<(int)blocks, 256, 0, s>>>(
        (bf16_t*)out, (const bf16_t*)gate_up, rows, I, interleaved, 1);
  } else {
    silu_mul_kernel<float, float><<<(int)blocks, 256, 0, s>>>((float*)out, (const float*)gate_up,
                                                              rows, I, interleaved, 1);
  }
  return he_check_launch("he_silu_mul");
}
