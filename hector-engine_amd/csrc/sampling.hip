// Sampling over fp32 logit rows, one workgroup per row: argmax (lowest index on
// ties), window penalties, and temperature / top-k / top-p sampling by inverse
// CDF with a supplied 32-bit uniform.
//
// Rule (the reference's, kernels/sampling.cu:411-451, on sorted candidates):
// order the row by value descending (ties by ascending index); keep the first
// top_k; p_i = exp((v_i - v_max) / T); keep the shortest prefix whose mass
// reaches top_p of the kept mass; draw r uniformly below the mass of that prefix
// and take the first element whose cumulative mass exceeds r.
//
// No sort is done. Every p_i is turned into a 40-bit fixed-point integer, so
// sums are exact and independent of the order of addition, and each "first
// prefix whose cumulative count / mass reaches t" is found by a four-pass radix
// descent over the order-preserving integer image of the floats.
#include "common.h"
#include "hector_kernels.h"

#define SAMP_THREADS 1024
#define SAMP_FIXED_ONE 1099511627776.0f  // 2^40

// ---------------------------------------------------------------- argmax
// The lowest index among the maxima of each row. A row is cut into parts of ARGMAX_PART
// elements, one workgroup each, so that a long vocabulary is read by many compute units at
// once; a second small launch takes the best of a row's parts (with one part the first
// launch writes the result itself).
#define ARGMAX_PART 8192
#define ARGMAX_THREADS 256

__device__ __forceinline__ void argmax_take(float& best, int& bi, float v, int i) {
  if (v > best || (v == best && i < bi)) {
    best = v;
    bi = i;
  }
}

// Reduces (best, bi) over the workgroup; valid in thread 0.
__device__ __forceinline__ void argmax_block(float& best, int& bi) {
  __shared__ float sval[ARGMAX_THREADS / HE_WAVE];
  __shared__ int sidx[ARGMAX_THREADS / HE_WAVE];
#pragma unroll
  for (int off = HE_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, HE_WAVE);
    const int oi = __shfl_xor(bi, off, HE_WAVE);
    argmax_take(best, bi, ov, oi);
  }
  const int lane = threadIdx.x & (HE_WAVE - 1), wave = threadIdx.x >> 6;
  if (lane == 0) {
    sval[wave] = best;
    sidx[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) argmax_take(best, bi, sval[w], sidx[w]);
}

// grid (parts, rows)
__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_parts_kernel(
    int32_t* __restrict__ out, float* __restrict__ part_val, int32_t* __restrict__ part_idx,
    const float* __restrict__ logits, int V, int64_t stride) {
  const float* x = logits + blockIdx.y * stride;
  const int lo = blockIdx.x * ARGMAX_PART, hi = min(V, lo + ARGMAX_PART);
  float best = -INFINITY;
  int bi = 0x7fffffff;
  const bool vec = ((stride & 3) == 0) && ((((uintptr_t)logits) & 15) == 0);
  if (vec) {
    for (int i = lo + 4 * threadIdx.x; i < hi; i += 4 * ARGMAX_THREADS) {
      if (i + 4 <= hi) {
        const float4 v = *reinterpret_cast<const float4*>(x + i);
        argmax_take(best, bi, v.x, i);
        argmax_take(best, bi, v.y, i + 1);
        argmax_take(best, bi, v.z, i + 2);
        argmax_take(best, bi, v.w, i + 3);
      } else {
        for (int j = i; j < hi; ++j) argmax_take(best, bi, x[j], j);
      }
    }
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += ARGMAX_THREADS) argmax_take(best, bi, x[i], i);
  }
  argmax_block(best, bi);
  if (threadIdx.x == 0) {
    if (gridDim.x == 1) {
      out[blockIdx.y] = bi == 0x7fffffff ? 0 : bi;   // a row of NaN only
    } else {
      part_val[blockIdx.y * gridDim.x + blockIdx.x] = best;
      part_idx[blockIdx.y * gridDim.x + blockIdx.x] = bi;
    }
  }
}

// grid rows, one wavefront
__global__ __launch_bounds__(HE_WAVE) void argmax_join_kernel(int32_t* __restrict__ out,
                                                              const float* __restrict__ part_val,
                                                              const int32_t* __restrict__ part_idx,
                                                              int parts) {
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int p = threadIdx.x; p < parts; p += HE_WAVE)
    argmax_take(best, bi, part_val[blockIdx.x * parts + p], part_idx[blockIdx.x * parts + p]);
#pragma unroll
  for (int off = HE_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, HE_WAVE);
    const int oi = __shfl_xor(bi, off, HE_WAVE);
    argmax_take(best, bi, ov, oi);
  }
  if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

extern "C" int64_t he_argmax_workspace_bytes(int rows, int V) {
  if (rows <= 0 || V <= ARGMAX_PART) return 0;
  return (int64_t)rows * ((V + ARGMAX_PART - 1) / ARGMAX_PART) * 8;
}

extern "C" int he_argmax_rows(void* out_i32, const void* logits_f32, int rows, int V,
                              int64_t row_stride, void* workspace, int64_t workspace_bytes,
                              void* stream) {
  HE_REQUIRE(rows >= 0 && V > 0 && row_stride >= V, "he_argmax_rows: bad sizes rows=%d V=%d", rows,
             V);
  HE_REQUIRE(rows <= 65535, "he_argmax_rows: %d rows above 65535", rows);
  if (rows == 0) return 0;
  const int parts = (V + ARGMAX_PART - 1) / ARGMAX_PART;
  const int64_t need = he_argmax_workspace_bytes(rows, V);
  HE_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need),
             "he_argmax_rows: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
             (long long)need);
  float* part_val = (float*)workspace;
  int32_t* part_idx = (int32_t*)workspace + (int64_t)rows * parts;
  hipStream_t s = (hipStream_t)stream;
  argmax_parts_kernel<<<dim3(parts, rows), ARGMAX_THREADS, 0, s>>>(
      (int32_t*)out_i32, part_val, part_idx, (const float*)logits_f32, V, row_stride);
  int rc = he_check_launch("he_argmax_rows");
  if (rc || parts == 1) return rc;
  argmax_join_kernel<<<rows, HE_WAVE, 0, s>>>((int32_t*)out_i32, part_val, part_idx, parts);
  return he_check_launch("he_argmax_rows join");
}

// ---------------------------------------------------------------- penalties
// For each (id, count) of a row's window: logit > 0 ? logit / rep : logit * rep,
// then minus freq * count, minus presence (reference: kernels/sampling.cu:542-565).
// The ids of one row are distinct, so no two threads touch the same logit.
__global__ void penalties_kernel(float* __restrict__ logits, int V, int64_t stride,
                                 const int32_t* __restrict__ ids,
                                 const int32_t* __restrict__ counts,
                                 const int32_t* __restrict__ offsets, float rep, float freq,
                                 float pres) {
  float* x = logits + blockIdx.x * stride;
  const int b = offsets[blockIdx.x], e = offsets[blockIdx.x + 1];
  for (int i = b + threadIdx.x; i < e; i += blockDim.x) {
    const int id = ids[i];
    if (id < 0 || id >= V) continue;
    float v = x[id];
    if (rep != 1.0f) v = v > 0.f ? v / rep : v * rep;
    if (freq != 0.0f) v -= freq * (float)counts[i];
    if (pres != 0.0f) v -= pres;
    x[id] = v;
  }
}

extern "C" int he_apply_penalties(void* logits_f32, int rows, int V, int64_t row_stride,
                                  const void* ids, const void* counts, const void* offsets,
                                  float rep, float freq, float pres, void* stream) {
  HE_REQUIRE(rows >= 0 && V > 0 && row_stride >= V, "he_apply_penalties: bad sizes");
  if (rows == 0) return 0;
  penalties_kernel<<<rows, 128, 0, (hipStream_t)stream>>>(
      (float*)logits_f32, V, row_stride, (const int32_t*)ids, (const int32_t*)counts,
      (const int32_t*)offsets, rep, freq, pres);
  return he_check_launch("he_apply_penalties");
}

// ---------------------------------------------------------------- sampling
typedef unsigned long long u64;

// order-preserving map float -> uint32 (ascending)
__device__ __forceinline__ uint32_t ordered_key(float x) {
  const uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
  const uint32_t b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(b);
}
__device__ __forceinline__ float clean(float x) { return x != x ? -INFINITY : x; }
__device__ __forceinline__ u64 fixed_mass(float x, float m, float inv_temp) {
  const float w = expf((x - m) * inv_temp);
  return (u64)(w * SAMP_FIXED_ONE);
}

// The current candidate set: every element whose key is above `key`, plus the
// first `ties` elements (by index) whose key equals `key`. any == 0: all.
struct Cut {
  uint32_t key;
  uint32_t ties;
  int any;
};

struct SampShared {
  u64 hist[256];
  u64 red[SAMP_THREADS];
  u64 t;
  uint32_t prefix;
  float m;
};

__device__ u64 block_sum_u64(u64 v, SampShared& sh) {
  __syncthreads();
  sh.red[threadIdx.x] = v;
  __syncthreads();
  for (int s = SAMP_THREADS / 2; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) sh.red[threadIdx.x] += sh.red[threadIdx.x + s];
    __syncthreads();
  }
  const u64 r = sh.red[0];
  __syncthreads();
  return r;
}

template <bool MASS>
__device__ u64 set_total(const float* x, int V, float m, float inv_temp, Cut cut,
                         SampShared& sh) {
  u64 local = 0;
  for (int i = threadIdx.x; i < V; i += SAMP_THREADS) {
    const float v = clean(x[i]);
    const uint32_t k = ordered_key(v);
    if (cut.any && k <= cut.key) continue;
    local += MASS ? fixed_mass(v, m, inv_temp) : 1ull;
  }
  if (threadIdx.x == 0 && cut.any)
    local += (MASS ? fixed_mass(key_to_float(cut.key), m, inv_temp) : 1ull) * (u64)cut.ties;
  return block_sum_u64(local, sh);
}

// Finds, in descending order inside `cut`, the element at which the cumulative
// count (MASS = false) or mass (MASS = true) first reaches t (t >= 1), and
// returns the set of everything up to and including it.
template <bool MASS>
__device__ Cut descend(const float* x, int V, float m, float inv_temp, Cut cut, u64 t,
                       SampShared& sh) {
  uint32_t prefix = 0;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    __syncthreads();
    if (threadIdx.x < 256) sh.hist[threadIdx.x] = 0;
    __syncthreads();
    int cur = -1;
    u64 run = 0;
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS) {
      const float v = clean(x[i]);
      const uint32_t k = ordered_key(v);
      if (pass > 0 && (k >> (shift + 8)) != (prefix >> (shift + 8))) continue;
      if (cut.any && k <= cut.key) continue;
      const int b = (k >> shift) & 255;
      if (b != cur) {
        if (cur >= 0) atomicAdd(&sh.hist[cur], run);
        cur = b;
        run = 0;
      }
      run += MASS ? fixed_mass(v, m, inv_temp) : 1ull;
    }
    if (cur >= 0) atomicAdd(&sh.hist[cur], run);
    if (threadIdx.x == 0 && cut.any && cut.ties > 0 &&
        (pass == 0 || (cut.key >> (shift + 8)) == (prefix >> (shift + 8)))) {
      const u64 w = MASS ? fixed_mass(key_to_float(cut.key), m, inv_temp) : 1ull;
      atomicAdd(&sh.hist[(cut.key >> shift) & 255], w * (u64)cut.ties);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      u64 acc = 0;
      int found = -1, last = -1;
      for (int b = 255; b >= 0; --b) {
        const u64 hb = sh.hist[b];
        if (hb == 0) continue;
        last = b;
        if (acc < t && t <= acc + hb) {
          found = b;
          break;
        }
        acc += hb;
      }
      if (found < 0) {  // t beyond the total: end at the last element
        found = last < 0 ? 0 : last;
        t = last < 0 ? 1 : sh.hist[found];
      } else {
        t -= acc;
      }
      sh.prefix = prefix | ((uint32_t)found << shift);
      sh.t = t;
    }
    __syncthreads();
    prefix = sh.prefix;
    t = sh.t;
  }
  const u64 w = MASS ? fixed_mass(key_to_float(prefix), m, inv_temp) : 1ull;
  Cut r;
  r.key = prefix;
  r.any = 1;
  r.ties = (uint32_t)(w > 0 ? (t + w - 1) / w : 1);
  if (r.ties < 1) r.ties = 1;
  if (cut.any && prefix == cut.key && r.ties > cut.ties) r.ties = cut.ties;
  return r;
}

__global__ __launch_bounds__(SAMP_THREADS) void sample_rows_kernel(
    int32_t* __restrict__ out, const float* __restrict__ logits, int V, int64_t stride,
    const uint32_t* __restrict__ uniforms, float inv_temp, int top_k, float top_p) {
  __shared__ SampShared sh;
  __shared__ int s_counts[SAMP_THREADS];
  const float* x = logits + blockIdx.x * stride;

  // row maximum
  float best = -INFINITY;
  for (int i = threadIdx.x; i < V; i += SAMP_THREADS) best = fmaxf(best, clean(x[i]));
  best = wave_max(best);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.red[threadIdx.x >> 6] = (u64)__float_as_uint(best);
  __syncthreads();
  if (threadIdx.x == 0) {
    float mm = -INFINITY;
    for (int w = 0; w < SAMP_THREADS / HE_WAVE; ++w)
      mm = fmaxf(mm, __uint_as_float((uint32_t)sh.red[w]));
    sh.m = mm;
  }
  __syncthreads();
  const float m = sh.m;
  if (!(m > -INFINITY)) {  // nothing finite: fall back to index 0
    if (threadIdx.x == 0) out[blockIdx.x] = 0;
    return;
  }

  Cut cut;
  cut.any = 0;
  cut.key = 0;
  cut.ties = 0;
  if (top_k > 0 && top_k < V) cut = descend<false>(x, V, m, inv_temp, cut, (u64)top_k, sh);
  u64 Z = set_total<true>(x, V, m, inv_temp, cut, sh);
  if (top_p > 0.f && top_p < 1.f) {
    u64 target = (u64)ceil((double)top_p * (double)Z);
    if (target < 1) target = 1;
    if (target > Z) target = Z;
    cut = descend<true>(x, V, m, inv_temp, cut, target, sh);
    Z = set_total<true>(x, V, m, inv_temp, cut, sh);
  }
  // r = floor(u * Z / 2^32), Z < 2^58
  const u64 u = (u64)uniforms[blockIdx.x];
  const u64 r = u * (Z >> 32) + ((u * (Z & 0xffffffffull)) >> 32);
  const Cut pick = descend<true>(x, V, m, inv_temp, cut, r + 1, sh);

  // the pick.ties-th element (by ascending index) whose key equals pick.key
  const int chunk = (V + SAMP_THREADS - 1) / SAMP_THREADS;
  const int b = threadIdx.x * chunk;
  const int e = min(V, b + chunk);
  int cnt = 0;
  for (int i = b; i < e; ++i) cnt += ordered_key(clean(x[i])) == pick.key;
  s_counts[threadIdx.x] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    int want = (int)pick.ties, acc = 0, res = -1;
    for (int th = 0; th < SAMP_THREADS && res < 0; ++th) {
      if (acc + s_counts[th] >= want) {
        const int bb = th * chunk, ee = min(V, bb + chunk);
        for (int i = bb; i < ee; ++i) {
          if (ordered_key(clean(x[i])) == pick.key && ++acc == want) {
            res = i;
            break;
          }
        }
      } else {
        acc += s_counts[th];
      }
    }
    out[blockIdx.x] = res < 0 ? 0 : res;
  }
}

extern "C" int he_sample_rows(void* out_i32, const void* logits_f32, int rows, int V,
                              int64_t row_stride, const void* uniforms_u32, float temperature,
                              int top_k, float top_p, void* stream) {
  HE_REQUIRE(rows >= 0 && V > 0 && row_stride >= V, "he_sample_rows: bad sizes");
  HE_REQUIRE(temperature > 0.f, "he_sample_rows: temperature %g must be positive", temperature);
  if (rows == 0) return 0;
  sample_rows_kernel<<<rows, SAMP_THREADS, 0, (hipStream_t)stream>>>(
      (int32_t*)out_i32, (const float*)logits_f32, V, row_stride, (const uint32_t*)uniforms_u32,
      1.0f / temperature, top_k, top_p);
  return he_check_launch("he_sample_rows");
}
