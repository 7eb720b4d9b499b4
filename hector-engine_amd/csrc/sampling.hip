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
#include <mutex>

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

// Reduces (best, bi) over the wavefront, every lane gets the result: the butterfly lane i with lane
// i ^ 32, 16, 8, 4, 2, 1 through lane swaps and DPP (which of two candidates wins does not depend
// on the order they are compared in). All 64 lanes must be active.
__device__ __forceinline__ void argmax_wave(float& best, int& bi) {
  {
    const auto v = __builtin_amdgcn_permlane32_swap(__float_as_uint(best), __float_as_uint(best), false, false);
    const auto i = __builtin_amdgcn_permlane32_swap((unsigned)bi, (unsigned)bi, false, false);
    best = __uint_as_float(v[0]), bi = (int)i[0];
    argmax_take(best, bi, __uint_as_float(v[1]), (int)i[1]);
  }
  {
    const auto v = __builtin_amdgcn_permlane16_swap(__float_as_uint(best), __float_as_uint(best), false, false);
    const auto i = __builtin_amdgcn_permlane16_swap((unsigned)bi, (unsigned)bi, false, false);
    best = __uint_as_float(v[0]), bi = (int)i[0];
    argmax_take(best, bi, __uint_as_float(v[1]), (int)i[1]);
  }
  argmax_take(best, bi, __uint_as_float(lane_xor_bits<8>(__float_as_uint(best))), (int)lane_xor_bits<8>((unsigned)bi));
  argmax_take(best, bi, __uint_as_float(lane_xor_bits<4>(__float_as_uint(best))), (int)lane_xor_bits<4>((unsigned)bi));
  argmax_take(best, bi, __uint_as_float(lane_xor_bits<2>(__float_as_uint(best))), (int)lane_xor_bits<2>((unsigned)bi));
  argmax_take(best, bi, __uint_as_float(lane_xor_bits<1>(__float_as_uint(best))), (int)lane_xor_bits<1>((unsigned)bi));
}

// Reduces (best, bi) over the workgroup; valid in thread 0.
__device__ __forceinline__ void argmax_block(float& best, int& bi) {
  __shared__ float sval[ARGMAX_THREADS / HE_WAVE];
  __shared__ int sidx[ARGMAX_THREADS / HE_WAVE];
  argmax_wave(best, bi);
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
  const bool vec = V >= 4 && ((stride & 3) == 0) && ((((uintptr_t)logits) & 15) == 0);
  if (vec) {
    // a thread's eight loads of four values go out together (one after the other, each waited for
    // the one before: 8 us a part); a load that would pass the part's end reads the row's start
    // and is not used, the few elements behind the last whole four are taken one by one
    constexpr int LOADS = ARGMAX_PART / (4 * ARGMAX_THREADS);
    float4 v[LOADS];
#pragma unroll
    for (int u = 0; u < LOADS; ++u) {
      const int i = lo + 4 * (int)threadIdx.x + 4 * ARGMAX_THREADS * u;
      v[u] = *reinterpret_cast<const float4*>(x + (i + 4 <= hi ? i : 0));
    }
#pragma unroll
    for (int u = 0; u < LOADS; ++u) {
      const int i = lo + 4 * (int)threadIdx.x + 4 * ARGMAX_THREADS * u;
      if (i + 4 <= hi) {
        argmax_take(best, bi, v[u].x, i);
        argmax_take(best, bi, v[u].y, i + 1);
        argmax_take(best, bi, v[u].z, i + 2);
        argmax_take(best, bi, v[u].w, i + 3);
      } else if (i < hi) {
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
  argmax_wave(best, bi);
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

// The same argmax for callers that cannot allocate: the parts of the rows go into a static
// device array instead of a workspace the caller brings. Host code never uses the array's
// name as an address: each device's copy is looked up once (he_argmax_rows_static_setup, or the
// first call on that device) and the kernels get that pointer.
static __device__ __align__(256) unsigned char he_static_scratch[HE_ARGMAX_STATIC_SCRATCH_BYTES];

#define HE_MAX_DEVICES 64
static std::mutex g_static_mutex;
static void* g_static_ptr[HE_MAX_DEVICES];   // per device: the address of its copy of he_static_scratch

// The current device's copy of the array, or null after recording an error.
static void* static_scratch_of_current_device() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= HE_MAX_DEVICES) {
    he_set_error("he_argmax_rows_static: no current device below %d (%s)", HE_MAX_DEVICES,
                 hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(g_static_mutex);
  if (g_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(he_static_scratch));
    if (e != hipSuccess || p == nullptr) {
      he_set_error("he_argmax_rows_static: hipGetSymbolAddress on device %d: %s", dev,
                   hipGetErrorString(e));
      return nullptr;
    }
    g_static_ptr[dev] = p;
  }
  return g_static_ptr[dev];
}

extern "C" int he_argmax_rows_static_setup(void) {
  return static_scratch_of_current_device() != nullptr ? 0 : -1;
}

extern "C" int he_argmax_rows_static(void* out_i32, const void* logits_f32, int rows, int V,
                                     int64_t row_stride, void* stream) {
  HE_REQUIRE(rows >= 0 && V > 0 && row_stride >= V, "he_argmax_rows_static: bad sizes rows=%d V=%d",
             rows, V);
  HE_REQUIRE(rows <= 65535, "he_argmax_rows_static: %d rows above 65535", rows);
  if (rows == 0) return 0;
  const int parts = (V + ARGMAX_PART - 1) / ARGMAX_PART;
  const int64_t need = he_argmax_workspace_bytes(rows, V);
  HE_REQUIRE(need <= HE_ARGMAX_STATIC_SCRATCH_BYTES,
             "he_argmax_rows_static: %d rows of %d logits need %lld bytes of scratch, the static "
             "array holds %d (use he_argmax_rows with a workspace)",
             rows, V, (long long)need, HE_ARGMAX_STATIC_SCRATCH_BYTES);
  void* scratch = static_scratch_of_current_device();
  if (scratch == nullptr) return -1;
  // every part of every row is written by the first launch before the second reads it:
  // nothing of an earlier call's contents is read, so nothing has to be cleared
  float* part_val = (float*)scratch;
  int32_t* part_idx = (int32_t*)scratch + (int64_t)rows * parts;
  hipStream_t s = (hipStream_t)stream;
  argmax_parts_kernel<<<dim3(parts, rows), ARGMAX_THREADS, 0, s>>>(
      (int32_t*)out_i32, part_val, part_idx, (const float*)logits_f32, V, row_stride);
  int rc = he_check_launch("he_argmax_rows_static");
  if (rc || parts == 1) return rc;
  argmax_join_kernel<<<rows, HE_WAVE, 0, s>>>((int32_t*)out_i32, part_val, part_idx, parts);
  return he_check_launch("he_argmax_rows_static join");
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

// The same penalties from a window of recent tokens that lives on the device, so that a run of
// queued steps needs no token on the host in between: window [rows][W] is a ring (the token
// appended as number n lies at n % W), appended[row] counts what was ever appended. One
// workgroup a row first appends last_ids[row] (the token sampled by the step before; null:
// nothing), then counts the distinct ids among the last min(appended, W) tokens in a hash table
// in LDS (open addressing, twice as many places as the window has tokens: linear in the window)
// and changes each one's logit once, with the arithmetic of penalties_kernel. The result
// depends on the counts alone, not on the order in which the threads meet the ids.
#define PEN_WINDOW_MAX 4096
#define PEN_TABLE_MAX (2 * PEN_WINDOW_MAX)
__global__ __launch_bounds__(256) void penalties_window_kernel(
    float* __restrict__ logits, int V, int64_t stride, int32_t* __restrict__ window,
    int32_t* __restrict__ appended, int W, const int32_t* __restrict__ last_ids, float rep,
    float freq, float pres) {
  __shared__ int32_t keys[PEN_TABLE_MAX];     // -1: free
  __shared__ int32_t counts[PEN_TABLE_MAX];
  float* x = logits + blockIdx.x * stride;
  int32_t* ring = window + (int64_t)blockIdx.x * W;
  int total = appended[blockIdx.x];
  const int fresh = last_ids != nullptr ? last_ids[blockIdx.x] : 0;
  const int at = total % W;
  if (last_ids != nullptr) ++total;
  const int n = total < W ? total : W;
  int places = 64;
  while (places < 2 * n) places <<= 1;        // at most PEN_TABLE_MAX, as n <= W <= PEN_WINDOW_MAX
  for (int i = threadIdx.x; i < places; i += blockDim.x) keys[i] = -1, counts[i] = 0;
  __syncthreads();          // every thread has read the count before it is written
  if (threadIdx.x == 0 && last_ids != nullptr) appended[blockIdx.x] = total;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int id = last_ids != nullptr && i == at ? fresh : ring[i];
    if (last_ids != nullptr && i == at) ring[at] = fresh;
    if (id < 0 || id >= V) continue;
    unsigned h = ((unsigned)id * 2654435761u) >> 7;
    for (int probe = 0; probe < places; ++probe, ++h) {   // a free place exists: the table is at most half full
      const int slot = h & (places - 1);
      const int seen = atomicCAS(&keys[slot], -1, id);
      if (seen == -1 || seen == id) {
        atomicAdd(&counts[slot], 1);
        break;
      }
    }
  }
  __syncthreads();
  for (int slot = threadIdx.x; slot < places; slot += blockDim.x) {
    const int id = keys[slot];
    if (id < 0) continue;
    float v = x[id];
    if (rep != 1.0f) v = v > 0.f ? v / rep : v * rep;
    if (freq != 0.0f) v -= freq * (float)counts[slot];
    if (pres != 0.0f) v -= pres;
    x[id] = v;
  }
}

extern "C" int he_apply_penalties_window(void* logits_f32, int rows, int V, int64_t row_stride,
                                         void* window_i32, void* appended_i32, int W,
                                         const void* last_ids_i32, float rep, float freq, float pres,
                                         void* stream) {
  HE_REQUIRE(rows >= 0 && V > 0 && row_stride >= V, "he_apply_penalties_window: bad sizes");
  HE_REQUIRE(W >= 1 && W <= PEN_WINDOW_MAX, "he_apply_penalties_window: a window of %d tokens (1 to %d)", W,
             PEN_WINDOW_MAX);
  HE_REQUIRE(window_i32 != nullptr && appended_i32 != nullptr, "he_apply_penalties_window: no window");
  if (rows == 0) return 0;
  penalties_window_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(
      (float*)logits_f32, V, row_stride, (int32_t*)window_i32, (int32_t*)appended_i32, W,
      (const int32_t*)last_ids_i32, rep, freq, pres);
  return he_check_launch("he_apply_penalties_window");
}

// ---------------------------------------------------------------- sampling
typedef unsigned long long u64;

// order-preserving map float -> uint32 (ascending)
__device__ __forceinline__ uint32_t ordered_key(float x) {
  const uint32_t b = __float_as_uint(x);
  return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);   // negative: all bits turned; else the sign bit set
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
  const uint32_t b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(b);
}
// NaN counts as -inf; -0.0 becomes +0.0, which it equals: as keys the two would differ, and equal
// values are ordered by index alone.
// (x + 0 turns -0.0 into +0.0 and leaves everything else; the maximum with -inf is -inf for a NaN)
__device__ __forceinline__ float clean(float x) { return fmaxf(x + 0.f, -INFINITY); }
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
  int few;      // elements gathered by choose_few
};

// Exact (integer) sum over the workgroup: wavefronts first, then their 16 sums in order.
__device__ u64 block_sum_u64(u64 v, SampShared& sh) {
#pragma unroll
  for (int off = HE_WAVE / 2; off > 0; off >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)v, off, HE_WAVE);
    const uint32_t hi = __shfl_xor((uint32_t)(v >> 32), off, HE_WAVE);
    v += ((u64)hi << 32) | lo;
  }
  __syncthreads();
  if ((threadIdx.x & (HE_WAVE - 1)) == 0) sh.red[threadIdx.x >> 6] = v;
  __syncthreads();
  u64 r = 0;
  for (int w = 0; w < SAMP_THREADS / HE_WAVE; ++w) r += sh.red[w];
  __syncthreads();
  return r;
}

// Where the elements come from: the whole row in global memory, or a list in LDS of the
// row's largest elements (value and index), in no particular order.
// for_each(f): f(value, index) for every element, the workgroup's threads sharing them out.
struct RowSource {
  const float* x;
  int n;
  // Four 16-byte loads of a thread are on their way at a time where the row allows them: with
  // one 4-byte load a turn a pass over a row of 152,064 waits 148 times for memory (50 us; the
  // passes of a nearly flat row, whose draw lies beyond the list, took 340 us together).
  template <typename F>
  __device__ __forceinline__ void for_each(F&& f) const {
    int done = 0;
    if ((((uintptr_t)x) & 15) == 0) {
      done = n & ~3;
      for (int i0 = 4 * threadIdx.x; i0 < done; i0 += 16 * SAMP_THREADS) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 4 * SAMP_THREADS;
          v[u] = *reinterpret_cast<const float4*>(x + (i < done ? i : i0));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 4 * SAMP_THREADS;
          if (i < done) {
            f(clean(v[u].x), i);
            f(clean(v[u].y), i + 1);
            f(clean(v[u].z), i + 2);
            f(clean(v[u].w), i + 3);
          }
        }
      }
    }
    for (int i = done + threadIdx.x; i < n; i += SAMP_THREADS) f(clean(x[i]), i);
  }
};
struct ListSource {   // n slots; a slot with index -1 is empty
  const float* v;
  const int* idx;
  int n;
  template <typename F>
  __device__ __forceinline__ void for_each(F&& f) const {
    for (int i = threadIdx.x; i < n; i += SAMP_THREADS)
      if (idx[i] >= 0) f(v[i], idx[i]);
  }
};

template <bool MASS, typename Source>
__device__ u64 set_total(const Source& src, float m, float inv_temp, Cut cut, SampShared& sh) {
  u64 local = 0;
  src.for_each([&](float v, int) {
    if (cut.any && ordered_key(v) <= cut.key) return;
    local += MASS ? fixed_mass(v, m, inv_temp) : 1ull;
  });
  if (threadIdx.x == 0 && cut.any)
    local += (MASS ? fixed_mass(key_to_float(cut.key), m, inv_temp) : 1ull) * (u64)cut.ties;
  return block_sum_u64(local, sh);
}

// Adds every lane's pending (bin, run) to the histogram. Lanes of a wavefront that hold the
// same bin - all of them in the passes over the upper key bytes - are summed first and one
// lane adds the sum: a thousand 64-bit LDS atomics on one address take tens of microseconds.
// Where the lanes' bins differ (the passes over the lower key bytes) that summing, a dozen
// exchanges across the wavefront a bin, would be the slow part: once a bin is shared by fewer
// than eight lanes, or three bins have been dealt with, the lanes left add their own.
__device__ __forceinline__ void flush_runs(u64* hist, int bin, u64 run) {
  const int lane = threadIdx.x & (HE_WAVE - 1);
  unsigned long long pending = __builtin_amdgcn_ballot_w64(bin >= 0);
  int dealt = 0;
  while (pending) {
    const int leader = __builtin_ctzll(pending);
    const int lb = __shfl(bin, leader, HE_WAVE);
    const bool same = bin == lb;
    const unsigned long long sharing = __builtin_amdgcn_ballot_w64(same);
    if (__builtin_popcountll(sharing) < 8 || dealt == 3) {
      if ((pending >> lane) & 1ull) atomicAdd(&hist[bin], run);
      return;
    }
    u64 v = same ? run : 0ull;
#pragma unroll
    for (int off = HE_WAVE / 2; off > 0; off >>= 1) {
      const uint32_t lo = __shfl_xor((uint32_t)v, off, HE_WAVE);
      const uint32_t hi = __shfl_xor((uint32_t)(v >> 32), off, HE_WAVE);
      v += ((u64)hi << 32) | lo;
    }
    if (lane == leader) atomicAdd(&hist[lb], v);
    pending &= ~sharing;
    ++dealt;
  }
}

// Finds, in descending order inside `cut`, the element at which the cumulative
// count (MASS = false) or mass (MASS = true) first reaches t (t >= 1), and
// returns the set of everything up to and including it.
// passes < 4: the descent stops with the upper 8 * passes bits of the key (the lower ones zero): the
// key of the bin the element lies in, for a caller that wants a bound and not the element.
template <bool MASS, typename Source>
__device__ Cut descend(const Source& src, float m, float inv_temp, Cut cut, u64 t,
                       SampShared& sh, int passes = 4) {
  uint32_t prefix = 0;
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = 24 - 8 * pass;
    __syncthreads();
    if (threadIdx.x < 256) sh.hist[threadIdx.x] = 0;
    __syncthreads();
    int cur = -1;
    u64 run = 0;
    src.for_each([&](float v, int) {
      const uint32_t k = ordered_key(v);
      if (pass > 0 && (k >> (shift + 8)) != (prefix >> (shift + 8))) return;
      if (cut.any && k <= cut.key) return;
      const int b = (k >> shift) & 255;
      if (b != cur) {
        if (cur >= 0) atomicAdd(&sh.hist[cur], run);
        cur = b;
        run = 0;
      }
      run += MASS ? fixed_mass(v, m, inv_temp) : 1ull;
    });
    flush_runs(sh.hist, cur, run);
    if (threadIdx.x == 0 && cut.any && cut.ties > 0 &&
        (pass == 0 || (cut.key >> (shift + 8)) == (prefix >> (shift + 8)))) {
      const u64 w = MASS ? fixed_mass(key_to_float(cut.key), m, inv_temp) : 1ull;
      atomicAdd(&sh.hist[(cut.key >> shift) & 255], w * (u64)cut.ties);
    }
    __syncthreads();
    if (threadIdx.x < HE_WAVE) {
      // Walk the bins from 255 down to the one in which the running total reaches t: lane l
      // owns bins 4l..4l+3, a suffix sum over the lanes gives what lies above each, one lane
      // finds the crossing among its four.
      const int lane = threadIdx.x;
      u64 h[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) h[j] = sh.hist[4 * lane + j];
      const u64 mine = (h[0] + h[1]) + (h[2] + h[3]);
      u64 incl = mine;
#pragma unroll
      for (int off = 1; off < HE_WAVE; off <<= 1) {
        const uint32_t lo = __shfl_down((uint32_t)incl, off, HE_WAVE);
        const uint32_t hi = __shfl_down((uint32_t)(incl >> 32), off, HE_WAVE);
        if (lane + off < HE_WAVE) incl += ((u64)hi << 32) | lo;
      }
      const u64 above = incl - mine;
      const bool has = mine > 0 && above < t && t <= above + mine;
      const unsigned long long crossing = __builtin_amdgcn_ballot_w64(has);
      const unsigned long long filled = __builtin_amdgcn_ballot_w64(mine > 0);
      if (crossing) {
        if (has) {
          u64 acc = above;
          for (int j = 3; j >= 0; --j) {
            if (h[j] == 0) continue;
            if (acc < t && t <= acc + h[j]) {
              sh.prefix = prefix | ((uint32_t)(4 * lane + j) << shift);
              sh.t = t - acc;
              break;
            }
            acc += h[j];
          }
        }
      } else if (filled) {   // t beyond the total: end at the last (lowest) element
        if (lane == __builtin_ctzll(filled)) {
          int j = 0;
          while (h[j] == 0) ++j;
          sh.prefix = prefix | ((uint32_t)(4 * lane + j) << shift);
          sh.t = h[j];
        }
      } else if (lane == 0) {
        sh.prefix = prefix;
        sh.t = 1;
      }
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

// For a lane's four elements from i on (i a multiple of 4), four such groups 256 elements apart:
// bit c of mk[u] says that element i + 256 u + c lies before `e` and has the key. The loads of
// the four groups go out together.
__device__ __forceinline__ void row_masks(const float* x, int V, bool vec, int e, int i0,
                                          uint32_t key, int mk[4]) {
  const int full = vec ? (V & ~3) : 0;      // 16-byte loads stay before this index
  float4 q[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int i = i0 + 256 * u;
    q[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (full > 0) q[u] = *reinterpret_cast<const float4*>(x + (i < full && i < e ? i : 0));
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int i = i0 + 256 * u;
    int m = 0;
    if (i < e) {
      if (i < full) {      // (e is a multiple of 256 or V itself: the four lie before it)
        m = (int)(ordered_key(clean(q[u].x)) == key) | (int)(ordered_key(clean(q[u].y)) == key) << 1 |
            (int)(ordered_key(clean(q[u].z)) == key) << 2 | (int)(ordered_key(clean(q[u].w)) == key) << 3;
      } else {
        for (int c = 0; c < 4; ++c)
          if (i + c < e) m |= (int)(ordered_key(clean(x[i + c])) == key) << c;
      }
    }
    mk[u] = m;
  }
}

// The index of the pick.ties-th element, by ascending index, whose key equals pick.key. Every
// wavefront counts the equal keys of a stretch of the row (256 elements a load, so that the
// lanes read neighbouring addresses; a thread walking a stretch of its own read 64 cache lines
// an instruction: 140 us for a row of 152,064); the wavefront in whose stretch the wanted one
// lies walks it again and finds it through the lanes' counts.
__device__ int pick_index_row(const float* x, int V, Cut pick, int* s_counts) {
  __shared__ int s_res;
  constexpr int WAVES = SAMP_THREADS / HE_WAVE;
  const int lane = threadIdx.x & (HE_WAVE - 1), wave = threadIdx.x >> 6;
  const bool vec = (((uintptr_t)x) & 15) == 0;
  const int stretch = ((V + WAVES - 1) / WAVES + 255) & ~255;
  const int b = min(V, wave * stretch), e = min(V, b + stretch);
  int cnt = 0;
  for (int i0 = b + 4 * lane; i0 < e; i0 += 1024) {
    int mk[4];
    row_masks(x, V, vec, e, i0, pick.key, mk);
    cnt += __builtin_popcount(mk[0]) + __builtin_popcount(mk[1]) + __builtin_popcount(mk[2]) +
           __builtin_popcount(mk[3]);
  }
#pragma unroll
  for (int off = HE_WAVE / 2; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off, HE_WAVE);
  __syncthreads();
  if (lane == 0) s_counts[wave] = cnt;
  if (threadIdx.x == 0) s_res = 0;              // fewer equal keys than the rank: index 0
  __syncthreads();
  int want = (int)pick.ties, holder = -1;
  for (int w = 0; w < WAVES && holder < 0; ++w) {
    if (want <= s_counts[w]) holder = w;
    else want -= s_counts[w];
  }
  if (wave == holder) {
    const unsigned long long below = (1ull << lane) - 1ull;
    int passed = 0;
    bool found = false;
    for (int i0 = b + 4 * lane; i0 - 4 * lane < e && !found; i0 += 1024) {   // (the same turns in every lane)
      int mk[4];
      row_masks(x, V, vec, e, i0, pick.key, mk);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (found) continue;
        const int c = __builtin_popcount(mk[u]);
        int before = 0, total = 0;
#pragma unroll
        for (int bit = 0; bit < 3; ++bit) {       // a lane has at most 4
          const unsigned long long with = __builtin_amdgcn_ballot_w64((c >> bit) & 1);
          before += __builtin_popcountll(with & below) << bit;
          total += __builtin_popcountll(with) << bit;
        }
        if (passed + total >= want) {
          const int rank = want - passed - before;      // among this lane's: 1 .. c if it is here
          if (rank >= 1 && rank <= c) {
            int m = mk[u];
            for (int k = 1; k < rank; ++k) m &= m - 1;
            s_res = i0 + 256 * u + __builtin_ctz(m);
          }
          found = true;
        }
        passed += total;
      }
    }
  }
  __syncthreads();
  return s_res;
}

// The same on a list, for a small rank: the lowest index among the equal keys, then the
// next one, ... `ties` times. Returns -1 when the rank is not small (the caller then walks
// the row).
#define SAMP_PICK_ROUNDS 16
__device__ int pick_index_list(const ListSource& src, Cut pick, SampShared& sh) {
  if (pick.ties > SAMP_PICK_ROUNDS) return -1;
  int after = -1;
  for (uint32_t round = 0; round < pick.ties; ++round) {
    int best = 0x7fffffff;
    for (int i = threadIdx.x; i < src.n; i += SAMP_THREADS) {
      const int id = src.idx[i];
      if (id > after && id < best && ordered_key(src.v[i]) == pick.key) best = id;
    }
#pragma unroll
    for (int off = HE_WAVE / 2; off > 0; off >>= 1) best = min(best, __shfl_xor(best, off, HE_WAVE));
    __syncthreads();
    if ((threadIdx.x & (HE_WAVE - 1)) == 0) sh.red[threadIdx.x >> 6] = (u64)(uint32_t)best;
    __syncthreads();
    for (int w = 0; w < SAMP_THREADS / HE_WAVE; ++w) best = min(best, (int)(uint32_t)sh.red[w]);
    __syncthreads();
    if (best == 0x7fffffff) return 0;   // fewer equal keys than the rank: not for a consistent pick
    after = best;
  }
  return after;
}

__device__ __forceinline__ u64 shfl_xor_u64(u64 v, int mask) {
  const uint32_t lo = __shfl_xor((uint32_t)v, mask, HE_WAVE);
  const uint32_t hi = __shfl_xor((uint32_t)(v >> 32), mask, HE_WAVE);
  return ((u64)hi << 32) | lo;
}
__device__ __forceinline__ u64 shfl_u64(u64 v, int lane) {
  const uint32_t lo = __shfl((uint32_t)v, lane, HE_WAVE);
  const uint32_t hi = __shfl((uint32_t)(v >> 32), lane, HE_WAVE);
  return ((u64)hi << 32) | lo;
}

// top-p and the draw after a top-k of at most a wavefront's width, in one wavefront: the
// elements at or above the top-k's last key (`cut.key`) go one to a lane, are sorted by
// descending value and ascending index, the first top_k of them keep their mass, and a
// running sum over the lanes stands for the descents (12 passes over the list otherwise:
// 20 us of a sampled step). The order and the masses are those of the descents, so the token
// is the same. Returns false, with nothing decided, when more than a wavefront's width of
// elements lie at or above that key (many ties at it).
template <typename Source>
__device__ bool choose_few(const Source& src, float m, float inv_temp, int top_k, float top_p,
                           u64 u, Cut cut, SampShared& sh, int* index_out) {
  __syncthreads();
  if (threadIdx.x == 0) sh.few = 0;
  __syncthreads();
  src.for_each([&](float v, int index) {
    const uint32_t k = ordered_key(v);
    if (k < cut.key) return;
    const int at = atomicAdd(&sh.few, 1);
    if (at < HE_WAVE) sh.hist[at] = ((u64)k << 32) | (u64)(0xffffffffu - (uint32_t)index);
  });
  __syncthreads();
  const int n = sh.few;
  if (n > HE_WAVE) return false;
  if (threadIdx.x < HE_WAVE) {
    const int lane = threadIdx.x;
    u64 e = lane < n ? sh.hist[lane] : 0ull;     // (an empty lane sorts behind every element)
    // bitonic sort, descending over the lanes
#pragma unroll
    for (int size = 2; size <= HE_WAVE; size <<= 1) {
#pragma unroll
      for (int stride = size >> 1; stride > 0; stride >>= 1) {
        const u64 other = shfl_xor_u64(e, stride);
        const bool descending = (lane & size) == 0;
        const bool first = (lane & stride) == 0;
        const u64 hi = e > other ? e : other, lo = e > other ? other : e;
        e = (first == descending) ? hi : lo;
      }
    }
    const float v = key_to_float((uint32_t)(e >> 32));
    const u64 mass = lane < top_k && lane < n ? fixed_mass(v, m, inv_temp) : 0ull;
    u64 upto = mass;                             // inclusive running sum
#pragma unroll
    for (int off = 1; off < HE_WAVE; off <<= 1) {
      const uint32_t lo = __shfl_up((uint32_t)upto, off, HE_WAVE);
      const uint32_t hi = __shfl_up((uint32_t)(upto >> 32), off, HE_WAVE);
      if (lane >= off) upto += ((u64)hi << 32) | lo;
    }
    u64 Z = shfl_u64(upto, HE_WAVE - 1);
    int last = HE_WAVE - 1;                      // the last lane of the kept set
    if (top_p > 0.f && top_p < 1.f) {
      u64 target = (u64)ceil((double)top_p * (double)Z);
      if (target < 1) target = 1;
      if (target > Z) target = Z;
      const unsigned long long reached = __builtin_amdgcn_ballot_w64(upto >= target);
      last = __builtin_ctzll(reached);           // (Z > 0: the row's maximum is among the elements)
      Z = shfl_u64(upto, last);
    }
    const u64 r = u * (Z >> 32) + ((u * (Z & 0xffffffffull)) >> 32);
    const unsigned long long reached = __builtin_amdgcn_ballot_w64(lane <= last && upto >= r + 1);
    const int pick = reached ? __builtin_ctzll(reached) : 0;
    const u64 chosen = shfl_u64(e, pick);
    if (lane == 0) sh.prefix = 0xffffffffu - (uint32_t)chosen;
  }
  __syncthreads();
  *index_out = (int)sh.prefix;
  return true;
}

// top-k, top-p and the draw on one source. rest: mass of the row's elements that are not
// in the source (they all come after every element of the source in descending order).
// Returns false when the answer needs elements outside the source (rest > 0 only).
template <typename Source>
__device__ bool choose(const Source& src, float m, float inv_temp, int top_k, float top_p, int V,
                       u64 u, u64 rest, SampShared& sh, Cut* pick_out, int* index_out) {
  Cut cut;
  cut.any = 0;
  cut.key = 0;
  cut.ties = 0;
  *index_out = -1;
  if (top_k > 0 && top_k < V) {
    if ((u64)top_k > set_total<false>(src, m, inv_temp, cut, sh)) return false;
    cut = descend<false>(src, m, inv_temp, cut, (u64)top_k, sh);
    rest = 0;   // the set is inside the source
    if (top_k <= HE_WAVE && choose_few(src, m, inv_temp, top_k, top_p, u, cut, sh, index_out)) return true;
  }
  u64 inside = set_total<true>(src, m, inv_temp, cut, sh);
  u64 Z = inside + rest;
  if (top_p > 0.f && top_p < 1.f) {
    u64 target = (u64)ceil((double)top_p * (double)Z);
    if (target < 1) target = 1;
    if (target > Z) target = Z;
    if (target > inside) return false;
    cut = descend<true>(src, m, inv_temp, cut, target, sh);
    inside = set_total<true>(src, m, inv_temp, cut, sh);
    Z = inside;
  }
  // r = floor(u * Z / 2^32), Z < 2^58
  const u64 r = u * (Z >> 32) + ((u * (Z & 0xffffffffull)) >> 32);
  if (r + 1 > inside) return false;
  *pick_out = descend<true>(src, m, inv_temp, cut, r + 1, sh);
  return true;
}

// One workgroup per row. Two passes over the row: (1) its maximum; (2) its largest
// elements - all whose key is at least a threshold - go into a list in LDS, and the mass
// of all others is summed. The threshold is the value that a strided sample of the row
// puts at the rank which aims at SAMP_AIM list elements (the list holds twice that; a row
// no longer than the list goes in whole). With a top-k nobody asks for the mass of the
// others, and the maximum is taken in the list pass: one pass over the row. top-k, top-p
// and the draw then run on the list (behind a top-k of at most 64 in one wavefront:
// choose_few). When they need more than the list holds (a top-k beyond it, a nucleus or a
// draw that reaches into the rest, a list that overflowed) the same steps run on the whole
// row instead, many passes over it: rare for the peaked rows of a trained model (the rule
// for nearly flat rows without a top-k, as random weights give them), and the result is
// the same either way.
#define SAMP_LIST 6144
#define SAMP_AIM 3072
#define SAMP_SAMPLE 4096

__global__ __launch_bounds__(SAMP_THREADS) void sample_rows_kernel(
    int32_t* __restrict__ out, const float* __restrict__ logits, int V, int64_t stride,
    const uint32_t* __restrict__ uniforms, float inv_temp, int top_k, float top_p) {
  __shared__ SampShared sh;
  __shared__ int s_counts[SAMP_THREADS];
  __shared__ float list_v[SAMP_LIST];
  __shared__ int list_i[SAMP_LIST];
  __shared__ int list_n;
  const float* x = logits + blockIdx.x * stride;

  const bool aligned = ((stride & 3) == 0) && ((((uintptr_t)logits) & 15) == 0);
  // With a top-k the kept set lies inside the list (or the whole row is walked instead) and the
  // mass of the rest is never asked for: its 150,000 exponentials, most of the list pass, are left
  // out, and the row's maximum, which nothing before the list needs then, is taken in that pass.
  const bool need_rest = !(top_k > 0 && top_k < V);
  const bool max_with_list = !need_rest && V > SAMP_LIST && aligned;

  // the workgroup's maximum of `best`; false (index 0 stored) when the row has nothing finite
  auto row_max = [&](float best, float* m_out) -> bool {
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
    *m_out = sh.m;
    if (!(sh.m > -INFINITY)) {
      if (threadIdx.x == 0) out[blockIdx.x] = 0;
      return false;
    }
    return true;
  };

  // pass 1: row maximum
  float best = -INFINITY, m = -INFINITY;
  if (!max_with_list) {
    if (aligned) {
      // four loads on their way at a time: one workgroup reads the whole row, and a load takes
      // about a microsecond (more in flight gain nothing: a compute unit alone takes in about 64
      // bytes a cycle, 4.5 us for a row of 152,064)
      const int V4 = V & ~3;
      for (int i0 = 4 * threadIdx.x; i0 < V4; i0 += 16 * SAMP_THREADS) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 4 * SAMP_THREADS;
          v[u] = i < V4 ? *reinterpret_cast<const float4*>(x + i) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          best = fmaxf(fmaxf(best, clean(v[u].x)), fmaxf(clean(v[u].y), fmaxf(clean(v[u].z), clean(v[u].w))));
      }
      for (int i = V4 + threadIdx.x; i < V; i += SAMP_THREADS) best = fmaxf(best, clean(x[i]));
    } else {
      for (int i = threadIdx.x; i < V; i += SAMP_THREADS) best = fmaxf(best, clean(x[i]));
    }
    if (!row_max(best, &m)) return;   // nothing finite: index 0
  }
  const u64 u = (u64)uniforms[blockIdx.x];
  Cut pick;

  // the threshold key of the list
  uint32_t threshold = 0;
  if (V > SAMP_LIST) {
    const int n = SAMP_SAMPLE;
    for (int j = threadIdx.x; j < n; j += SAMP_THREADS) {
      list_v[j] = clean(x[(int)(((int64_t)j * V) / n)]);
      list_i[j] = j;
    }
    __syncthreads();
    ListSource sample;
    sample.v = list_v;
    sample.idx = list_i;
    sample.n = n;
    Cut none;
    none.any = 0;
    none.key = 0;
    none.ties = 0;
    // the upper 24 bits of the key at that rank are bound enough: the list then takes the whole bin,
    // 2^-15 of the value wide, a handful of elements more
    const u64 rank = ((u64)n * SAMP_AIM + V - 1) / V + 1;
    threshold = descend<false>(sample, 0.f, inv_temp, none, rank, sh, 3).key;
    __syncthreads();
  }

  // pass 2: the list and the mass of the rest. Every wavefront fills a segment of its own;
  // the slot of an element follows from the ballot of the lanes that append in this turn, so
  // the wavefronts neither wait for one another nor for a counter in memory.
  constexpr int SEGMENT = SAMP_LIST / (SAMP_THREADS / HE_WAVE);
  for (int i = threadIdx.x; i < SAMP_LIST; i += SAMP_THREADS) list_i[i] = -1;
  if (threadIdx.x == 0) list_n = 0;   // becomes 1 when a segment overflows
  __syncthreads();
  const int lane = threadIdx.x & (HE_WAVE - 1), wave = threadIdx.x >> 6;
  int filled = 0;                     // the same in all lanes of the wavefront
  u64 rest_local = 0;
  auto take = [&](float raw, int i, bool in_range) {
    const float v = clean(raw);
    const bool mine = in_range && ordered_key(v) >= threshold;
    const unsigned long long appenders = __builtin_amdgcn_ballot_w64(mine);
    if (mine) {
      const int at = filled + __builtin_popcountll(appenders & ((1ull << lane) - 1ull));
      if (at < SEGMENT) {
        list_v[wave * SEGMENT + at] = v;
        list_i[wave * SEGMENT + at] = i;
      }
    } else if (in_range && need_rest) {
      rest_local += fixed_mass(v, m, inv_temp);
    }
    filled += __builtin_popcountll(appenders);
  };
  if (V > SAMP_LIST && aligned) {
    // 16 bytes a load, four loads a group, the next group on its way while this one is looked
    // at; all lanes of a wavefront make the same number of turns
    const int V4 = V & ~3;
    constexpr int STEP = 4 * SAMP_THREADS;
    const int groups = (V4 + 4 * STEP - 1) / (4 * STEP);
    int i = 4 * threadIdx.x;
    float4 cur[4], nxt[4];
    auto load_group = [&](float4 (&g)[4], int at) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        g[u] = at + u * STEP < V4 ? *reinterpret_cast<const float4*>(x + at + u * STEP) : make_float4(0.f, 0.f, 0.f, 0.f);
    };
    load_group(cur, i);
    const unsigned long long below = (1ull << lane) - 1ull;     // the lanes in front of this one
    for (int gi = 0; gi < groups; ++gi) {
      load_group(nxt, i + 4 * STEP);
      // A lane's sixteen elements of the group as a bit mask of those that go into the list (two in
      // a hundred do); where the lane's first one goes follows from the counts of the lanes in front
      // of it, taken bit by bit of the count through ballots: one such sum a group, not one ballot an
      // element. The few elements that go are then fetched again by their index.
      uint32_t mask = 0;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool in = i + u * STEP < V4;
        const float c4[4] = {cur[u].x, cur[u].y, cur[u].z, cur[u].w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const float v = clean(c4[c]);
          if (in) best = fmaxf(best, v);      // (the row's maximum, where no pass before this one took it)
          const bool mine = in && ordered_key(v) >= threshold;
          mask |= (uint32_t)mine << (4 * u + c);
          if (need_rest && in && !mine) rest_local += fixed_mass(v, m, inv_temp);
        }
      }
      const int count = __builtin_popcount(mask);
      int before = 0, total = 0;
#pragma unroll
      for (int bit = 0; bit < 5; ++bit) {       // a lane has at most 16
        const unsigned long long with = __builtin_amdgcn_ballot_w64((count >> bit) & 1);
        before += __builtin_popcountll(with & below) << bit;
        total += __builtin_popcountll(with) << bit;
      }
      int at = filled + before;
      for (uint32_t left = mask; left != 0; left &= left - 1) {
        const int e = __builtin_ctz(left);
        const int idx = i + (e >> 2) * STEP + (e & 3);
        if (at < SEGMENT) {
          list_v[wave * SEGMENT + at] = clean(x[idx]);
          list_i[wave * SEGMENT + at] = idx;
        }
        ++at;
      }
      filled += total;
#pragma unroll
      for (int u = 0; u < 4; ++u) cur[u] = nxt[u];
      i += 4 * STEP;
    }
    const int j = V4 + threadIdx.x;
    if (j < V) best = fmaxf(best, clean(x[j]));
    take(j < V ? x[j] : 0.f, j, j < V);   // at most three elements are left
  } else {
    const int turns = (V + SAMP_THREADS - 1) / SAMP_THREADS;
    for (int t = 0; t < turns; ++t) {
      const int i = threadIdx.x + t * SAMP_THREADS;
      take(i < V ? x[i] : 0.f, i, i < V);
    }
  }
  if (lane == 0 && filled > SEGMENT) list_n = 1;
  if (max_with_list && !row_max(best, &m)) return;
  const u64 rest = block_sum_u64(rest_local, sh);   // its barriers also publish list_n
  ListSource list;
  list.v = list_v;
  list.idx = list_i;
  list.n = SAMP_LIST;
  int res;                             // the token, where choose() found it itself; else -1
  if (list_n == 0 && choose(list, m, inv_temp, top_k, top_p, V, u, rest, sh, &pick, &res)) {
    if (res < 0) res = pick_index_list(list, pick, sh);
    if (res < 0) res = pick_index_row(x, V, pick, s_counts);
    if (threadIdx.x == 0) out[blockIdx.x] = res;
    return;
  }
  RowSource row;
  row.x = x;
  row.n = V;
  choose(row, m, inv_temp, top_k, top_p, V, u, 0, sh, &pick, &res);
  if (res < 0) res = pick_index_row(x, V, pick, s_counts);
  if (threadIdx.x == 0) out[blockIdx.x] = res;
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
