// Shared helpers of the gfx950 kernel library: storage types, conversions,
// wave/block reductions and the error channel of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// dtype codes used across the C ABI
#define HE_F32 0
#define HE_BF16 1
#define HE_F16 2   // as the stored dtype of an uploaded tensor only

// Tokens per page of the key/value cache. Both pools are [page][kv_head][elements of a page];
// inside a page the elements lie in the order the MFMA attention kernels read their operands
// (cache_layout.h: K as [half][key tile][k step][lane][8], V as [half][dim tile][lane][8]).
#define HE_PAGE_TOKENS 64
#define HE_PAGE_SHIFT 6

#define HE_WAVE 64
// L2 domains (XCDs) of the part; consecutive workgroups of a launch go to them in turn
#define HE_XCDS 8
// compute units of the MI355X: the default of he_cus(), and what the prompt attention's order of
// work inside the kernel is written for
#define HE_CUS 256

struct bf16_t {
  uint16_t v;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// two floats to two bf16 in one register, round to nearest even (v_cvt_pk_bf16_f32)
typedef __bf16 he_bf16x2 __attribute__((ext_vector_type(2)));
typedef float he_float2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  const he_float2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, he_bf16x2));
}

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return bf16_bits_to_float(x.v); }

template <typename T>
__device__ __forceinline__ T from_float(float f);
template <>
__device__ __forceinline__ float from_float<float>(float f) {
  return f;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  bf16_t r;
  r.v = float_to_bf16_bits(f);
  return r;
}

// A small parameter vector (norm gain, bias) may be stored in either dtype
// independently of the activation dtype.
__device__ __forceinline__ float load_param(const void* p, int64_t i, int dtype) {
  return dtype == HE_BF16 ? bf16_bits_to_float(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}

// sin and cos of an fp32 angle to fp32 accuracy: the quadrant is taken off in double
// (k = rint(a * 2/pi), r = a - k * pi/2, |r| <= pi/4), the two short series are summed
// in double and rounded once. The library routine's path for large arguments is far
// slower, and angles here reach tens of thousands of radians.
__device__ __forceinline__ void sincos_angle(float a, float* sn, float* cs) {
  const double x = (double)a;
  const double k = rint(x * 0.63661977236758134308);
  const double r = fma(-k, 6.123233995736766036e-17, fma(-k, 1.57079632679489655800, x));
  const double r2 = r * r;
  const double sp = r * (1.0 + r2 * (-1.0 / 6 + r2 * (1.0 / 120 + r2 * (-1.0 / 5040 + r2 * (1.0 / 362880 + r2 * (-1.0 / 39916800))))));
  const double cp = 1.0 + r2 * (-0.5 + r2 * (1.0 / 24 + r2 * (-1.0 / 720 + r2 * (1.0 / 40320 + r2 * (-1.0 / 3628800 + r2 * (1.0 / 479001600))))));
  const int q = (int)((long long)k & 3);
  const double sv = (q & 1) ? cp : sp;
  const double cv = (q & 1) ? sp : cp;
  *sn = (float)((q & 2) ? -sv : sv);
  *cs = (float)(((q + 1) & 2) ? -cv : cv);
}

// Exchange across the halves (32 lanes) or across neighbouring rows of 16 lanes with the
// gfx950 lane-swap instructions: a vector-ALU move, where __shfl_xor goes through the LDS
// crossbar with five instructions of address arithmetic. Both lanes of a pair get the
// same operands, so sums are bit-identical in both.
__device__ __forceinline__ float max_plain(float a, float b) {   // operands are never NaN here
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float xor32_max(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return max_plain(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor16_max(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return max_plain(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor16_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The value of lane i ^ 8, 4, 2, 1 through the data-parallel path of the vector ALU (DPP): a
// rotation by 8 inside a row of 16 lanes; the mirror image of a half row, then of its quads;
// permutations inside a quad. All 64 lanes must be active.
template <int CTRL>
__device__ __forceinline__ unsigned dpp_bits(unsigned x) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xF, 0xF, false);
}
// OFF: 8, 4, 2 or 1
template <int OFF>
__device__ __forceinline__ unsigned lane_xor_bits(unsigned x) {
  static_assert(OFF == 8 || OFF == 4 || OFF == 2 || OFF == 1, "lane_xor_bits: 8, 4, 2 or 1");
  if (OFF == 8) return dpp_bits<0x128>(x);                    // row_ror:8
  if (OFF == 4) return dpp_bits<0x1B>(dpp_bits<0x141>(x));    // row_half_mirror, quad_perm:[3,2,1,0]
  if (OFF == 2) return dpp_bits<0x4E>(x);                     // quad_perm:[2,3,0,1]
  return dpp_bits<0xB1>(x);                                   // quad_perm:[1,0,3,2]
}
__device__ __forceinline__ float lane_xor8(float x) { return __uint_as_float(lane_xor_bits<8>(__float_as_uint(x))); }
__device__ __forceinline__ float lane_xor4(float x) { return __uint_as_float(lane_xor_bits<4>(__float_as_uint(x))); }
__device__ __forceinline__ float lane_xor2(float x) { return __uint_as_float(lane_xor_bits<2>(__float_as_uint(x))); }
__device__ __forceinline__ float lane_xor1(float x) { return __uint_as_float(lane_xor_bits<1>(__float_as_uint(x))); }

// Sum and maximum over the wavefront, every lane gets the result: the butterfly lane i with lane
// i ^ 32, 16, 8, 4, 2, 1 in that order (an addition gives both lanes of a pair the same bits). Through
// the lane swaps and DPP it is a dozen vector-ALU instructions; six __shfl_xor go through the LDS
// crossbar one after the other (a key of the plain attention 0.6 us, most of it this sum).
__device__ __forceinline__ float wave_sum(float v) {
  v = xor32_sum(v);
  v = xor16_sum(v);
  v += lane_xor8(v);
  v += lane_xor4(v);
  v += lane_xor2(v);
  v += lane_xor1(v);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
  v = xor32_max(v);
  v = xor16_max(v);
  v = fmaxf(v, lane_xor8(v));
  v = fmaxf(v, lane_xor4(v));
  v = fmaxf(v, lane_xor2(v));
  v = fmaxf(v, lane_xor1(v));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` needs 16 floats of shared memory. The order of the additions is
// fixed by the block shape alone.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (HE_WAVE - 1);
  const int wave = threadIdx.x >> 6;
  const int nwaves = (blockDim.x + HE_WAVE - 1) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

// ---- error channel -------------------------------------------------------
void he_set_error(const char* fmt, ...);
int he_check_launch(const char* what);
// compute units of the current device (errors.hip); the host-side plans count in them
int he_cus();
// attention_mfma.hip: joins attention parts that were all stored (the fused one-token kernel's, the
// prompt kernel's); row_seq may be null: every row has a sequence
int he_attention_merge_parts(void* out, const float* ws_o, const float* ws_ml, const void* row_seq,
                             int rows, int H, int hd, int parts, int out_pieces, void* stream);

// attention_prefill_wide.hip: prompt attention, 32 queries a wavefront (head sizes up to 128; arguments
// checked by the caller). parts > 1: the keys of a block of queries are cut into that many parts, each
// a workgroup of its own that leaves its sums in ws_o / ws_ml for he_attention_merge_parts.
int he_attention_prefill_wide(void* out, const void* q, const void* kpool, const void* vpool,
                              const void* cu_seqlens, const void* seq_slot, const void* seq_start,
                              const void* page_table, int max_blocks, int num_pages, int num_seqs,
                              int max_q_len, int H, int KVH, int hd, int window, float scale,
                              int parts, float* ws_o, float* ws_ml, void* stream);

#define HE_REQUIRE(cond, ...)      \
  do {                             \
    if (!(cond)) {                 \
      he_set_error(__VA_ARGS__);   \
      return -1;                   \
    }                              \
  } while (0)
