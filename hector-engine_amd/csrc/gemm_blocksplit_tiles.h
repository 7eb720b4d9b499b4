// The kernel of gemm_blocksplit.hip and its launch, shared by the files that each compile its
// tilings for one epilogue and output type (gemm_blocksplit_tiles_*.hip): compiled in one file
// they would set the time of the whole build.
#pragma once
#include "common.h"
#include "hector_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

template <bool CHECKED>
__device__ __forceinline__ bf16x8 bs_load8(const uint16_t* p, bool ok) {
  if (!CHECKED) return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
  uint4 v = make_uint4(0, 0, 0, 0);
  if (ok) v = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, v);
}

// Four neighbouring outputs. align: how many elements the address is a multiple of (4, 2 or 1).
template <typename TC>
__device__ __forceinline__ void bs_store4(TC* p, const float v[4], int align, int valid);
template <>
__device__ __forceinline__ void bs_store4<float>(float* p, const float v[4], int align, int valid) {
  if (align >= 4 && valid == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else if (align >= 2 && valid == 4) {
    *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
    *reinterpret_cast<float2*>(p + 2) = make_float2(v[2], v[3]);
  } else {
    for (int i = 0; i < valid; ++i) p[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void bs_store4<bf16_t>(bf16_t* p, const float v[4], int align,
                                                  int valid) {
  const uint32_t lo = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
  const uint32_t hi = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
  if (align >= 4 && valid == 4) {
    *reinterpret_cast<uint2*>(p) = make_uint2(lo, hi);
  } else if (align >= 2 && valid == 4) {
    *reinterpret_cast<uint32_t*>(p) = lo;
    *reinterpret_cast<uint32_t*>(p + 2) = hi;
  } else {
    for (int i = 0; i < valid; ++i) p[i].v = float_to_bf16_bits(v[i]);
  }
}

template <typename TC>
__device__ __forceinline__ void bs_store2(TC* p, const float v[2], bool vec, int valid);
template <>
__device__ __forceinline__ void bs_store2<float>(float* p, const float v[2], bool vec, int valid) {
  if (vec && valid == 2) {
    *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
  } else {
    for (int i = 0; i < valid; ++i) p[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void bs_store2<bf16_t>(bf16_t* p, const float v[2], bool vec,
                                                  int valid) {
  if (vec && valid == 2) {
    *reinterpret_cast<uint32_t*>(p) =
        (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
  } else {
    for (int i = 0; i < valid; ++i) p[i].v = float_to_bf16_bits(v[i]);
  }
}

// `count` (2 or 4) neighbouring columns of row m from column `col` on, into a piece-major
// [M, D] bf16 tensor; `valid` of them exist.
__device__ __forceinline__ void bs_store_pieces(uint16_t* base, int M, int m, int col, const float* v,
                                                int count, int valid) {
  auto at = [&](int c) { return base + ((int64_t)(c >> 3) * M + m) * 8 + (c & 7); };
  if (valid == count && (col & 1) == 0) {        // pairs never straddle a piece
    const uint32_t lo = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
    if (count == 2) {
      *reinterpret_cast<uint32_t*>(at(col)) = lo;
      return;
    }
    const uint32_t hi = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
    if ((col & 3) == 0) {
      *reinterpret_cast<uint2*>(at(col)) = make_uint2(lo, hi);
    } else {
      *reinterpret_cast<uint32_t*>(at(col)) = lo;
      *reinterpret_cast<uint32_t*>(at(col + 2)) = hi;
    }
    return;
  }
  for (int i = 0; i < valid; ++i) *at(col + i) = float_to_bf16_bits(v[i]);
}

// Registers hold the operands of two steps (the loads of the next step are issued before
// the products of this one), 16 U (R + MT) of them; above 4 tile pairs the workgroup is
// limited to 8 wavefronts so that each may use 256 registers.
constexpr int bs_max_waves(int MT, int R, int U) { return U * (R + MT) <= 4 ? 16 : 8; }

template <int MT, int R, int U>
struct BsFrags {
  bf16x8 a[U][R][2], b[U][MT][2];
};

// CHECKED: the step may reach past k_end (it then loads nothing there and adds zeros). Unchecked
// loads carry no branch, so the compiler counts them and waits for the older fragments only,
// not for all that are in flight.
template <int MT, int R, int U, bool PIECES, bool CHECKED>
__device__ __forceinline__ void bs_load(BsFrags<MT, R, U>& f, const uint16_t* const* wp,
                                        const uint16_t* const* xp, int k, int lg, int k_end, int M) {
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int kk = k + 64 * u + lg * 16;   // this lane's 16 k values of the step
    const bool ok0 = !CHECKED || kk + 8 <= k_end, ok1 = !CHECKED || kk + 16 <= k_end;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      f.a[u][r][0] = bs_load8<CHECKED>(wp[r] + k + 64 * u, ok0);
      f.a[u][r][1] = bs_load8<CHECKED>(wp[r] + k + 64 * u + 8, ok1);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      if (PIECES) {   // piece-major X: the piece of 8 k values from kk on lies at kk M (+ 8 row)
        f.b[u][t][0] = bs_load8<CHECKED>(xp[t] + (k + 64 * u) * M, ok0);
        f.b[u][t][1] = bs_load8<CHECKED>(xp[t] + (k + 64 * u + 8) * M, ok1);
      } else {
        f.b[u][t][0] = bs_load8<CHECKED>(xp[t] + k + 64 * u, ok0);
        f.b[u][t][1] = bs_load8<CHECKED>(xp[t] + k + 64 * u + 8, ok1);
      }
    }
  }
}

template <int MT, int R, int U>
__device__ __forceinline__ void bs_multiply(const BsFrags<MT, R, U>& f, floatx4 (&acc)[R][MT]) {
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.a[u][r][h], f.b[u][t][h], acc[r][t],
                                                              0, 0, 0);
}

struct BsFusion {
  const float* scale_partials;   // [M][scale_count] or null: sums of squares of the input rows
  int scale_count;
  float scale_eps;
  int scale_dim;
  float* resid;                  // [M][N] fp32 or null: residual rows, updated in place
  const void* gain;              // [N] gain of the following norm
  int gain_dtype;
  uint16_t* xg;                  // [M][N] bf16 out: resid * gain
  float* sq_out;                 // [M][gridDim.x] out: sum of resid^2 over this workgroup's columns
  int out_pieces;                // the bf16 output (C, or xg) is written piece-major
};

// The residual values and gains of output item (tile, lane) of a non-gated product:
// row m = 16 t + lane % 16, columns n0 + 16 r + 4 (lane / 16) .. + 4.
// With few rows the 16 columns of the activation tile hold each row several times: column c
// is row c >> spread (spread 2 up to 4 rows, 1 up to 8), so that the four lanes the memory
// pipeline takes together read one or two rows, not four (1-4 % of a product's time). The
// first column of a row owns its outputs.
template <int MT>
__device__ __forceinline__ int bs_spread(int M) {
  return MT == 1 ? (M <= 4 ? 2 : (M <= 8 ? 1 : 0)) : 0;
}

template <int MT>
__device__ __forceinline__ void bs_load_resid(const BsFusion& fu, int item, int n0, int n_end, int M,
                                              int N, float res[4], float gain[4]) {
  const int spread = bs_spread<MT>(M);
  const int ot = item >> 6, ol = item & 63;
  const int col = 16 * (ot % MT) + (ol & 15);
  const int m = col >> spread;
  const int n = n0 + 16 * (ot / MT) + 4 * (ol >> 4);
  const int valid = (m < M && (m << spread) == col) ? max(0, min(4, n_end - n)) : 0;
  if (valid == 4 && ((N | n0) & 3) == 0) {
    const float4 r4 = *reinterpret_cast<const float4*>(fu.resid + (int64_t)m * N + n);
    res[0] = r4.x, res[1] = r4.y, res[2] = r4.z, res[3] = r4.w;
  } else if (valid == 4 && ((N | n0) & 1) == 0) {
    const float2 a = *reinterpret_cast<const float2*>(fu.resid + (int64_t)m * N + n);
    const float2 b = *reinterpret_cast<const float2*>(fu.resid + (int64_t)m * N + n + 2);
    res[0] = a.x, res[1] = a.y, res[2] = b.x, res[3] = b.y;
  } else {
    for (int i = 0; i < 4; ++i) res[i] = i < valid ? fu.resid[(int64_t)m * N + n + i] : 0.f;
  }
  if (valid == 4 && fu.gain_dtype == HE_BF16 && (n & 1) == 0 && (((uintptr_t)fu.gain) & 3) == 0) {
    const uint32_t* g = reinterpret_cast<const uint32_t*>((const uint16_t*)fu.gain + n);
    const uint32_t a = g[0], b = g[1];
    gain[0] = __uint_as_float(a << 16), gain[1] = __uint_as_float(a & 0xffff0000u);
    gain[2] = __uint_as_float(b << 16), gain[3] = __uint_as_float(b & 0xffff0000u);
  } else {
    for (int i = 0; i < 4; ++i) gain[i] = i < valid ? load_param(fu.gain, n + i, fu.gain_dtype) : 0.f;
  }
}

// grid: one workgroup per 16*R weight rows; block: 64 * NW threads.
template <int MT, int R, int U, bool GATED, bool PIECES, typename TC>
__global__ __launch_bounds__(64 * bs_max_waves(MT, R, U)) void gemm_blocksplit_kernel(
    TC* __restrict__ C, const uint16_t* __restrict__ X, const uint16_t* __restrict__ W,
    const void* __restrict__ bias, int bias_dtype, int M, int N, int K, int kslice, int rows_per_block,
    BsFusion fu) {
  extern __shared__ float4 tiles[];   // [NW][R*MT][64]
  __shared__ float row_scale[16 * MT];
  __shared__ float row_sq[R * MT][16];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  // the workgroup's weight rows [n0, n_end): at most 16 R, fewer when the rows are dealt out evenly
  const int n0 = blockIdx.x * rows_per_block;
  const int n_end = min(N, n0 + rows_per_block);
  const int k_begin = wave * kslice;
  const int k_end = min(K, k_begin + kslice);
  const int lr = lane & 15, lg = lane >> 4;
  const int spread = bs_spread<MT>(M);

  const uint16_t* wp[R];
  const uint16_t* xp[MT];
#pragma unroll
  for (int r = 0; r < R; ++r) wp[r] = W + (int64_t)min(n0 + 16 * r + lr, n_end - 1) * K + lg * 16;
#pragma unroll
  for (int t = 0; t < MT; ++t)
    xp[t] = PIECES ? X + (2 * lg * M + min((16 * t + lr) >> spread, M - 1)) * 8
                   : X + (int64_t)min((16 * t + lr) >> spread, M - 1) * K + lg * 16;

  floatx4 acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Loads the epilogue needs are issued here, ahead of the weight stream, so that their
  // latency is not added at the end: the partial sums of squares of the input rows
  // (wavefront w takes the rows w, w + nw, ... up to four; lanes hold strided partials) and, for the
  // residual epilogue (a little further down, behind the first weight loads), the residual
  // values and gains of this thread's first outputs.
  constexpr int OUT_TILES = R * MT;
  const int out_align = ((N | n0) & 3) == 0 ? 4 : (((N | n0) & 1) == 0 ? 2 : 1);
  const bool scaled = fu.scale_partials != nullptr;
  const bool to_resid = !GATED && fu.resid != nullptr;
  constexpr int SCALE_ROWS = 4;           // rows a wavefront takes: 16 rows with 4 wavefronts
  const bool scale_early = scaled && fu.scale_count <= 256 && M <= SCALE_ROWS * nw;
  float pv[SCALE_ROWS][4];
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);   // in a scalar register: rows beyond M cost a scalar branch
  if (scale_early) {
#pragma unroll
    for (int j = 0; j < SCALE_ROWS; ++j) {
      const int m = wave_s + j * nw;
#pragma unroll
      for (int q = 0; q < 4; ++q) pv[j][q] = 0.f;
      if (m < M) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int i = lane + 64 * q;
          if (i < fu.scale_count) pv[j][q] = fu.scale_partials[(int64_t)m * fu.scale_count + i];
        }
      }
    }
  }
  float res0[4] = {0.f, 0.f, 0.f, 0.f}, gain0[4] = {0.f, 0.f, 0.f, 0.f};

  // Two steps of 64 U k values per turn. The whole turns of a wavefront's slice run without
  // bounds checks, two fragments in flight: the loads of one are waited for while the other's
  // are on their way. They start at a point of the slice that differs from workgroup to
  // workgroup and wrap around: workgroups that run in step then read addresses that do not
  // all sit at the same offset of their (equally spaced) weight rows. What is left of the
  // slice is one checked turn at the end (a step past k_end loads nothing and adds zeros).
  BsFrags<MT, R, U> f0, f1;
  constexpr int TURN = 128 * U;
  const int span = max(k_end - k_begin, 0);
  const int full = span / TURN;
  const int k_full = k_begin + full * TURN;
  const bool tail = span > full * TURN;
  int k = full > 0 ? k_begin + (int)((blockIdx.x * 3u) % (unsigned)full) * TURN : k_begin;
  if (full > 0) bs_load<MT, R, U, PIECES, false>(f0, wp, xp, k, lg, k_end, M);
  else if (tail) bs_load<MT, R, U, PIECES, true>(f0, wp, xp, k_begin, lg, k_end, M);
  if (to_resid && threadIdx.x < OUT_TILES * 64)   // behind the first weights, ahead of the rest
    bs_load_resid<MT>(fu, threadIdx.x, n0, n_end, M, N, res0, gain0);
  if (full > 0) {
    for (int j = 0; j + 1 < full; ++j) {
      bs_load<MT, R, U, PIECES, false>(f1, wp, xp, k + 64 * U, lg, k_end, M);
      __builtin_amdgcn_sched_barrier(0);   // the loads of a fragment go out together, ahead of the products
      bs_multiply<MT, R, U>(f0, acc);
      k += TURN;
      if (k >= k_full) k = k_begin;
      __builtin_amdgcn_sched_barrier(0);
      bs_load<MT, R, U, PIECES, false>(f0, wp, xp, k, lg, k_end, M);
      __builtin_amdgcn_sched_barrier(0);
      bs_multiply<MT, R, U>(f1, acc);
      __builtin_amdgcn_sched_barrier(0);
    }
    bs_load<MT, R, U, PIECES, false>(f1, wp, xp, k + 64 * U, lg, k_end, M);
    bs_multiply<MT, R, U>(f0, acc);
    if (tail) bs_load<MT, R, U, PIECES, true>(f0, wp, xp, k_full, lg, k_end, M);
    bs_multiply<MT, R, U>(f1, acc);
  }
  if (tail) {
    bs_load<MT, R, U, PIECES, true>(f1, wp, xp, k_full + 64 * U, lg, k_end, M);
    bs_multiply<MT, R, U>(f0, acc);
    bs_multiply<MT, R, U>(f1, acc);
  }

  if (scaled) {
    if (scale_early) {
#pragma unroll
      for (int j = 0; j < SCALE_ROWS; ++j) {
        const int m = wave_s + j * nw;
        if (m < M) {
          const float total = wave_sum(((pv[j][0] + pv[j][1]) + pv[j][2]) + pv[j][3]);
          if (lane == 0) row_scale[m] = 1.0f / sqrtf(total / (float)fu.scale_dim + fu.scale_eps);
        }
      }
    } else {
      for (int m = wave; m < M; m += nw) {
        float part = 0.f;
        for (int i = lane; i < fu.scale_count; i += 64)
          part += fu.scale_partials[(int64_t)m * fu.scale_count + i];
        const float total = wave_sum(part);
        if (lane == 0) row_scale[m] = 1.0f / sqrtf(total / (float)fu.scale_dim + fu.scale_eps);
      }
    }
  }

  // every wavefront leaves its tiles; acc[r][t][i] = D[n0 + 16r + 4lg + i][16t + lr]
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t)
      tiles[(wave * (R * MT) + r * MT + t) * 64 + lane] =
          make_float4(acc[r][t][0], acc[r][t][1], acc[r][t][2], acc[r][t][3]);
  __syncthreads();

  // thread (tile, lane) adds the slices in wavefront order and writes 4 outputs; a
  // wavefront works on one tile at a time (item >> 6 is the same in all its lanes)
  for (int item = threadIdx.x; item < OUT_TILES * 64; item += blockDim.x) {
    const int ot = item >> 6, ol = item & 63;
    const int olr = ol & 15, olg = ol >> 4;
    const int t = ot % MT;
    const int r = ot / MT;
    const int col = 16 * t + olr, m = col >> spread;
    const bool owner = m < M && (m << spread) == col;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int w = 0; w < nw; ++w) {
      const float4 v = tiles[(w * (R * MT) + r * MT + t) * 64 + ol];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    float v[4] = {s.x, s.y, s.z, s.w};
    const float rs = (scaled && m < M) ? row_scale[m] : 1.f;
    if (GATED) {
      // the thread's four weight rows are two (gate, up) pairs: two outputs
      const int NO = N >> 1;
      const int n = n0 + 16 * r + 4 * olg;
      const int valid = owner ? max(0, min(4, n_end - n)) >> 1 : 0;
      if (valid <= 0) continue;
      float y[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const float g = v[2 * i] * rs;
        y[i] = g / (1.f + expf(-g)) * (v[2 * i + 1] * rs);
      }
      if (fu.out_pieces)
        bs_store_pieces(reinterpret_cast<uint16_t*>(C), M, m, n >> 1, y, 2, valid);
      else
        bs_store2<TC>(C + (int64_t)m * NO + (n >> 1), y, ((NO | (n0 >> 1)) & 1) == 0, valid);
    } else {
      const int n = n0 + 16 * r + 4 * olg;
      const int valid = owner ? max(0, min(4, n_end - n)) : 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= rs;
      if (bias != nullptr)
        for (int i = 0; i < valid; ++i) v[i] += load_param(bias, n + i, bias_dtype);
      if (!to_resid) {
        if (valid > 0) {
          if (fu.out_pieces)
            bs_store_pieces(reinterpret_cast<uint16_t*>(C), M, m, n, v, 4, valid);
          else
            bs_store4<TC>(C + (int64_t)m * N + n, v, out_align, valid);
        }
        continue;
      }
      if (item != threadIdx.x) bs_load_resid<MT>(fu, item, n0, n_end, M, N, res0, gain0);
      float sq = 0.f, x[4], xgv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x[i] = res0[i] + v[i];
        xgv[i] = x[i] * gain0[i];
        if (i < valid) sq += x[i] * x[i];
      }
      if (valid > 0) {
        const int64_t at = (int64_t)m * N + n;
        bs_store4<float>(fu.resid + at, x, out_align, valid);
        if (fu.out_pieces)
          bs_store_pieces(fu.xg, M, m, n, xgv, 4, valid);
        else
          bs_store4<bf16_t>(reinterpret_cast<bf16_t*>(fu.xg) + at, xgv, out_align, valid);
      }
      // the four lane groups hold the row's other columns of this tile
      sq = xor16_sum(sq);     // lane swaps, not the LDS crossbar: the same sums
      sq = xor32_sum(sq);
      if (olg == 0) row_sq[ot][olr] = sq;
    }
  }
  if (to_resid) {
    __syncthreads();
    const int m = threadIdx.x;
    if (m < M && m < 16 * MT) {
      float sq = 0.f;
      const int col = m << spread;
      for (int r = 0; r < R; ++r) sq += row_sq[r * MT + col / 16][col % 16];
      fu.sq_out[(int64_t)m * gridDim.x + blockIdx.x] = sq;
    }
  }
}

struct BlockSplitPlan {
  int MT, R, U, NW, kslice;
  int rows_per_block;   // weight rows of a workgroup, at most 16 R
};

template <int MT, int R, int U, bool GATED, typename TC>
static inline void launch_blocksplit(const BlockSplitPlan& p, void* C, const void* X, const void* W,
                              const void* bias, int bias_dtype, int M, int N, int K,
                              const BsFusion& fu, bool x_pieces, hipStream_t s) {
  const int blocks = (N + p.rows_per_block - 1) / p.rows_per_block;
  const size_t lds = (size_t)p.NW * R * MT * 64 * sizeof(float4);
  if constexpr (MT == 1) {   // piece-major activations are for up to 16 rows
    if (x_pieces) {
      gemm_blocksplit_kernel<MT, R, U, GATED, true, TC><<<blocks, 64 * p.NW, lds, s>>>(
          (TC*)C, (const uint16_t*)X, (const uint16_t*)W, bias, bias_dtype, M, N, K, p.kslice,
          p.rows_per_block, fu);
      return;
    }
  }
  gemm_blocksplit_kernel<MT, R, U, GATED, false, TC><<<blocks, 64 * p.NW, lds, s>>>(
      (TC*)C, (const uint16_t*)X, (const uint16_t*)W, bias, bias_dtype, M, N, K, p.kslice,
      p.rows_per_block, fu);
}

// Every tiling with one epilogue and output type: a function per file of
// gemm_blocksplit_tiles_*.hip. Returns 0 after a launch, -1 with the error set when the plan
// names no tiling.
#define HE_BS_DISPATCH_ARGS                                                                         \
  const BlockSplitPlan &p, void *C, const void *X, const void *W, const void *bias, int bias_dtype, \
      int M, int N, int K, const BsFusion &fu, bool x_pieces, hipStream_t s
int he_blocksplit_tiles_bf16(HE_BS_DISPATCH_ARGS);
int he_blocksplit_tiles_f32(HE_BS_DISPATCH_ARGS);
int he_blocksplit_tiles_gated_bf16(HE_BS_DISPATCH_ARGS);
int he_blocksplit_tiles_gated_f32(HE_BS_DISPATCH_ARGS);

#define HE_BS_TILING(MT_, R_, U_, GATED_, TC_)                                                      \
  if (p.MT == MT_ && p.R == R_ && p.U == U_) {                                                      \
    launch_blocksplit<MT_, R_, U_, GATED_, TC_>(p, C, X, W, bias, bias_dtype, M, N, K, fu, x_pieces, s); \
    return 0;                                                                                       \
  }
#define HE_BS_ALL_TILINGS(GATED_, TC_)                                                              \
  HE_BS_TILING(1, 1, 1, GATED_, TC_) HE_BS_TILING(1, 1, 2, GATED_, TC_)                             \
  HE_BS_TILING(1, 1, 4, GATED_, TC_) HE_BS_TILING(2, 1, 1, GATED_, TC_)                             \
  HE_BS_TILING(2, 1, 2, GATED_, TC_) HE_BS_TILING(1, 2, 1, GATED_, TC_)                             \
  HE_BS_TILING(1, 2, 2, GATED_, TC_) HE_BS_TILING(1, 2, 4, GATED_, TC_)                             \
  HE_BS_TILING(2, 2, 1, GATED_, TC_) HE_BS_TILING(2, 2, 2, GATED_, TC_)                             \
  HE_BS_TILING(1, 4, 1, GATED_, TC_) HE_BS_TILING(1, 4, 2, GATED_, TC_)                             \
  he_set_error("he_gemm_blocksplit_bf16: no kernel for MT=%d R=%d U=%d", p.MT, p.R, p.U);           \
  return -1
