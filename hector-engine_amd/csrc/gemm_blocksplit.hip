// bf16 matrix product for few rows (M <= 32) with K cut inside the workgroup:
// C[M,N] = X[M,K] * W[N,K]^T (+ bias), or the gated activation of a gate||up
// weight. One workgroup owns up to 16*R weight rows (the rows are dealt out evenly over the
// compute units, see blocksplit_plan); its NW wavefronts take one K slice
// each (operands straight from global memory into the MFMA registers, in the operand
// layout gemm_rows.hip describes), leave their fp32
// tiles in LDS, and the workgroup adds the slices in wavefront order and writes
// the result. The sum is complete inside one launch: no partial sums in global
// memory, no second kernel, no atomics, and the order of the additions is fixed.
// With 16 wavefronts a product as small as 3584 x 3584 still puts 3584
// wavefronts on the chip.
//
// Gated epilogue: the weight alternates gate and up rows (gate i at row 2i, its up at
// 2i + 1), so the four neighbouring weight rows whose sums a thread holds are two
// (gate, up) pairs, and the output is silu(gate) * up, [M, N/2] (reference:
// kernels/activations.cu:183-198 as a kernel of its own).
//
// Two more epilogues carry an RMS norm across a pair of products without a kernel of
// its own (reference: kernels/fused_add_rmsnorm.cu:47-81 as a separate kernel):
//   residual: r[m][n] += acc (+ bias), stored fp32 in place; xg[m][n] = bf16(r * g[n]) with
//     the gain g of the norm that follows; and the sum of r^2 over the workgroup's columns
//     per row, one partial per workgroup: sq[m][block].
//   row scale: the consumer of xg adds the partials of a row in a fixed order,
//     s[m] = 1 / sqrt(sum / dim + eps), and multiplies its sums by s[m] before bias or
//     gate: W (r g s) = s W (r g). The norm's statistics stay fp32.
//
// Activations between two such products may lie piece-major instead of row-major: a [M, D]
// bf16 tensor as 16-byte pieces [D / 8][M][8], element (m, d) at ((d / 8) M + m) 8 + d % 8.
// The 16 lanes of an activation operand load then read 16 neighbouring pieces (two lines)
// instead of 16 rows (16 lines): the cost of the activation rows, which grows with their
// number (gate||up 48 us at 1 row, 50 at 8, 59 at 16), all but goes (49 and 55 us). The
// producing epilogue writes the layout, the consuming product reads it (x_pieces / out_pieces).
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
      sq += __shfl_xor(sq, 16, HE_WAVE);
      sq += __shfl_xor(sq, 32, HE_WAVE);
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

// Tilings measured on MI355X (graph-timed sweeps over R, U and NW at the Qwen2.5-7B, Qwen2.5-32B
// and Qwen2-72B shapes). The rule depends on the sizes only, so a product always runs the same way.
static BlockSplitPlan blocksplit_plan(int M, int N, int K, int gated, int R, int U, int NW) {
  BlockSplitPlan p;
  p.MT = (M + 15) / 16;
  int r, u, nw;
  if (N >= 65536) {                 // output head
    if (M <= 8) r = 2, u = 1, nw = 8;
    else if (p.MT == 1) r = 4, u = 2, nw = 4;
    else r = 2, u = 2, nw = 4;
  } else if (K >= 8192) {           // long K
    const int groups = (N + 31) / 32, last_round = groups % 256;   // with two tiles a workgroup
    if (N < 4096) {                 // few weight rows: one tile a workgroup, or the chip is not filled
      r = 1, u = 1, nw = p.MT == 1 ? 8 : 4;
    } else if (p.MT == 2) {
      r = 2, u = 2, nw = 4;
    } else if (M > 8 && N >= 10240) {
      r = 4, u = 2, nw = 4;         // the activation rows are read half as often
    } else if (groups < 256) {
      r = 2, u = 1, nw = 8;         // under one workgroup a compute unit: more wavefronts each
    } else if (groups < 1024 && last_round > 0 && last_round <= 128) {
      r = 1, u = 1, nw = 8;         // the last round of whole tiles would fill under half of the chip:
                                    // the rows are dealt out below, 20 a workgroup for 10240
    } else if (K >= 16384) {
      r = 2, u = 2, nw = 8;         // 8192 x 29568 at 8 rows: 85.3 us against 89.2 us for the next line's tiling
    } else {
      r = 2, u = 4, nw = 4;
    }
  } else if (N >= 16384) {          // wide N (gate||up)
    r = 2, u = 1, nw = 8;
    if (p.MT == 2 || K < 5120) u = 2, nw = 4;   // 37888 x 3584 at 8 rows: 47.7 us against 48.5 us
    else if (M > 8) r = 4;
  } else {                          // small products (q||k||v, o)
    r = N >= 4096 ? 2 : 1;
    u = p.MT == 1 && K < 5120 ? 4 : 1;   // 5120 x 5120 at 8 rows: 12.8 us unrolled once, 13.5 us four times
    nw = 8;
  }
  // Weight rows are dealt out evenly over the 256 compute units (or twice, three times ... 256
  // workgroups, at most 32 rows each) rather than in whole tiles of 16: 4608 rows as 256
  // workgroups of 18 rows instead of 144 of 32, the 37888 rows of gate||up as 1280 of 30
  // instead of 1184 of 32 (4.6 a compute unit). The last tile of such a workgroup is partly
  // empty. A workgroup's rows are an even number: a gate stays with its up, and outputs can be
  // stored in pairs.
  int rows = 0;
  if (R <= 0 && r <= 2 && N >= 2048 && N < 65536) {
    const int rounds = (N + 256 * 32 - 1) / (256 * 32);
    rows = ((N + 256 * rounds - 1) / (256 * rounds) + 1) & ~1;
    r = rows > 16 ? 2 : 1;
  }
  p.R = R > 0 ? R : r;
  p.U = U > 0 ? U : u;
  if (NW <= 0) {
    NW = nw;
    while (NW > 1 && K / NW < 128) NW >>= 1;
  }
  if (NW > bs_max_waves(p.MT, p.R, p.U)) NW = bs_max_waves(p.MT, p.R, p.U);
  p.NW = NW;
  int ks = (K + NW - 1) / NW;
  p.kslice = (ks + 63) / 64 * 64;
  p.rows_per_block = rows > 0 ? rows : 16 * p.R;
  return p;
}

template <int MT, int R, int U, bool GATED, typename TC>
static void launch_blocksplit(const BlockSplitPlan& p, void* C, const void* X, const void* W,
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

template <bool GATED, typename TC>
static int dispatch_blocksplit(const BlockSplitPlan& p, void* C, const void* X, const void* W,
                               const void* bias, int bias_dtype, int M, int N, int K,
                               const BsFusion& fu, bool x_pieces, hipStream_t s) {
#define BS(MT_, R_, U_)                                                              \
  if (p.MT == MT_ && p.R == R_ && p.U == U_) {                                       \
    launch_blocksplit<MT_, R_, U_, GATED, TC>(p, C, X, W, bias, bias_dtype, M, N, K, fu, x_pieces, s); \
    return 0;                                                                        \
  }
  BS(1, 1, 1) BS(1, 1, 2) BS(1, 1, 4) BS(2, 1, 1) BS(2, 1, 2)
  BS(1, 2, 1) BS(1, 2, 2) BS(1, 2, 4) BS(2, 2, 1) BS(2, 2, 2) BS(1, 4, 1) BS(1, 4, 2)
#undef BS
  he_set_error("he_gemm_blocksplit_bf16: no kernel for MT=%d R=%d U=%d", p.MT, p.R, p.U);
  return -1;
}

// Workgroups (= partial sums of squares per row) the residual epilogue of this product gives.
extern "C" int he_gemm_blocksplit_blocks(int M, int N, int K) {
  if (M <= 0 || M > HE_BLOCKSPLIT_MAX_M || N <= 0 || K <= 0) return 0;
  const BlockSplitPlan p = blocksplit_plan(M, N, K, 0, 0, 0, 0);
  return (N + p.rows_per_block - 1) / p.rows_per_block;
}

// R, U, NW <= 0 choose the heuristic tiling (NW wavefronts = K slices per workgroup).
// scale_partials: sums of squares of the input rows (the rows are then scaled before
// bias or gate); resid: the residual epilogue (C is not written; gain, xg, sq_out needed).
extern "C" int he_gemm_blocksplit_fused_bf16(void* C, const void* A, const void* W,
                                             const void* bias, int M, int N, int K, int out_dtype,
                                             int bias_dtype, int gated, int R, int U, int NW,
                                             const void* scale_partials, int scale_count,
                                             float scale_eps, void* resid, const void* gain,
                                             int gain_dtype, void* xg, void* sq_out,
                                             int sq_count, int x_pieces, int out_pieces,
                                             void* stream) {
  HE_REQUIRE(M > 0 && M <= HE_BLOCKSPLIT_MAX_M, "he_gemm_blocksplit_bf16: M=%d outside [1, %d]", M,
             HE_BLOCKSPLIT_MAX_M);
  HE_REQUIRE(N > 0 && K > 0, "he_gemm_blocksplit_bf16: bad sizes N=%d K=%d", N, K);
  HE_REQUIRE((K & 7) == 0, "he_gemm_blocksplit_bf16: K=%d must be a multiple of 8", K);
  HE_REQUIRE(out_dtype == HE_BF16 || out_dtype == HE_F32, "he_gemm_blocksplit_bf16: bad out dtype");
  HE_REQUIRE((((uintptr_t)A | (uintptr_t)W) & 15) == 0,
             "he_gemm_blocksplit_bf16: operands must be 16-byte aligned");
  HE_REQUIRE(!gated || ((N & 1) == 0 && bias == nullptr),
             "he_gemm_blocksplit_bf16: the gated epilogue needs an even N=%d and no bias", N);
  HE_REQUIRE(scale_partials == nullptr || scale_count > 0,
             "he_gemm_blocksplit_bf16: row scale without partial sums");
  HE_REQUIRE(!(x_pieces || out_pieces) || M <= 16,
             "he_gemm_blocksplit_bf16: piece-major activations are for up to 16 rows, not %d", M);
  HE_REQUIRE(!out_pieces || ((resid != nullptr || out_dtype == HE_BF16) && ((gated ? N / 2 : N) & 7) == 0),
             "he_gemm_blocksplit_bf16: a piece-major output is bf16 and a multiple of 8 wide");
  const BlockSplitPlan p = blocksplit_plan(M, N, K, gated, R, U, NW);
  HE_REQUIRE(p.NW >= 1 && p.NW <= 16, "he_gemm_blocksplit_bf16: %d wavefronts outside [1, 16]",
             p.NW);
  const int blocks = (N + p.rows_per_block - 1) / p.rows_per_block;
  if (resid != nullptr) {
    HE_REQUIRE(!gated && gain != nullptr && xg != nullptr && sq_out != nullptr,
               "he_gemm_blocksplit_bf16: the residual epilogue needs gain, xg and sq_out, and no gate");
    HE_REQUIRE(sq_count == blocks,
               "he_gemm_blocksplit_bf16: %d partial sums per row given, the product has %d workgroups",
               sq_count, blocks);
    HE_REQUIRE(gain_dtype == HE_F32 || gain_dtype == HE_BF16, "he_gemm_blocksplit_bf16: bad gain dtype");
  } else {
    HE_REQUIRE(C != nullptr, "he_gemm_blocksplit_bf16: no output");
  }
  BsFusion fu;
  fu.scale_partials = (const float*)scale_partials;
  fu.scale_count = scale_count;
  fu.scale_eps = scale_eps;
  fu.scale_dim = K;
  fu.resid = (float*)resid;
  fu.gain = gain;
  fu.gain_dtype = gain_dtype;
  fu.xg = (uint16_t*)xg;
  fu.sq_out = (float*)sq_out;
  fu.out_pieces = out_pieces;
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (gated)
    rc = out_dtype == HE_BF16
             ? dispatch_blocksplit<true, bf16_t>(p, C, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s)
             : dispatch_blocksplit<true, float>(p, C, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s);
  else
    rc = out_dtype == HE_BF16
             ? dispatch_blocksplit<false, bf16_t>(p, C, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s)
             : dispatch_blocksplit<false, float>(p, C, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s);
  if (rc) return rc;
  return he_check_launch("he_gemm_blocksplit_bf16");
}

extern "C" int he_gemm_blocksplit_bf16(void* C, const void* A, const void* W, const void* bias,
                                       int M, int N, int K, int out_dtype, int bias_dtype,
                                       int gated, int R, int U, int NW, void* stream) {
  return he_gemm_blocksplit_fused_bf16(C, A, W, bias, M, N, K, out_dtype, bias_dtype, gated, R, U,
                                       NW, nullptr, 0, 0.f, nullptr, nullptr, HE_F32, nullptr,
                                       nullptr, 0, 0, 0, stream);
}
