// The kernel of gemm_rows.hip and its launch, shared by the files that each compile one part
// of its tilings (gemm_rows_tiles_*.hip): the tilings are many and each costs about half a
// second to compile, so one file for all of them would set the time of the whole build.
#pragma once
#include "common.h"
#include "hector_kernels.h"


typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define ROWS_KC 128   // k values of a chunk

struct RowsFusion {
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

template <int R>
struct RowsA {
  bf16x8 a[2][R][2];
};

// TAIL: the chunk may reach past k_end (such loads read a safe address and give zeros).
template <int R, bool TAIL>
__device__ __forceinline__ void rows_load_a(RowsA<R>& f, const uint16_t* const* wp, const uint16_t* safe,
                                            int k, int lg, int k_end) {
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kk = k + 64 * u + 16 * lg + 8 * h;
      const bool ok = !TAIL || kk + 8 <= k_end;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint16_t* p = ok ? wp[r] + k + 64 * u + 8 * h : safe;
        uint4 v = *reinterpret_cast<const uint4*>(p);
        if (TAIL && !ok) v = make_uint4(0, 0, 0, 0);
        f.a[u][r][h] = __builtin_bit_cast(bf16x8, v);
      }
    }
}

// The pieces (8 k values of one row) of a chunk that this thread copies: piece e of the chunk
// is k piece e / M16 of row e % M16.
template <int MT, int NT, bool XP, bool TAIL>
__device__ __forceinline__ void rows_load_b(uint4 (&st)[(MT * 256 + NT - 1) / NT], const uint16_t* X,
                                            int M, int K, int k, int k_end) {
  constexpr int M16 = 16 * MT;
  constexpr int BL = (MT * 256 + NT - 1) / NT;
#pragma unroll
  for (int q = 0; q < BL; ++q) {
    const int e = threadIdx.x + q * NT;
    const int pk = e / M16, m = min(e % M16, M - 1);
    const bool inside = MT * 256 % NT == 0 || e < MT * 256;
    const bool ok = inside && (!TAIL || k + 8 * pk + 8 <= k_end);
    const int kp = ok ? k + 8 * pk : 0;
    const uint16_t* p = XP ? X + ((int64_t)(kp >> 3) * M + m) * 8 : X + (int64_t)m * K + kp;
    uint4 v = *reinterpret_cast<const uint4*>(p);
    if (!ok) v = make_uint4(0, 0, 0, 0);
    st[q] = v;
  }
}

template <int MT, int NT>
__device__ __forceinline__ void rows_store_b(const uint4 (&st)[(MT * 256 + NT - 1) / NT],
                                             unsigned char* buf) {
  constexpr int M16 = 16 * MT;
  constexpr int BL = (MT * 256 + NT - 1) / NT;
#pragma unroll
  for (int q = 0; q < BL; ++q) {
    const int e = threadIdx.x + q * NT;
    if (MT * 256 % NT != 0 && e >= MT * 256) break;
    const int pk = e / M16, m = e % M16;
    const int u = pk >> 3, p = pk & 7;
    const int off = u * (MT * 2048) + ((((m >> 4) * 2 + (p & 1)) * 4 + (p >> 1)) * 16 + (m & 15)) * 16;
    *reinterpret_cast<uint4*>(buf + off) = st[q];
  }
}

template <int MT, int R>
__device__ __forceinline__ void rows_multiply(const RowsA<R>& f, const unsigned char* buf, int lane,
                                              floatx4 (&acc)[R][MT]) {
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      bf16x8 b[MT];
#pragma unroll
      for (int t = 0; t < MT; ++t)
        b[t] = __builtin_bit_cast(
            bf16x8, *reinterpret_cast<const uint4*>(buf + u * (MT * 2048) + (t * 2 + h) * 1024 + lane * 16));
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.a[u][r][h], b[t], acc[r][t], 0, 0, 0);
    }
}

template <typename TC>
__device__ __forceinline__ void rows_store4(TC* p, const float v[4], int align, int valid);
template <>
__device__ __forceinline__ void rows_store4<float>(float* p, const float v[4], int align, int valid) {
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
__device__ __forceinline__ void rows_store4<bf16_t>(bf16_t* p, const float v[4], int align, int valid) {
  if (align >= 4 && valid == 4) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
  } else if (align >= 2 && valid == 4) {
    *reinterpret_cast<uint32_t*>(p) = pack2_bf16(v[0], v[1]);
    *reinterpret_cast<uint32_t*>(p + 2) = pack2_bf16(v[2], v[3]);
  } else {
    for (int i = 0; i < valid; ++i) p[i].v = float_to_bf16_bits(v[i]);
  }
}

// `count` (2 or 4) neighbouring columns of row m from column `col` on (col a multiple of
// count), into a piece-major [M, D] bf16 tensor; `valid` of them exist.
__device__ __forceinline__ void rows_store_pieces(uint16_t* base, int M, int m, int col, const float* v,
                                                  int count, int valid) {
  uint16_t* at = base + ((int64_t)(col >> 3) * M + m) * 8 + (col & 7);
  if (valid == count && (col & (count - 1)) == 0) {
    if (count == 2) {
      *reinterpret_cast<uint32_t*>(at) = pack2_bf16(v[0], v[1]);
    } else {
      *reinterpret_cast<uint2*>(at) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
    }
    return;
  }
  for (int i = 0; i < valid; ++i) base[((int64_t)((col + i) >> 3) * M + m) * 8 + ((col + i) & 7)] = float_to_bf16_bits(v[i]);
}

// grid: (groups of 16 R NWV weight rows, K slices); block: 64 NWV threads.
template <int MT, int R, int NWV, bool XP, bool GATED, bool TAIL, typename TC>
__global__ __launch_bounds__(64 * NWV) void gemm_rows_kernel(
    TC* __restrict__ C, float* __restrict__ partial, const uint16_t* __restrict__ X,
    const uint16_t* __restrict__ W, const void* __restrict__ bias, int bias_dtype, int M, int N, int K,
    int kslice, int rows_per_block, RowsFusion fu) {
  constexpr int NT = 64 * NWV;
  constexpr int BL = (MT * 256 + NT - 1) / NT;
  __shared__ __align__(16) unsigned char xs[2][MT * 4096];
  __shared__ float row_sq[NWV][16 * MT];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  // the workgroup's weight rows [n0, n_end): at most 16 R NWV, fewer when the rows are dealt out
  // evenly over the compute units (the last wavefronts then have a partly empty tile, or none)
  const int n0 = blockIdx.x * rows_per_block;
  const int n_end = min(N, n0 + rows_per_block);
  const int n_wave = n0 + wave * (16 * R);
  const int k_begin = blockIdx.y * kslice;
  const int k_end = min(K, k_begin + kslice);
  const int nchunks = k_end > k_begin ? (k_end - k_begin + ROWS_KC - 1) / ROWS_KC : 0;

  const uint16_t* wp[R];
#pragma unroll
  for (int r = 0; r < R; ++r) wp[r] = W + (int64_t)min(n_wave + 16 * r + lr, n_end - 1) * K + lg * 16;

  floatx4 acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // The owed row scale of a carried norm, 1 / sqrt(sum of the row's partials / dim + eps): lane m of
  // every wavefront sums row m's partials in index order. The loads of the first eight go out
  // here, ahead of the weight stream, and are added behind it, so that their latency is not
  // in front of the first product.
  const bool scaled = fu.scale_partials != nullptr;
  constexpr int SCALE_EARLY = 8;
  float pv[SCALE_EARLY];
  const float* sp = fu.scale_partials + (int64_t)min(lane, M - 1) * fu.scale_count;
  if (scaled) {
#pragma unroll
    for (int i = 0; i < SCALE_EARLY; ++i) pv[i] = sp[min(i, fu.scale_count - 1)];
  }

  // Two chunks of weights are in flight per wavefront: chunk j + 2 is asked for as soon as chunk j
  // has been multiplied (more sets in flight cost registers, hence resident wavefronts, and
  // measured no faster). The activation rows of chunk j + 1 go from registers to LDS during chunk
  // j; they were asked for a chunk earlier and ahead of that turn's weights: loads complete in
  // order, so waiting for them waits for no weights but those the next turn needs anyway.
  uint4 bst0[BL], bst1[BL];     // the rows of an even / an odd chunk on their way to LDS
  RowsA<R> a0, a1;
  // Every workgroup starts at a chunk of its own and wraps around: workgroups that run in step
  // then do not all read the same offset of their (equally spaced) weight rows at once.
  const int rot = nchunks > 0 ? (int)((blockIdx.x * 5u) % (unsigned)nchunks) : 0;
  const auto kof = [&](int c) {
    const int cc = c + rot;
    return k_begin + (cc >= nchunks ? cc - nchunks : cc) * ROWS_KC;
  };
  // one chunk (A_: its weights, B_: its LDS buffer, N_: the register set of the next chunk's
  // rows). GUARD: near the end of the slice some of it is left out. WORK: false in a wavefront
  // without weight rows (rows dealt out evenly leave some): it only helps to copy the rows.
#define ROWS_STEP(A_, B_, N_, JJ_, GUARD_, WORK_)                                                  \
  {                                                                                                \
    const int jj = (JJ_);                                                                          \
    if (WORK_) rows_multiply<MT, R>(A_, xs[B_], lane, acc);                                        \
    if (!(GUARD_) || jj + 1 < nchunks) rows_store_b<MT, NT>(N_, xs[(B_) ^ 1]);                     \
    if (!(GUARD_) || jj + 3 < nchunks) rows_load_b<MT, NT, XP, TAIL>(N_, X, M, K, kof(jj + 3), k_end); \
    if ((WORK_) && (!(GUARD_) || jj + 2 < nchunks)) rows_load_a<R, TAIL>(A_, wp, W, kof(jj + 2), lg, k_end); \
    __syncthreads();                                                                               \
  }
  int j = 0;
  if (n_wave < n_end && nchunks > 4) {
    // The usual case, with nothing conditional ahead of its loop. The compiler places its waits
    // for loads by what may be in flight on any path into a loop; with the loads below behind
    // conditions (as in the general case further down) it had to assume, inside the loop and in
    // every turn, that the rows' loads were the newest, and drained the weights of the next chunk
    // with them: one chunk of weights in flight instead of two. The loads are issued in the
    // order of the loop (rows, then weights) so that both ways into it look alike.
    // (the scheduler would move the loads among each other; each sched_barrier keeps one group in its place)
    rows_load_b<MT, NT, XP, TAIL>(bst0, X, M, K, kof(0), k_end);
    __builtin_amdgcn_sched_barrier(0);
    rows_load_b<MT, NT, XP, TAIL>(bst1, X, M, K, kof(1), k_end);
    __builtin_amdgcn_sched_barrier(0);
    rows_load_a<R, TAIL>(a0, wp, W, kof(0), lg, k_end);
    __builtin_amdgcn_sched_barrier(0);
    rows_store_b<MT, NT>(bst0, xs[0]);
    rows_load_b<MT, NT, XP, TAIL>(bst0, X, M, K, kof(2), k_end);
    __builtin_amdgcn_sched_barrier(0);
    rows_load_a<R, TAIL>(a1, wp, W, kof(1), lg, k_end);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    for (; j + 4 < nchunks; j += 2) {
      ROWS_STEP(a0, 0, bst1, j, false, true)
      ROWS_STEP(a1, 1, bst0, j + 1, false, true)
    }
    for (; j < nchunks; j += 2) {
      ROWS_STEP(a0, 0, bst1, j, true, true)
      if (j + 1 >= nchunks) break;
      ROWS_STEP(a1, 1, bst0, j + 1, true, true)
    }
  } else {
    if (nchunks > 0) {
      rows_load_b<MT, NT, XP, TAIL>(bst0, X, M, K, kof(0), k_end);
      if (nchunks > 1) rows_load_b<MT, NT, XP, TAIL>(bst1, X, M, K, kof(1), k_end);
      if (n_wave < n_end) rows_load_a<R, TAIL>(a0, wp, W, kof(0), lg, k_end);
      rows_store_b<MT, NT>(bst0, xs[0]);
      if (nchunks > 2) rows_load_b<MT, NT, XP, TAIL>(bst0, X, M, K, kof(2), k_end);
      if (n_wave < n_end && nchunks > 1) rows_load_a<R, TAIL>(a1, wp, W, kof(1), lg, k_end);
    }
    __syncthreads();
    if (n_wave < n_end) {
      for (; j < nchunks; j += 2) {
        ROWS_STEP(a0, 0, bst1, j, true, true)
        if (j + 1 >= nchunks) break;
        ROWS_STEP(a1, 1, bst0, j + 1, true, true)
      }
    } else {
      for (; j < nchunks; j += 2) {
        ROWS_STEP(a0, 0, bst1, j, true, false)
        if (j + 1 >= nchunks) break;
        ROWS_STEP(a1, 1, bst0, j + 1, true, false)
      }
    }
  }
#undef ROWS_STEP

  float my_scale = 1.f;     // of row `lane`
  if (scaled) {
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < SCALE_EARLY; ++i) total += i < fu.scale_count ? pv[i] : 0.f;
    for (int i = SCALE_EARLY; i < fu.scale_count; ++i) total += sp[i];
    my_scale = 1.0f / sqrtf(total / (float)fu.scale_dim + fu.scale_eps);
  }

  // acc[r][t][i] = D[n_wave + 16 r + 4 lg + i][16 t + lr]
  const int out_align = ((N | n0) & 3) == 0 ? 4 : (((N | n0) & 1) == 0 ? 2 : 1);
  float rsc[MT];            // the scale of this lane's row of each tile
#pragma unroll
  for (int t = 0; t < MT; ++t) rsc[t] = __shfl(my_scale, 16 * t + lr, HE_WAVE);
  if (gridDim.y > 1) {     // this slice's sums; the reader adds the slices in order
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = n_wave + 16 * r + 4 * lg;
      const int valid = min(4, n_end - n);
      if (valid <= 0) continue;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + lr;
        if (m >= M) continue;
        const float rs = rsc[t];     // the owed scale is per row: each slice takes it
        const float v[4] = {acc[r][t][0] * rs, acc[r][t][1] * rs, acc[r][t][2] * rs, acc[r][t][3] * rs};
        rows_store4<float>(partial + ((int64_t)blockIdx.y * M + m) * N + n, v, out_align, valid);
      }
    }
    return;
  }

  const bool to_resid = !GATED && fu.resid != nullptr;
  float sq[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) sq[t] = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = n_wave + 16 * r + 4 * lg;
    const int valid = max(0, min(4, n_end - n));
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = 16 * t + lr;
      if (m >= M || valid <= 0) continue;
      const float rs = rsc[t];
      float v[4] = {acc[r][t][0] * rs, acc[r][t][1] * rs, acc[r][t][2] * rs, acc[r][t][3] * rs};
      if (GATED) {   // the four weight rows are two (gate, up) pairs: two outputs
        const int NO = N >> 1;
        float y[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) y[i] = v[2 * i] / (1.f + expf(-v[2 * i])) * v[2 * i + 1];
        if (fu.out_pieces)
          rows_store_pieces(reinterpret_cast<uint16_t*>(C), M, m, n >> 1, y, 2, valid >> 1);
        else if (((NO | (n >> 1)) & 1) == 0 && valid == 4) {
          if constexpr (sizeof(TC) == 2)
            *reinterpret_cast<uint32_t*>(C + (int64_t)m * NO + (n >> 1)) = pack2_bf16(y[0], y[1]);
          else
            *reinterpret_cast<float2*>(C + (int64_t)m * NO + (n >> 1)) = make_float2(y[0], y[1]);
        } else {
          for (int i = 0; i < (valid >> 1); ++i) C[(int64_t)m * NO + (n >> 1) + i] = from_float<TC>(y[i]);
        }
        continue;
      }
      if (bias != nullptr)
        for (int i = 0; i < valid; ++i) v[i] += load_param(bias, n + i, bias_dtype);
      if (!to_resid) {
        if (fu.out_pieces)
          rows_store_pieces(reinterpret_cast<uint16_t*>(C), M, m, n, v, 4, valid);
        else
          rows_store4<TC>(C + (int64_t)m * N + n, v, out_align, valid);
        continue;
      }
      float x[4], xgv[4];
      const int64_t at = (int64_t)m * N + n;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool in = i < valid;
        x[i] = (in ? fu.resid[at + i] : 0.f) + v[i];
        xgv[i] = in ? x[i] * load_param(fu.gain, n + i, fu.gain_dtype) : 0.f;
        if (in) sq[t] += x[i] * x[i];
      }
      rows_store4<float>(fu.resid + at, x, out_align, valid);
      if (fu.out_pieces)
        rows_store_pieces(fu.xg, M, m, n, xgv, 4, valid);
      else
        rows_store4<bf16_t>(reinterpret_cast<bf16_t*>(fu.xg) + at, xgv, out_align, valid);
    }
  }
  if (to_resid) {
    // sums of squares of each row over the workgroup's columns: across the four lane groups,
    // then across the wavefronts in their order
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float s = sq[t];
      s = xor16_sum(s);     // lane swaps, not the LDS crossbar: the same sums
      s = xor32_sum(s);
      if (lg == 0) row_sq[wave][16 * t + lr] = s;
    }
    __syncthreads();
    const int m = threadIdx.x;
    if (m < M && m < 16 * MT) {
      float s = 0.f;
      for (int w = 0; w < NWV; ++w) s += row_sq[w][m];
      fu.sq_out[(int64_t)m * gridDim.x + blockIdx.x] = s;
    }
  }
}

struct RowsPlan {
  int MT, R, NWV, splits, kslice, groups, rows_per_block;
};

template <int MT, int R, int NWV, bool GATED, typename TC>
static inline void launch_rows(const RowsPlan& p, void* C, float* partial, const void* X, const void* W,
                        const void* bias, int bias_dtype, int M, int N, int K, const RowsFusion& fu,
                        bool x_pieces, hipStream_t s) {
  const dim3 grid(p.groups, p.splits);
  const bool tail = K % ROWS_KC != 0;
#define ROWS_LAUNCH(XP_, TAIL_)                                                                    \
  gemm_rows_kernel<MT, R, NWV, XP_, GATED, TAIL_, TC><<<grid, 64 * NWV, 0, s>>>(                   \
      (TC*)C, partial, (const uint16_t*)X, (const uint16_t*)W, bias, bias_dtype, M, N, K, p.kslice,    \
      p.rows_per_block, fu)
  if (x_pieces) {
    if (tail) ROWS_LAUNCH(true, true); else ROWS_LAUNCH(true, false);
  } else {
    if (tail) ROWS_LAUNCH(false, true); else ROWS_LAUNCH(false, false);
  }
#undef ROWS_LAUNCH
}

// One tile count's tilings with one epilogue: a function per file of gemm_rows_tiles_*.hip.
// Returns 0 after a launch, -1 with the error set when the plan names no tiling of this file.
#define HE_ROWS_DISPATCH_ARGS                                                                       \
  const RowsPlan &p, void *C, float *partial, const void *X, const void *W, const void *bias,      \
      int bias_dtype, int M, int N, int K, const RowsFusion &fu, bool x_pieces, hipStream_t s
int he_rows_tiles2_bf16(HE_ROWS_DISPATCH_ARGS);
int he_rows_tiles2_f32(HE_ROWS_DISPATCH_ARGS);
int he_rows_tiles2_gated(HE_ROWS_DISPATCH_ARGS);
int he_rows_tiles4_bf16(HE_ROWS_DISPATCH_ARGS);
int he_rows_tiles4_f32(HE_ROWS_DISPATCH_ARGS);
int he_rows_tiles4_gated(HE_ROWS_DISPATCH_ARGS);

#define HE_ROWS_TILING(MT_, R_, NWV_, GATED_, TC_)                                                  \
  if (p.MT == MT_ && p.R == R_ && p.NWV == NWV_) {                                                  \
    launch_rows<MT_, R_, NWV_, GATED_, TC_>(p, C, partial, X, W, bias, bias_dtype, M, N, K, fu,     \
                                            x_pieces, s);                                           \
    return 0;                                                                                       \
  }
#define HE_ROWS_NO_TILING                                                                           \
  he_set_error("he_gemm_rows_bf16: no kernel for MT=%d R=%d NWV=%d", p.MT, p.R, p.NWV);             \
  return -1
