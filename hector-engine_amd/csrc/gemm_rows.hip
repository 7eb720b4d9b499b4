// bf16 matrix product for 17 to 64 rows (one-token steps of larger batches):
// C[M,N] = X[M,K] * W[N,K]^T with the epilogues of gemm_blocksplit.hip (bias, gated
// SiLU x up, residual + rows for the next norm, owed row scale), where the reference calls
// its BLAS library (kernels/matmul_cublas.cu:240-277) and runs norm and activation as
// kernels of their own (kernels/fused_add_rmsnorm.cu, kernels/activations.cu:183-198).
//
// With more than 16 rows the activation rows cost as much to fetch as the weights when every
// wavefront fetches its own (gemm_blocksplit.hip). Here a workgroup's
// wavefronts all walk the same k range, each over 16 R weight rows of its own, so the
// activation rows of a k chunk are fetched once per workgroup: all threads copy the chunk
// [16 MT rows][128 k] into LDS, in the order of the MFMA's B operand (a wavefront's
// ds_read_b128 is one contiguous KiB), double-buffered with one barrier a chunk. The weights
// go straight from global memory into the A operand registers, the loads of the next chunk
// in flight while this one is multiplied. Operand layout of v_mfma_f32_16x16x32_bf16 as used here
// (the k slots of an instruction may hold any 8 k values as long as A and B agree):
//   A: lane l holds W[n0 + l % 16][k + 64 u + 16 (l / 16) + 8 h .. + 8]
//   B: lane l holds X[16 t + l % 16][the same k]
//   D: lane l holds D[n0 + 4 (l / 16) + i][16 t + l % 16], i = 0..3
//
// Products with few weight rows are also cut along K across workgroups (grid y): each slice
// leaves its fp32 sums [slices][M][N] and the reader adds them in slice order
// (he_splitk_reduce, he_splitk_reduce_residual): no atomics, a fixed order of additions.
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
      s += __shfl_xor(s, 16, HE_WAVE);
      s += __shfl_xor(s, 32, HE_WAVE);
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

// Tilings measured on MI355X at the Qwen2.5-7B shapes; the rule depends on the sizes only, so a
// product always runs the same way. Wide products (gate||up, the output head) run in one K
// slice, their weight rows dealt out evenly over the workgroups the chip holds at once (two
// a compute unit: 37888 rows as 499 workgroups of 76, the last three of whose eight wavefronts
// only help to copy the activation rows; not 296 of 128, of which 40 would run after the
// others; above 32 rows one workgroup of sixteen wavefronts a compute unit); narrow ones are cut along K until the grid holds about a workgroup a compute unit.
static RowsPlan rows_plan(int M, int N, int K, int R, int NWV, int splits) {
  RowsPlan p;
  p.MT = M <= 32 ? 2 : 4;
  if (R <= 0 || NWV <= 0) {
    if (N >= 65536) R = 2, NWV = 8;                        // the output head
    else if (N >= 16384) R = 1, NWV = p.MT == 4 ? 16 : 8;  // gate||up: at 33 to 64 rows one workgroup a compute
                                                           // unit, so that the unit fetches the activation rows
                                                           // once, not twice (gate||up at 64 rows 61.1 -> 57.2 us;
                                                           // without that copying it takes 53.6)
    else R = 1, NWV = (K >= 8192 || N >= 4096) ? 8 : 4;
  }
  p.R = R;
  p.NWV = NWV;
  const int cap = 16 * R * NWV;
  int rows = cap;
  if (N >= 16384 && splits <= 1) {
    // dealt out evenly over the workgroups the chip holds at once: one a compute unit where a workgroup
    // has 256 rows (the head; sixteen wavefronts), two otherwise
    const int slots = 256 * ((R == 2 && NWV == 8) || NWV == 16 ? 1 : 2);
    const int rounds = (N + slots * cap - 1) / (slots * cap);
    rows = ((N + slots * rounds - 1) / (slots * rounds) + 3) & ~3;
    if (rows > cap) rows = cap;
  }
  p.rows_per_block = rows;
  p.groups = (N + p.rows_per_block - 1) / p.rows_per_block;
  int s = splits;
  if (s <= 0) {
    s = 1;
    while (p.groups * s < 192 && K / (2 * s) >= 512 && s < 32) s *= 2;
  }
  int ks = (K + s - 1) / s;
  ks = (ks + ROWS_KC - 1) / ROWS_KC * ROWS_KC;
  p.kslice = ks;
  p.splits = (K + ks - 1) / ks;
  return p;
}

extern "C" int he_gemm_rows_plan(int M, int N, int K, int* groups, int* splits) {
  if (M <= 0 || M > HE_GEMM_ROWS_MAX_M || N <= 0 || K <= 0) return -1;
  const RowsPlan p = rows_plan(M, N, K, 0, 0, 0);
  if (groups) *groups = p.groups;
  if (splits) *splits = p.splits;
  return 0;
}

template <int MT, int R, int NWV, bool GATED, typename TC>
static void launch_rows(const RowsPlan& p, void* C, float* partial, const void* X, const void* W,
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

template <bool GATED, typename TC>
static int dispatch_rows(const RowsPlan& p, void* C, float* partial, const void* X, const void* W,
                         const void* bias, int bias_dtype, int M, int N, int K, const RowsFusion& fu,
                         bool x_pieces, hipStream_t s) {
#define RW(MT_, R_, NWV_)                                                                      \
  if (p.MT == MT_ && p.R == R_ && p.NWV == NWV_) {                                             \
    launch_rows<MT_, R_, NWV_, GATED, TC>(p, C, partial, X, W, bias, bias_dtype, M, N, K, fu, x_pieces, s); \
    return 0;                                                                                  \
  }
  RW(2, 1, 4) RW(4, 1, 4) RW(4, 2, 4) RW(2, 1, 8) RW(4, 1, 8) RW(2, 2, 8) RW(4, 2, 8) RW(2, 1, 16) RW(4, 1, 16)
#undef RW
  he_set_error("he_gemm_rows_bf16: no kernel for MT=%d R=%d NWV=%d", p.MT, p.R, p.NWV);
  return -1;
}

extern "C" int he_gemm_rows_bf16(void* C, void* partial_f32, int64_t partial_floats, const void* A,
                                 const void* W, const void* bias, int M, int N, int K, int out_dtype,
                                 int bias_dtype, int gated, int R, int NWV, int splits,
                                 const void* scale_partials, int scale_count, float scale_eps,
                                 void* resid, const void* gain, int gain_dtype, void* xg, void* sq_out,
                                 int sq_count, int x_pieces, int out_pieces, int* splits_used,
                                 void* stream) {
  HE_REQUIRE(M > 0 && M <= HE_GEMM_ROWS_MAX_M, "he_gemm_rows_bf16: M=%d outside [1, %d]", M,
             HE_GEMM_ROWS_MAX_M);
  HE_REQUIRE(N > 0 && K > 0, "he_gemm_rows_bf16: bad sizes N=%d K=%d", N, K);
  HE_REQUIRE((K & 7) == 0, "he_gemm_rows_bf16: K=%d must be a multiple of 8", K);
  HE_REQUIRE(out_dtype == HE_BF16 || out_dtype == HE_F32, "he_gemm_rows_bf16: bad out dtype");
  HE_REQUIRE((((uintptr_t)A | (uintptr_t)W) & 15) == 0, "he_gemm_rows_bf16: operands must be 16-byte aligned");
  HE_REQUIRE(!gated || ((N & 1) == 0 && bias == nullptr),
             "he_gemm_rows_bf16: the gated epilogue needs an even N=%d and no bias", N);
  HE_REQUIRE(scale_partials == nullptr || scale_count > 0, "he_gemm_rows_bf16: row scale without partial sums");
  HE_REQUIRE(!out_pieces || ((resid != nullptr || out_dtype == HE_BF16) && ((gated ? N / 2 : N) & 7) == 0),
             "he_gemm_rows_bf16: a piece-major output is bf16 and a multiple of 8 wide");
  HE_REQUIRE(R <= 0 || R == 1 || R == 2, "he_gemm_rows_bf16: R=%d is not 1 or 2", R);
  HE_REQUIRE(NWV <= 0 || NWV == 4 || NWV == 8 || NWV == 16, "he_gemm_rows_bf16: %d wavefronts, not 4, 8 or 16", NWV);
  HE_REQUIRE((R <= 0) == (NWV <= 0), "he_gemm_rows_bf16: give both R and NWV, or neither");
  HE_REQUIRE(!(R == 2 && NWV == 4) || M > 32,
             "he_gemm_rows_bf16: two tiles a wavefront in four wavefronts are for more than 32 rows");
  const RowsPlan p = rows_plan(M, N, K, R, NWV, splits);
  HE_REQUIRE(p.groups <= 0x7fffffff && p.splits >= 1 && p.splits <= 65535, "he_gemm_rows_bf16: grid too large");
  if (splits_used) *splits_used = p.splits;
  const bool epilogue = gated || resid != nullptr || out_pieces || bias != nullptr;
  if (p.splits > 1) {
    HE_REQUIRE(!epilogue, "he_gemm_rows_bf16: a product cut into %d K slices leaves plain partial sums; "
               "bias and the gated, residual and piece-major epilogues need one slice", p.splits);
    const int64_t need = (int64_t)p.splits * M * N;
    HE_REQUIRE(partial_f32 != nullptr && partial_floats >= need && (((uintptr_t)partial_f32) & 15) == 0,
               "he_gemm_rows_bf16: room for %lld partial sums, need %lld (16-byte aligned)",
               (long long)partial_floats, (long long)need);
  } else if (resid != nullptr) {
    HE_REQUIRE(!gated && gain != nullptr && xg != nullptr && sq_out != nullptr,
               "he_gemm_rows_bf16: the residual epilogue needs gain, xg and sq_out, and no gate");
    HE_REQUIRE(sq_count == p.groups, "he_gemm_rows_bf16: %d partial sums per row given, the product has %d workgroups",
               sq_count, p.groups);
    HE_REQUIRE(gain_dtype == HE_F32 || gain_dtype == HE_BF16, "he_gemm_rows_bf16: bad gain dtype");
  } else {
    HE_REQUIRE(C != nullptr, "he_gemm_rows_bf16: no output");
  }
  RowsFusion fu;
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
  float* partial = (float*)partial_f32;
  int rc;
  HE_REQUIRE(!gated || out_dtype == HE_BF16, "he_gemm_rows_bf16: the gated epilogue writes bfloat16");
  if (gated)
    rc = dispatch_rows<true, bf16_t>(p, C, partial, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s);
  else
    rc = out_dtype == HE_BF16
             ? dispatch_rows<false, bf16_t>(p, C, partial, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s)
             : dispatch_rows<false, float>(p, C, partial, A, W, bias, bias_dtype, M, N, K, fu, x_pieces != 0, s);
  if (rc) return rc;
  return he_check_launch("he_gemm_rows_bf16");
}

// ---- the K slices of a product into a tensor -----------------------------------------
// out[m][n] = sum_s partial[s][m][n] (+ bias[n]), slices added in index order. Four neighbouring
// elements a thread where the width allows it; the loads of up to eight slices go out together
// before the first is added (a loop over the slices would wait for each in turn).
template <typename TC, int VEC>
__global__ void splitk_reduce_kernel(TC* __restrict__ C, const float* __restrict__ partial,
                                     const void* __restrict__ bias, int bias_dtype, int64_t total,
                                     int N, int splits) {
  const int64_t i = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * VEC;
  if (i >= total) return;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float v[8][VEC];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int sp = min(s0 + j, splits - 1);
      if (VEC == 4) {
        const float4 f = *reinterpret_cast<const float4*>(partial + sp * total + i);
        v[j][0] = f.x, v[j][1] = f.y, v[j][2] = f.z, v[j][3] = f.w;
      } else {
        v[j][0] = partial[sp * total + i];
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s0 + j < splits)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += v[j][e];
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e)
    if (bias != nullptr) acc[e] += load_param(bias, (i + e) % N, bias_dtype);
  if constexpr (VEC == 4) {
    rows_store4<TC>(C + i, acc, 4, 4);
  } else {
    C[i] = from_float<TC>(acc[0]);
  }
}

extern "C" int he_splitk_reduce(void* C, const void* partial_f32, const void* bias, int M, int N,
                                int splits, int out_dtype, int bias_dtype, void* stream) {
  HE_REQUIRE(M >= 0 && N > 0 && splits > 0, "he_splitk_reduce: bad sizes");
  HE_REQUIRE(out_dtype == HE_BF16 || out_dtype == HE_F32, "he_splitk_reduce: unknown dtype %d", out_dtype);
  if (M == 0) return 0;
  const int64_t total = (int64_t)M * N;
  const bool vec = (total & 3) == 0 && ((((uintptr_t)partial_f32) | ((uintptr_t)C)) & 15) == 0;
  const int64_t items = vec ? total / 4 : total;
  HE_REQUIRE((items + 255) / 256 <= 0x7fffffff, "he_splitk_reduce: too many elements for one launch");
  const unsigned blocks = (unsigned)((items + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
#define REDUCE(TC_, VEC_)                                                                        \
  splitk_reduce_kernel<TC_, VEC_><<<blocks, 256, 0, s>>>((TC_*)C, (const float*)partial_f32, bias, \
                                                         bias_dtype, total, N, splits)
  if (out_dtype == HE_BF16) {
    if (vec) REDUCE(bf16_t, 4); else REDUCE(bf16_t, 1);
  } else {
    if (vec) REDUCE(float, 4); else REDUCE(float, 1);
  }
#undef REDUCE
  return he_check_launch("he_splitk_reduce");
}

// ---- the K slices of a product into the residual stream -------------------------------
// resid[m][n] += sum_s partial[s][m][n] (+ bias[n]), slices in index order; xg[m][n] =
// bf16(resid * gain[n]) (row-major, or piece-major); sq[m][block] = the sum of resid^2 over the
// block's columns: what the residual epilogue of a one-slice product leaves (rows for the next
// norm, whose scale the next product applies). grid (column blocks of 1024, rows), 256 threads.
__global__ __launch_bounds__(256) void splitk_reduce_residual_kernel(
    float* __restrict__ resid, const float* __restrict__ partial, const void* __restrict__ bias,
    int bias_dtype, const void* __restrict__ gain, int gain_dtype, uint16_t* __restrict__ xg,
    float* __restrict__ sq_out, int M, int N, int splits, int out_pieces) {
  __shared__ float red[4];
  const int m = blockIdx.y;
  const int n = blockIdx.x * 1024 + 4 * threadIdx.x;
  float sq = 0.f;
  if (n < N) {
    const int valid = min(4, N - n);
    const int64_t at = (int64_t)m * N + n;
    const bool vec = valid == 4 && (N & 3) == 0;
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {
      const float4 r4 = *reinterpret_cast<const float4*>(resid + at);
      x[0] = r4.x, x[1] = r4.y, x[2] = r4.z, x[3] = r4.w;
    } else {
      for (int i = 0; i < valid; ++i) x[i] = resid[at + i];
    }
    float d[4] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {     // the loads of up to eight slices go out together, then they are added in order
      for (int s0 = 0; s0 < splits; s0 += 8) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          v[j] = *reinterpret_cast<const float4*>(partial + (int64_t)min(s0 + j, splits - 1) * M * N + at);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (s0 + j < splits) d[0] += v[j].x, d[1] += v[j].y, d[2] += v[j].z, d[3] += v[j].w;
      }
    } else {
      for (int s = 0; s < splits; ++s) {
        const float* p = partial + (int64_t)s * M * N + at;
        for (int i = 0; i < valid; ++i) d[i] += p[i];
      }
    }
    float g[4];
    for (int i = 0; i < 4; ++i) {
      const bool in = i < valid;
      if (in && bias != nullptr) d[i] += load_param(bias, n + i, bias_dtype);
      x[i] += d[i];
      g[i] = in ? x[i] * load_param(gain, n + i, gain_dtype) : 0.f;
      if (in) sq += x[i] * x[i];
    }
    if (vec) {
      *reinterpret_cast<float4*>(resid + at) = make_float4(x[0], x[1], x[2], x[3]);
    } else {
      for (int i = 0; i < valid; ++i) resid[at + i] = x[i];
    }
    if (out_pieces) {
      rows_store_pieces(xg, M, m, n, g, 4, valid);
    } else if (vec) {
      *reinterpret_cast<uint2*>(xg + at) = make_uint2(pack2_bf16(g[0], g[1]), pack2_bf16(g[2], g[3]));
    } else {
      for (int i = 0; i < valid; ++i) xg[at + i] = float_to_bf16_bits(g[i]);
    }
  }
  sq = wave_sum(sq);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sq;
  __syncthreads();
  if (threadIdx.x == 0) sq_out[(int64_t)m * gridDim.x + blockIdx.x] = ((red[0] + red[1]) + red[2]) + red[3];
}

extern "C" int he_splitk_reduce_residual_blocks(int N) { return N > 0 ? (N + 1023) / 1024 : 0; }

extern "C" int he_splitk_reduce_residual(void* resid_f32, const void* partial_f32, const void* bias,
                                         int bias_dtype, const void* gain, int gain_dtype, void* xg,
                                         void* sq_out, int sq_count, int M, int N, int splits,
                                         int out_pieces, void* stream) {
  HE_REQUIRE(M >= 0 && M <= 65535 && N > 0 && splits > 0, "he_splitk_reduce_residual: bad sizes");
  HE_REQUIRE(resid_f32 && partial_f32 && gain && xg && sq_out, "he_splitk_reduce_residual: missing buffers");
  HE_REQUIRE(sq_count == he_splitk_reduce_residual_blocks(N),
             "he_splitk_reduce_residual: %d partial sums per row given, %d column blocks", sq_count,
             he_splitk_reduce_residual_blocks(N));
  HE_REQUIRE(!out_pieces || (N & 7) == 0, "he_splitk_reduce_residual: a piece-major output is a multiple of 8 wide");
  HE_REQUIRE((((uintptr_t)resid_f32 | (uintptr_t)partial_f32) & 15) == 0 && (((uintptr_t)xg) & 7) == 0,
             "he_splitk_reduce_residual: buffers must be 16-byte aligned");
  if (M == 0) return 0;
  splitk_reduce_residual_kernel<<<dim3(sq_count, M), 256, 0, (hipStream_t)stream>>>(
      (float*)resid_f32, (const float*)partial_f32, bias, bias_dtype, gain, gain_dtype, (uint16_t*)xg,
      (float*)sq_out, M, N, splits, out_pieces);
  return he_check_launch("he_splitk_reduce_residual");
}
