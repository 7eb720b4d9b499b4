// Prompt attention over the paged cache with 32 queries a wavefront as one 32x32 MFMA tile,
// the softmax of one step of 32 keys running beside the matrix products of its neighbours.
//
// grid (ceil(max_q_len / 128), H, num_seqs), 256 threads. A workgroup takes 128 consecutive
// queries of one sequence and head, wavefront w the 32 queries 32w..32w+31. Tiles are
// transposed as in the other MFMA attention kernels (attention_mfma.hip): keys are the rows
// of the score tile and queries its columns, so a lane holds, for the one query of its
// column, 16 of the 32 scores of a step, the softmax statistics are per-lane scalars, and
// the probabilities a lane computes are, as they stand, its part of the B operand of the
// value product.
//
//   S^T[32 keys x 32 queries] = K[32 x hd] Q^T      NT products v_mfma_f32_32x32x16_bf16
//   O^T[hd x 32 queries]     += V^T[hd x 32] P^T    2 products per 32 head dims
//
// Row rho of the score tile is key kappa(rho) = rho with bits 2 and 3 exchanged. With that
// order both operands come out of a cache page as it lies in LDS (cache_layout.h) by one
// 16-byte read a lane, 16 consecutive lanes reading 256 consecutive bytes (no bank
// conflicts): lane L reads, for the K operand of head dims 16kk..16kk+15, the piece
// (t = L bit 4, ks = kk / 2, lg = 2 (kk % 2) + L bit 5, lr = L % 16); the eight scores
// i = 4kk'..4kk'+3, 4kk'+8..4kk'+11 of a lane are eight consecutive keys, the V^T piece
// lg = 2kk' + L bit 5.
//
// Pages go from global memory straight into LDS (global_load_lds, 16 bytes a lane, no
// registers in between), K one page ahead of V: between two barriers ("epoch" j) K of page
// j and V of page j - 1 are readable while K of page j + 1 and V of page j arrive. A
// wavefront enters an epoch with the raw scores of the second half of page j - 1 and the
// probabilities of its first half; it leaves it with the same of page j. In between:
//
//   products  O += V(j-1, first half) P ; S = K(j, first half) Q    beside  softmax of (j-1, second half)
//   products  O += V(j-1, second half) P ; S = K(j, second half) Q  beside  softmax of (j, first half)
//
// so the matrix cores and the vector ALU of one wavefront work at the same time. That loop
// has no masks and no branches but one: the reference point of the softmax follows the
// running maximum only when that has grown by more than 2^PW_SLACK, and the accumulators are
// rescaled only then. Epochs that hold a masked step (the diagonal, a window's start, the
// first and the last of a tile) run through a plain variant of the same contract.
// Workgroups with many keys are launched first, over all heads and sequences (a launch that
// fits on the chip at once puts its lightest beside its heaviest); an XCD sees neighbouring
// heads. Head sizes up to 128.
//
// parts > 1: grid.x counts (block of queries, part). The pages of a block are dealt out evenly to its
// parts; a part runs the same loops over its own pages and leaves unnormalised sums, reference
// point and sum of weights per query and head (ws_o, ws_ml) for attention_merge_rows_kernel
// (attention_mfma.hip). For steps of few queries against many keys, which would otherwise keep
// a fraction of the chip busy.
//
// Measured at 28 heads of 128, 4 kv heads (causal flops): 0.61 PFLOP/s at 2048 tokens,
// 0.94 at 8192, 1.1 at 16384, 0.85 for eight prompts of 2048. In the long runs the shader
// clock sits near 1.4 GHz (s_memtime against the 100 MHz counter), so 1.1 PFLOP/s is four
// fifths of what the matrix cores give at that clock; at 2048 tokens the launch is as long
// as its longest wavefront (33 epochs of about 2650 cycles, 1024 of them products).
#include "attention_tiles.h"

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;

#define PW_WAVES 4
#define PW_QUERIES (32 * PW_WAVES)
#define PW_SLACK 16.0f

template <int NT>
struct Pw {
  static constexpr int HD = 16 * NT;
  static constexpr int KS = (HD + 31) / 32;
  static constexpr int DT = (NT + 1) / 2;          // 32-dim tiles of O^T
  static constexpr int K_PIECES = 2 * 2 * KS * 64; // 16-byte pieces of a page of K, of V^T
  static constexpr int V_PIECES = 2 * NT * 64;
  static constexpr int K_CHUNKS = K_PIECES / 64, V_CHUNKS = V_PIECES / 64;   // KiB, one a wavefront and load
};

template <int NT>
struct WideTile {
  bf16x8 qf[NT];             // Q operand of head dims 16kk + 8g .. + 8 of the lane's query
  floatx16 o[Pw<NT>::DT];    // O^T[32dt + 8a + 4g + r][query], i = 4a + r, unnormalised
  float m, l;                // reference point of the lane's query; this lane's share of the sum
  int lo, hi;                // keys the lane's query sees
};

// position of score i of a lane of half g inside its step of 32 keys
__device__ __forceinline__ constexpr int pw_key_of(int i, int g) {
  return 16 * ((i >> 2) & 1) + 8 * g + 4 * (i >> 3) + (i & 3);
}

// A page (K or V^T) of one kv head, global memory -> LDS, a KiB a wavefront and instruction
// (lane l's 16 bytes land at the destination + 16 l); wavefront w copies the KiB
// PER w .. PER w + PER - 1 with one setting of M0 (the LDS address) and the instruction's
// offset, which counts for both addresses (16 cycles of issue a load, measured beside running
// products; a workgroup's 32 KiB a page take the compute unit's path from L2 about 500 cycles).
// The instruction is written out: given
// the builtin, the compiler makes every LDS read that follows wait for the load (it cannot
// tell the buffer being filled from the one being read), which is the opposite of what the
// double buffer is for. pw_epoch_end() waits for these loads; the compiler's own counting
// of its loads can only come out too careful by them, since loads complete in order.
// buf_bytes: LDS byte address of the page buffer (the same in all lanes); src: the page of
// this kv head + 8 elements a lane.
template <int CHUNKS>
__device__ __forceinline__ void pw_stage(uint32_t buf_bytes, const uint16_t* src, int wave) {
  constexpr int PER = (CHUNKS + PW_WAVES - 1) / PW_WAVES;
  static_assert(PER <= 4, "the instruction's offset reaches 4095 bytes");
  const int c0 = PER * wave;
  const uint16_t* from = src + 512 * c0;
  const uint32_t to = buf_bytes + 1024u * c0;
  uint32_t m0_before;   // M0 is the compiler's register: put back
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0" : "=&s"(m0_before) : "s"(to) : "memory");
  if (CHUNKS % PER == 0 && CHUNKS / PER == PW_WAVES) {
    if (PER > 0) asm volatile("global_load_lds_dwordx4 %0, off" :: "v"(from) : "memory");
    if (PER > 1) asm volatile("global_load_lds_dwordx4 %0, off offset:1024" :: "v"(from) : "memory");
    if (PER > 2) asm volatile("global_load_lds_dwordx4 %0, off offset:2048" :: "v"(from) : "memory");
    if (PER > 3) asm volatile("global_load_lds_dwordx4 %0, off offset:3072" :: "v"(from) : "memory");
  } else {
    if (PER > 0 && c0 + 0 < CHUNKS) asm volatile("global_load_lds_dwordx4 %0, off" :: "v"(from) : "memory");
    if (PER > 1 && c0 + 1 < CHUNKS) asm volatile("global_load_lds_dwordx4 %0, off offset:1024" :: "v"(from) : "memory");
    if (PER > 2 && c0 + 2 < CHUNKS) asm volatile("global_load_lds_dwordx4 %0, off offset:2048" :: "v"(from) : "memory");
    if (PER > 3 && c0 + 3 < CHUNKS) asm volatile("global_load_lds_dwordx4 %0, off offset:3072" :: "v"(from) : "memory");
  }
  asm volatile("s_mov_b32 m0, %0" :: "s"(m0_before) : "memory");
}

__device__ __forceinline__ const uint16_t* pw_page(const uint16_t* __restrict__ pool, int page, int num_pages,
                                                   int64_t stride, int lane) {
  if (page < 0 || page >= num_pages) page = 0;   // never for an admitted batch
  return pool + (int64_t)page * stride + 8 * lane;
}

// what the loop without masks stages next: LDS byte addresses, sources, whether a next K page exists
struct PwNext {
  uint32_t k_buf, v_buf;
  const uint16_t *k_src, *v_src;
  bool k_on;
};

// every thread's own loads have arrived, then everyone's
__device__ __forceinline__ void pw_epoch_end() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
}

template <int NT>
__device__ __forceinline__ floatx16 pw_scores(const bf16x8 (&qf)[NT], const uint4* k_lds, int kl, int hh) {
  constexpr int KS = Pw<NT>::KS;
  floatx16 s;
#pragma unroll
  for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
  for (int kk = 0; kk < NT; ++kk) {
    const bf16x8 kf = __builtin_bit_cast(bf16x8, k_lds[kl + hh * 2 * KS * 64 + (kk >> 1) * 64 + (kk & 1) * 32]);
    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], s, 0, 0, 0);
  }
  return s;
}

template <int NT>
__device__ __forceinline__ void pw_values(floatx16 (&o)[Pw<NT>::DT], const uint4* v_lds, int vl, int vl_last,
                                          int hh, const bf16x8 (&p)[2]) {
  constexpr int DT = Pw<NT>::DT;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    // the upper 16 rows of the last tile of an odd head size read its lower 16 again (never stored)
    const int base = ((NT & 1) && dt == DT - 1) ? vl_last : vl;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const bf16x8 vf = __builtin_bit_cast(bf16x8, v_lds[base + hh * NT * 64 + 2 * dt * 64 + 32 * kk]);
      o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p[kk], o[dt], 0, 0, 0);
    }
  }
}

// Softmax of one step of 32 keys from key_base on. Leaves P^T in p; the factor for the
// accumulators in alpha when the reference point moved (the return value, the same in all
// lanes). m and l are updated; the caller rescales o, after the value products of earlier
// steps that are still under way.
template <int NT>
__device__ __forceinline__ bool pw_softmax(WideTile<NT>& t, const floatx16& s, int key_base, int g,
                                           float scale_log2, bf16x8 (&p)[2], float& alpha) {
  float v[16];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int key = key_base + pw_key_of(i, g);
    v[i] = (key >= t.lo && key <= t.hi) ? s[i] : -INFINITY;
    mx = fmaxf(mx, v[i]);
  }
  mx = xor32_max(mx) * scale_log2;
  const float m_new = mx > t.m + PW_SLACK ? mx : t.m;
  const bool moved = __builtin_amdgcn_ballot_w64(m_new != t.m) != 0;   // wave-uniform
  const float m_use = m_new == -INFINITY ? 0.f : m_new;
  float sum = 0.f;
  uint32_t packed[8];
#pragma unroll
  for (int i = 0; i < 16; i += 2) {
    const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(v[i], scale_log2, -m_use));
    const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(v[i + 1], scale_log2, -m_use));
    packed[i >> 1] = pack2_bf16(e0, e1);
    // the sum of the rounded probabilities, the ones the value product uses
    sum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed[i >> 1]),
                                          __builtin_bit_cast(bf16x2, 0x3f803f80u), sum, false);
  }
  // product kk takes the scores 4kk..4kk+3 and 4kk+8..4kk+11: eight consecutive keys
  p[0] = __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[4], packed[5]));
  p[1] = __builtin_bit_cast(bf16x8, make_uint4(packed[2], packed[3], packed[6], packed[7]));
  alpha = 1.f;
  if (moved) {
    alpha = __builtin_amdgcn_exp2f(t.m - m_use);
    t.l *= alpha;
    t.m = m_new;
  }
  t.l += sum;
  return moved;
}

template <int NT>
__device__ __forceinline__ void pw_rescale(WideTile<NT>& t, float alpha) {
#pragma unroll
  for (int dt = 0; dt < Pw<NT>::DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) t.o[dt][i] *= alpha;
}

// One epoch with masks and range checks: steps hsA..hsB are the tile's. s_pend / p_pend as
// described at the top. k_lds: page j, v_lds: page j - 1.
template <int NT>
__device__ __forceinline__ void pw_plain_epoch(WideTile<NT>& t, floatx16& s_pend, bf16x8 (&p_pend)[2], int j,
                                               int hsA, int hsB, const uint4* k_lds, const uint4* v_lds,
                                               int kl, int vl, int vl_last, int g, float scale_log2) {
  const int h0 = 2 * j - 2, h1 = 2 * j - 1, h2 = 2 * j, h3 = 2 * j + 1;
  float alpha;
  if (h0 >= hsA && h0 <= hsB) pw_values<NT>(t.o, v_lds, vl, vl_last, 0, p_pend);
  if (h1 >= hsA && h1 <= hsB) {
    bf16x8 p[2];
    if (pw_softmax<NT>(t, s_pend, 32 * h1, g, scale_log2, p, alpha)) pw_rescale<NT>(t, alpha);
    pw_values<NT>(t.o, v_lds, vl, vl_last, 1, p);
  }
  if (h2 >= hsA && h2 <= hsB) {
    const floatx16 s = pw_scores<NT>(t.qf, k_lds, kl, 0);
    if (pw_softmax<NT>(t, s, 32 * h2, g, scale_log2, p_pend, alpha)) pw_rescale<NT>(t, alpha);
  }
  if (h3 >= hsA && h3 <= hsB) s_pend = pw_scores<NT>(t.qf, k_lds, kl, 1);
}

// One step of the loop without masks: the softmax of the scores in s_pend (step h) beside
// the value product of step h - 1 (its P^T in p_pend, its V^T in half hh of v_lds) and the score
// product of step h + 1 (half hh of k_lds). A wavefront issues in order, so the order here is
// the order on the machine: all sixteen operands are asked for first (a read asked for just
// ahead of its product would stall the wavefront for the LDS latency every time); with STAGE
// the loads of the next pages are issued then, while the first operand is on its way; then
// the products, each with its piece of the softmax behind it.
template <int NT, bool STAGE>
__device__ __forceinline__ void pw_fast_step(WideTile<NT>& t, floatx16& s_pend, bf16x8 (&p_pend)[2],
                                             const uint4* k_lds, const uint4* v_lds, int kl, int vl,
                                             int vl_last, int hh, int g, float scale_log2,
                                             PwNext& next, int wave) {
  constexpr int KS = Pw<NT>::KS, DT = Pw<NT>::DT;
  bf16x8 vf[DT][2], kf[NT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int base = ((NT & 1) && dt == DT - 1) ? vl_last : vl;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
      vf[dt][kk] = __builtin_bit_cast(bf16x8, v_lds[base + hh * NT * 64 + 2 * dt * 64 + 32 * kk]);
  }
#pragma unroll
  for (int kk = 0; kk < NT; ++kk)
    kf[kk] = __builtin_bit_cast(bf16x8, k_lds[kl + hh * 2 * KS * 64 + (kk >> 1) * 64 + (kk & 1) * 32]);
  __builtin_amdgcn_sched_barrier(0);
  if (STAGE) {
    if (next.k_on) pw_stage<Pw<NT>::K_CHUNKS>(next.k_buf, next.k_src, wave);
    pw_stage<Pw<NT>::V_CHUNKS>(next.v_buf, next.v_src, wave);
  }
  __builtin_amdgcn_sched_barrier(0);

  // Product by product: the value products first (their P^T is ready), then the score products
  // (a chain on one accumulator costs nothing: measured 32.8 cycles a product, chained or not),
  // and after each product the piece of the softmax that runs beside it: a product keeps the
  // matrix cores busy for 32 cycles, and vector instructions worth about 24 cycles issued
  // behind it are free (measured: two multiply + exp2 pairs behind every product, 35.5 cycles a
  // product; three, 46.8). The softmax is cut into 16 pieces: four of the maximum (the last
  // with the exchange between the halves and the new reference point), eight of two exponentials
  // each, four that round two pairs and add them up; product n of P gets the pieces
  // ceil(16 n / P) .. ceil(16 (n + 1) / P) - 1.
  constexpr int P = NT + 2 * DT;
  floatx16 s_next;
#pragma unroll
  for (int i = 0; i < 16; ++i) s_next[i] = 0.f;
  float mx = -INFINITY, m_new = t.m, sum = 0.f;
  bool moved = false;
  float e[16];
  uint32_t packed[8];
#pragma unroll
  for (int n = 0; n < P; ++n) {
    if (n < 2 * DT) {
      const int dt = n % DT, kk = n / DT;
      t.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt][kk], p_pend[kk], t.o[dt], 0, 0, 0);
    } else {
      s_next = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[n - 2 * DT], t.qf[n - 2 * DT], s_next, 0, 0, 0);
    }
#pragma unroll
    for (int piece = (16 * n + P - 1) / P; piece < (16 * (n + 1) + P - 1) / P; ++piece) {
      if (piece < 4) {
#pragma unroll
        for (int i = 4 * piece; i < 4 * piece + 4; ++i) mx = fmaxf(mx, s_pend[i]);
        if (piece == 3) {
          mx = xor32_max(mx) * scale_log2;
          m_new = mx > t.m + PW_SLACK ? mx : t.m;
          moved = __builtin_amdgcn_ballot_w64(m_new != t.m) != 0;   // the same in all lanes
        }
      } else if (piece < 12) {
#pragma unroll
        for (int i = 2 * (piece - 4); i < 2 * (piece - 4) + 2; ++i)
          e[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_pend[i], scale_log2, -m_new));
      } else {
        // the sum is taken over the rounded probabilities, the ones the value product uses: one dot
        // product with (1, 1) per pair. (The empty statements keep the compiler from moving this
        // work behind the rescaling branch below, where no product would run beside it.)
#pragma unroll
        for (int q = 2 * (piece - 12); q < 2 * (piece - 12) + 2; ++q) {
          packed[q] = pack2_bf16(e[2 * q], e[2 * q + 1]);
          asm volatile("" : "+v"(packed[q]));
          sum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed[q]),
                                                __builtin_bit_cast(bf16x2, 0x3f803f80u), sum, false);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // product kk takes the scores 4kk..4kk+3 and 4kk+8..4kk+11: eight consecutive keys
  p_pend[0] = __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[4], packed[5]));
  p_pend[1] = __builtin_bit_cast(bf16x8, make_uint4(packed[2], packed[3], packed[6], packed[7]));
  if (moved) {
    const float alpha = __builtin_amdgcn_exp2f(t.m - m_new);
    t.l *= alpha;
    t.m = m_new;
    pw_rescale<NT>(t, alpha);
  }
  t.l += sum;
  s_pend = s_next;
}

template <int NT>
__global__ __launch_bounds__(64 * PW_WAVES) __attribute__((amdgpu_waves_per_eu(2, 2))) void
attention_prefill_wide_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q,
    const uint16_t* __restrict__ kpool, const uint16_t* __restrict__ vpool,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ page_table, int max_blocks,
    int num_pages, int H, int KVH, int window, float scale, int parts, float* __restrict__ ws_o,
    float* __restrict__ ws_ml) {
  constexpr int HD = Pw<NT>::HD, KS = Pw<NT>::KS, DT = Pw<NT>::DT;
  constexpr int KP = Pw<NT>::K_PIECES, VP = Pw<NT>::V_PIECES;
  __shared__ uint4 k_lds[2 * KP];
  __shared__ uint4 v_lds[2 * VP];

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 31, g = lane >> 5;
  // Order of the work. Workgroups start in the order of their number and go to the HE_XCDS
  // XCDs in turn. The query blocks with the most keys (the last of each sequence) come first,
  // over all heads and sequences, so that what is left for the end of the launch is short.
  // Of the rows (head, sequence) an XCD then sees every (HE_XCDS / g)-th, g = gcd(HE_XCDS,
  // rows); the rows are numbered so that these are neighbours, i.e. few kv heads, whose pages
  // the XCD's own L2 keeps.
  const int rows = gridDim.y * gridDim.z;
  const int launched = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  int gcd = HE_XCDS;
  while (rows % gcd) gcd >>= 1;               // HE_XCDS is a power of two
  // When the whole launch is on the chip at once (two workgroups a compute unit), a unit's second
  // workgroup is the one launched HE_CUS after its first (the 33rd of its XCD): the heaviest gets
  // the lightest beside it, and so on, and every unit has about the same to do (2048 tokens,
  // 28 heads: 52.1 -> 49.6 us).
  int rank = launched;
  if ((int)(gridDim.x * rows) <= 2 * HE_CUS) {
    const int x = launched % HE_XCDS, j = launched / HE_XCDS;
    const int of_xcd = ((int)(gridDim.x * rows) - x + HE_XCDS - 1) / HE_XCDS;
    rank = x + HE_XCDS * (j < HE_CUS / HE_XCDS ? j : of_xcd - 1 - (j - HE_CUS / HE_XCDS));
  }
  const int rho = rank % rows;
  const int row = (rho % gcd) * (rows / gcd) + rho / gcd;
  const int gx = gridDim.x - 1 - rank / rows;   // gridDim.x = query blocks x parts
  const int bx = gx / parts, part = gx - bx * parts;
  const int seq = row % gridDim.z, h = row / gridDim.z;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int row0 = cu_seqlens[seq];
  const int q_len = cu_seqlens[seq + 1] - row0;
  const int q0 = PW_QUERIES * bx;
  if (q0 >= q_len) return;
  const int start = seq_start[seq];
  const int kvh = h / (H / KVH);
  const int32_t* pt = page_table + (int64_t)slot * max_blocks;
  const int64_t k_stride = (int64_t)KVH * he_k_page_elems(HD), v_stride = (int64_t)KVH * he_v_page_elems(HD);
  const uint16_t* kp = kpool + (int64_t)kvh * he_k_page_elems(HD);
  const uint16_t* vp = vpool + (int64_t)kvh * he_v_page_elems(HD);
  const float scale_log2 = scale * 1.4426950408889634f;

  // the workgroup's pages: from the first key its first query sees to its last query
  const int blk_last = start + min(q0 + PW_QUERIES, q_len) - 1;
  const int blk_first = window > 0 ? max(0, start + q0 + 1 - window) : 0;
  int pbA = blk_first >> HE_PAGE_SHIFT, pbB = blk_last >> HE_PAGE_SHIFT;
  if (parts > 1) {
    // this workgroup's share of the block's pages; one without pages leaves empty parts
    const int per = (pbB - pbA + parts) / parts;
    pbA += part * per;
    pbB = min(pbB, pbA + per - 1);
  }

  // the wavefront's tile; a query beyond the sequence doubles the last one and is not stored
  const int qt = q0 + 32 * wave;
  const bool tile = qt < q_len;
  const int qi = min(qt + col, q_len - 1);
  if (pbA > pbB) {
    // a part without pages (more parts than the block has pages): empty parts for its queries
    if (tile && qt + col < q_len) {
      const int64_t idx = ((int64_t)(row0 + qi) * H + h) * parts + part;
      if (g == 0) *reinterpret_cast<float2*>(ws_ml + 2 * idx) = make_float2(-INFINITY, 0.f);
      for (int d = 4 * g; d < HD; d += 8) *reinterpret_cast<float4*>(ws_o + idx * HD + d) = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    return;
  }
  WideTile<NT> t;
  t.hi = start + qi;
  t.lo = window > 0 ? max(0, t.hi + 1 - window) : 0;
  t.m = -INFINITY;
  t.l = 0.f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) t.o[dt][i] = 0.f;
  {
    const uint16_t* qrow = q + ((int64_t)(row0 + qi) * H + h) * HD + 8 * g;
#pragma unroll
    for (int kk = 0; kk < NT; ++kk) t.qf[kk] = ld8(qrow + 16 * kk, true);
  }
  // steps of 32 keys (hs: keys 32hs..32hs+31) of the tile: hsA..hsB; without a mask: hsI0..hsI1-1
  const int first_pos = start + qt, last_pos = start + min(qt + 31, q_len - 1);
  const int lo_min = window > 0 ? max(0, first_pos + 1 - window) : 0;
  const int lo_max = window > 0 ? max(0, last_pos + 1 - window) : 0;
  // (a part has the steps of its own pages only)
  const int hsA = tile ? max(lo_min >> 5, 2 * pbA) : 1, hsB = tile ? min(last_pos >> 5, 2 * pbB + 1) : 0;
  const int hsI0 = (lo_max + 31) >> 5, hsI1 = (first_pos + 1) >> 5;
  // epochs of the loop without masks: steps 2j-2 .. 2j+1 are the tile's, 2j-1 and 2j unmasked
  int jF0 = max(max((hsA + 3) >> 1, (hsI0 + 2) >> 1), pbA + 1), jF1 = min((hsI1 - 1) >> 1, pbB);
  if (!tile || hsI1 < 1 || jF0 > jF1) { jF0 = pbB + 2; jF1 = pbB + 1; }

  const int kl = ((lane >> 4) & 1) * KS * 64 + 16 * g + (lane & 15);
  const int vl_last = 16 * g + (lane & 15), vl = vl_last + ((lane >> 4) & 1) * 64;

  const uint32_t k_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)k_lds;
  const uint32_t v_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)v_lds;
  floatx16 s_pend;
  bf16x8 p_pend[2];
#pragma unroll
  for (int i = 0; i < 16; ++i) s_pend[i] = 0.f;
  p_pend[0] = p_pend[1] = __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0));

  pw_stage<Pw<NT>::K_CHUNKS>(k_base + (pbA & 1) * KP * 16, pw_page(kp, pt[pbA], num_pages, k_stride, lane), wave);
  pw_epoch_end();
  // Q has arrived before the loops begin: a wait for it inside them would also wait for the page on its way
#pragma unroll
  for (int kk = 0; kk < NT; ++kk) asm volatile("" : "+v"(t.qf[kk]));
  int j = pbA;
  for (; j < jF0; ++j) {
    if (j + 1 <= pbB) pw_stage<Pw<NT>::K_CHUNKS>(k_base + ((j + 1) & 1) * KP * 16, pw_page(kp, pt[j + 1], num_pages, k_stride, lane), wave);
    if (j <= pbB) pw_stage<Pw<NT>::V_CHUNKS>(v_base + (j & 1) * VP * 16, pw_page(vp, pt[j], num_pages, v_stride, lane), wave);
    pw_plain_epoch<NT>(t, s_pend, p_pend, j, hsA, hsB, k_lds + (j & 1) * KP, v_lds + ((j - 1) & 1) * VP, kl, vl,
                       vl_last, g, scale_log2);
    pw_epoch_end();
  }
  // the pages the loop without masks stages in its first epoch; the numbers of the later ones are
  // read an epoch ahead
  int page_k = 0, page_v = 0;
  if (j <= jF1) {
    page_k = pt[min(j + 1, pbB)];
    page_v = pt[j];
    asm volatile("" :: "s"(page_k), "s"(page_v));   // arrived before the loop, for the same reason as below
  }
  for (; j <= jF1; ++j) {
    PwNext next;
    next.k_on = j + 1 <= pbB;
    next.k_buf = k_base + ((j + 1) & 1) * KP * 16;
    next.v_buf = v_base + (j & 1) * VP * 16;
    next.k_src = pw_page(kp, page_k, num_pages, k_stride, lane);
    next.v_src = pw_page(vp, page_v, num_pages, v_stride, lane);   // j <= pbB: the tile's own keys lie beyond step 2j
    const uint4* kb = k_lds + (j & 1) * KP;
    const uint4* vb = v_lds + ((j - 1) & 1) * VP;
    pw_fast_step<NT, true>(t, s_pend, p_pend, kb, vb, kl, vl, vl_last, 0, g, scale_log2, next, wave);
    pw_fast_step<NT, false>(t, s_pend, p_pend, kb, vb, kl, vl, vl_last, 1, g, scale_log2, next, wave);
    // asked for here, not earlier: scalar loads count with the LDS reads, and a wait for an LDS read
    // that follows one would wait for all of them; the barrier below waits for everything anyway
    __builtin_amdgcn_sched_barrier(0);
    page_k = pt[min(j + 2, pbB)];
    page_v = pt[min(j + 1, pbB)];
    pw_epoch_end();
  }
  for (; j <= pbB + 1; ++j) {
    if (j + 1 <= pbB) pw_stage<Pw<NT>::K_CHUNKS>(k_base + ((j + 1) & 1) * KP * 16, pw_page(kp, pt[j + 1], num_pages, k_stride, lane), wave);
    if (j <= pbB) pw_stage<Pw<NT>::V_CHUNKS>(v_base + (j & 1) * VP * 16, pw_page(vp, pt[j], num_pages, v_stride, lane), wave);
    pw_plain_epoch<NT>(t, s_pend, p_pend, j, hsA, hsB, k_lds + (j & 1) * KP, v_lds + ((j - 1) & 1) * VP, kl, vl,
                       vl_last, g, scale_log2);
    pw_epoch_end();
  }

  const float l = xor32_sum(t.l);
  if (!tile || qt + col >= q_len) return;
  if (parts > 1) {
    // one of several parts of the keys: the sums as they stand, with their reference point, for
    // attention_merge_kernel (O fp32 [hd], then (m, l) with m in the base-2 domain)
    const int64_t idx = ((int64_t)(row0 + qi) * H + h) * parts + part;
    if (g == 0) *reinterpret_cast<float2*>(ws_ml + 2 * idx) = make_float2(t.m, l);
    float* orow = ws_o + idx * HD + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        if (32 * dt + 8 * a >= HD) continue;
        *reinterpret_cast<float4*>(orow + 32 * dt + 8 * a) =
            make_float4(t.o[dt][4 * a], t.o[dt][4 * a + 1], t.o[dt][4 * a + 2], t.o[dt][4 * a + 3]);
      }
    return;
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  uint16_t* orow = out + ((int64_t)(row0 + qi) * H + h) * HD + 4 * g;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      if (32 * dt + 8 * a >= HD) continue;
      uint2 w;
      w.x = pack2_bf16(t.o[dt][4 * a] * inv, t.o[dt][4 * a + 1] * inv);
      w.y = pack2_bf16(t.o[dt][4 * a + 2] * inv, t.o[dt][4 * a + 3] * inv);
      *reinterpret_cast<uint2*>(orow + 32 * dt + 8 * a) = w;
    }
}

int he_attention_prefill_wide(void* out, const void* q, const void* kpool, const void* vpool,
                              const void* cu_seqlens, const void* seq_slot, const void* seq_start,
                              const void* page_table, int max_blocks, int num_pages, int num_seqs,
                              int max_q_len, int H, int KVH, int hd, int window, float scale,
                              int parts, float* ws_o, float* ws_ml, void* stream) {
  HE_REQUIRE(hd % 16 == 0 && hd >= 16 && hd <= 128,
             "he_attention_prefill_wide: head_dim %d must be a multiple of 16 up to 128", hd);
  HE_REQUIRE(parts >= 1 && parts <= 64 && (parts == 1 || (ws_o != nullptr && ws_ml != nullptr)),
             "he_attention_prefill_wide: %d parts (1 to 64, with room for them)", parts);
  const int64_t gx = (int64_t)((max_q_len + PW_QUERIES - 1) / PW_QUERIES) * parts;
  HE_REQUIRE(gx * H * num_seqs < (1ll << 31), "he_attention_prefill_wide: grid too large");
  dim3 grid((unsigned)gx, H, num_seqs);
  hipStream_t s = (hipStream_t)stream;
#define PREFILL_WIDE(NTV)                                                                       \
  case NTV:                                                                                     \
    attention_prefill_wide_kernel<NTV><<<grid, 64 * PW_WAVES, 0, s>>>(                          \
        (uint16_t*)out, (const uint16_t*)q, (const uint16_t*)kpool, (const uint16_t*)vpool,     \
        (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, (const int32_t*)seq_start,        \
        (const int32_t*)page_table, max_blocks, num_pages, H, KVH, window, scale, parts, ws_o,  \
        ws_ml);                                                                                 \
    break;
  switch (hd / 16) {
    PREFILL_WIDE(1) PREFILL_WIDE(2) PREFILL_WIDE(3) PREFILL_WIDE(4)
    PREFILL_WIDE(5) PREFILL_WIDE(6) PREFILL_WIDE(7) PREFILL_WIDE(8)
  }
#undef PREFILL_WIDE
  return he_check_launch("he_attention_prefill_wide");
}
