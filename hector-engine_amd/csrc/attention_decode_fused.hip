// One-token attention in one launch: projection bias, rotary encoding of q and of the
// new key, the cache write of the new key and value, attention over the cache and the
// merge of the key slices. It replaces three launches (the q/k/v kernel, the split
// attention kernel and its merge) where the encoding is a rotation of the whole head and
// the head size is 64 or 128, so that the two elements of a rotated pair sit in
// the same lane of the MFMA operand. Reference ops it covers: add_bias, rope, kv_cache_update,
// attention_cached (kernels/elementwise.cu:307-323, kernels/attention.cu:516-558,
// :1067-1097, :337-494).
//
// grid (KVH * head_tiles, rows, Z), 64 * NW threads. The workgroups (., ., z) own one
// sequence and kv head; the query heads of the group are the columns of the tiles
// (attention_tiles.h). The keys [first, p] are cut into Z * NW slices, one per wavefront.
// The wavefront whose slice holds the new position p first writes the new key (bias,
// rotation) and value into the cache and then reads them back with the rest of its
// slice - the same wavefront, behind a workgroup-scope fence; no other wavefront reads
// that row. Every wavefront leaves (m, l, O) of its slice in LDS and the workgroup joins
// them in wavefront order: O = sum_w O_w 2^(m_w - M), L = sum_w l_w 2^(m_w - M). With
// Z = 1 the workgroup stores O / L; with more (few sequences: one workgroup per sequence
// and kv head would leave most of the chip, and its memory bandwidth, idle) it stores
// (M, L, O) and attention_merge_kernel joins the Z parts in a second launch.
#include "attention_tiles.h"
#include "hector_kernels.h"

#define FUSED_MIN_CHUNK 64
#define FUSED_TAIL_SLICES 16   // from so many slices on, the step with the new position is a slice of its own

// q of the group's heads as B operand, from the un-biased projection row: lane (lr =
// head column, lg) holds dims 32ks + 8lg .. +8 of head lr for every k step ks. In two parts,
// so that the loads can be issued before anything else and the rotation done while the first
// keys are on their way: the biased values, then the rotation. The partner of dim d < half is
// d + half = the same lane's element in k step ks + half/32. sn, c: the sine and cosine of
// angle `lane` (lanes below half), fetched from the lane that holds them.
template <int NT>
struct QLoads {
  uint4 raw[NT / 2], bias[NT / 2];
  bool vec_bias;
};

// Issues the loads of q and, where the bias is bf16 and aligned, of its bias (eight values of
// a k step in one load). No load sits behind a per-lane condition (the caller's head index is
// clamped, so every lane has an address it may read; a column without a head is zeroed
// afterwards): loads behind branches are waited for one by one, these go out together and are
// waited for where q_biased() turns them into values, after everything else has been asked for.
template <int NT>
__device__ __forceinline__ void q_issue(QLoads<NT>& q, const uint16_t* qrow, const void* bias,
                                        int bias_dtype, int bias_off, int lg) {
  constexpr int KS = NT / 2;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) q.raw[ks] = *reinterpret_cast<const uint4*>(qrow + 32 * ks + 8 * lg);
  q.vec_bias = bias != nullptr && bias_dtype == HE_BF16 && (((uintptr_t)bias) & 15) == 0;
  // without such a bias the same loads read q again and their values are dropped: a branch around
  // them would end in register copies that wait for the loads
  const uint16_t* b = q.vec_bias ? (const uint16_t*)bias + bias_off : qrow;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) q.bias[ks] = *reinterpret_cast<const uint4*>(b + 32 * ks + 8 * lg);
}

template <int NT>
__device__ __forceinline__ void q_biased(float (&x)[NT / 2][8], const QLoads<NT>& q, const void* bias,
                                         int bias_dtype, int bias_off, bool valid, int lg) {
  constexpr int KS = NT / 2;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const uint32_t w[4] = {q.raw[ks].x, q.raw[ks].y, q.raw[ks].z, q.raw[ks].w};
    const uint32_t keep = q.vec_bias ? 0xffffffffu : 0u;
    const uint32_t bw[4] = {q.bias[ks].x & keep, q.bias[ks].y & keep, q.bias[ks].z & keep, q.bias[ks].w & keep};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float lo = __uint_as_float(w[j] << 16) + __uint_as_float(bw[j] << 16);
      const float hi = __uint_as_float(w[j] & 0xffff0000u) + __uint_as_float(bw[j] & 0xffff0000u);
      x[ks][2 * j] = valid ? lo : 0.f;
      x[ks][2 * j + 1] = valid ? hi : 0.f;
    }
  }
  if (bias != nullptr && !q.vec_bias && valid) {   // a bias in 32-bit, or not aligned: value by value
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) x[ks][j] += load_param(bias, bias_off + 32 * ks + 8 * lg + j, bias_dtype);
  }
}

// The projection row from the K slices of its product: the product of 17 to 64 rows is cut along K
// across workgroups and leaves fp32 sums [slices][rows][width] (gemm_rows.hip). Added in slice
// order and rounded to bfloat16, the values are the bits he_splitk_reduce would have written, and
// its launch is not needed. The loads of up to eight slices go out together.
template <typename V>
__device__ __forceinline__ V slices_sum(const float* part, int slices, int64_t slice_stride);
template <>
__device__ __forceinline__ float4 slices_sum<float4>(const float* part, int slices, int64_t slice_stride) {
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s0 = 0; s0 < slices; s0 += 8) {
    float4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const float4*>(part + (int64_t)min(s0 + j, slices - 1) * slice_stride);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s0 + j < slices) acc.x += v[j].x, acc.y += v[j].y, acc.z += v[j].z, acc.w += v[j].w;
  }
  return acc;
}
template <>
__device__ __forceinline__ float slices_sum<float>(const float* part, int slices, int64_t slice_stride) {
  float acc = 0.f;
  for (int s0 = 0; s0 < slices; s0 += 8) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = part[(int64_t)min(s0 + j, slices - 1) * slice_stride];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s0 + j < slices) acc += v[j];
  }
  return acc;
}
__device__ __forceinline__ float as_bf16(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }

template <int NT>
__device__ __forceinline__ void rotate_q(bf16x8* qf, float (&x)[NT / 2][8], int lg, float sn, float c) {
  constexpr int KS = NT / 2;
  constexpr int HS = KS / 2;   // k steps per half of the head
#pragma unroll
  for (int ks = 0; ks < HS; ++ks)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = 32 * ks + 8 * lg + j;
      const float si = __shfl(sn, i, HE_WAVE), ci = __shfl(c, i, HE_WAVE);
      const float a0 = x[ks][j], a1 = x[ks + HS][j];
      // one multiply-add each, written out: left to the compiler, the two instantiations of the
      // kernel may fuse the two products differently and differ in a last bit
      x[ks][j] = fmaf(a0, ci, -(a1 * si));
      x[ks + HS][j] = fmaf(a0, si, a1 * ci);
    }
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = __builtin_bit_cast(
        bf16x8, make_uint4(pack2_bf16(x[ks][0], x[ks][1]), pack2_bf16(x[ks][2], x[ks][3]),
                           pack2_bf16(x[ks][4], x[ks][5]), pack2_bf16(x[ks][6], x[ks][7])));
}

// SLICED: qkv is null and the projection row comes as the fp32 sums of its K slices,
// qkv_part [qkv_slices][.][qkv_stride], slice_stride elements from slice to slice.
template <int NT, bool SLICED>
__global__ __launch_bounds__(512) void attention_decode_fused_kernel(
    uint16_t* __restrict__ out, float* __restrict__ ws_o, float* __restrict__ ws_ml,
    const uint16_t* __restrict__ qkv, const float* __restrict__ qkv_part, int qkv_slices,
    int64_t slice_stride, int64_t qkv_stride,
    const void* __restrict__ bias, int bias_dtype, uint16_t* kpool, uint16_t* vpool,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ page_table, int max_blocks,
    int num_pages, const float* __restrict__ inv_freq, int rotary_dim, int H, int KVH,
    int head_tiles, int window, float scale, int write_kv, int out_pieces) {
  constexpr int HD = 16 * NT;
  constexpr int KS = (HD + 31) / 32;
  extern __shared__ __attribute__((aligned(16))) float lds[];   // [NW][GT][HD] O, then [NW][GT][2] (m, l)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int kvh = blockIdx.x / head_tiles, ht = blockIdx.x % head_tiles;
  const int row = blockIdx.y;
  const int G = H / KVH;
  const int GT = min(16, G - 16 * ht);     // heads of this tile
  const bool h_ok = lr < GT;
  const int h = kvh * G + 16 * ht + min(lr, GT - 1);
  // loads that need nothing but the row: issued first, used last
  // seq_slot null: the page table has a row per row of the step (the host has gathered the
  // sequences' page numbers into the step's metadata), so its address needs nothing but the row and
  // its lines are asked for at once: with the table of the cache the numbers come at the end of a
  // chain row -> sequence -> slot -> table (3.0 us after the kernel's start, measured with time
  // stamps inside it, the table's line from memory every time: the weights of a layer have passed
  // through the caches since the layer before read it).
  const bool by_row = seq_slot == nullptr;
  // (an ordinary load whose value is "used" by an empty statement at the kernel's end: the compiler
  // keeps the load, counts it, and holds its register until then. Written as inline assembly the
  // load's register counted as free at once, and what arrived later overwrote whatever lived there
  // by then; a volatile load bypasses the caches and is waited for where it stands.)
  int touched = 0;
  if (by_row && lane < ((max_blocks * 4 + 127) >> 7)) touched = page_table[(int64_t)row * max_blocks + 32 * lane];
  const uint16_t* qkv_row = SLICED ? nullptr : qkv + (int64_t)row * qkv_stride;
  const float* part_row = SLICED ? qkv_part + (int64_t)row * qkv_stride : nullptr;
  QLoads<NT> ql;
  if (!SLICED) q_issue<NT>(ql, qkv_row + (int64_t)h * HD, bias, bias_dtype, h * HD, lg);
  // SLICED: the first eight slices of the four q values this thread adds (see below) are asked for
  // here, with everything else that needs nothing but the row
  float4 q_early[8];
  const int q_col = (kvh * G + 16 * ht) * HD + 4 * min((int)threadIdx.x, GT * (HD / 4) - 1);
  if (SLICED) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      q_early[j] = *reinterpret_cast<const float4*>(part_row + q_col + (int64_t)min(j, qkv_slices - 1) * slice_stride);
  }
  const float freq = inv_freq[min(lane, HD / 2 - 1)];   // no condition in front of the load (the lanes beyond take no angle)
  const int seq = row_seq[row];
  const int Z = gridDim.z, z = blockIdx.z;
  // where dims d.. of head (column) hg of this tile go: row-major [rows, H HD], or piece-major
  // (16-byte pieces [H HD / 8][rows][8])
  auto out_at = [&](int hg, int d) {
    const int64_t c = (int64_t)(kvh * G + 16 * ht + hg) * HD + d;
    return out_pieces ? out + ((c >> 3) * gridDim.y + row) * 8 + (c & 7) : out + (int64_t)row * H * HD + c;
  };
  if (seq < 0) {                           // padding row: zeros (from the merge kernel if there is one)
    if (Z == 1)
      for (int i = threadIdx.x; i < GT * HD; i += blockDim.x) *out_at(i / HD, i % HD) = 0;
    return;
  }
  const int slot = by_row ? row : seq_slot[seq];
  const int p = positions[row];
  const int n_keys = p + 1;
  const int first = window > 0 ? max(0, n_keys - window) : 0;
  const int span_lo = first & ~31;
  const int slices = Z * nw;
  // With many slices the last one is the step of 32 keys that holds the new position, and the keys
  // before it are dealt out to the others: the wavefront that writes the new key reads its slice
  // only after the write, so its walk is the one the launch waits for, and it is now one step long
  // whatever the length (with equal slices the last one grew from one step to all of a slice as the
  // sequence grew: 11.9 to 14.3 us a layer at 8 sequences of 2100 to 2400 keys, now 11.9).
  const bool tail_slice = slices >= FUSED_TAIL_SLICES;
  const int body_end = tail_slice ? (p & ~31) : n_keys;
  const int body_slices = tail_slice ? slices - 1 : slices;
  int chunk = (body_end - span_lo + body_slices - 1) / body_slices;
  chunk = max(FUSED_MIN_CHUNK, (chunk + 31) & ~31);
  const int slice = z * nw + wave;
  const bool is_tail = tail_slice && slice == slices - 1;
  const int kb_begin = is_tail ? body_end : span_lo + slice * chunk;
  const int kb_end = is_tail ? n_keys : min(kb_begin + chunk, body_end);
  const int32_t* pt = page_table + (int64_t)slot * max_blocks;
  const bool has_keys = kb_begin < kb_end;   // uniform in the wavefront
  // the first keys and values are asked for before the angles are computed and q is rotated -
  // unless this wavefront writes the new key into that very step
  const bool writes = write_kv && p >= kb_begin && p < kb_end;
  const bool early = has_keys && !(writes && p < kb_begin + 32);
  // The page-table entries are asked for; what was asked for at the top is turned into values
  // while they come, so that nothing older than the keys has to be waited for once those are on
  // their way (behind their conditional loads the compiler waits for everything in flight).
  AttendCursor<NT> cursor;
  if (early) attend_pages<NT>(cursor, pt, max_blocks, kb_begin);
  float qx[NT / 2][8];
  if (!SLICED) q_biased<NT>(qx, ql, bias, bias_dtype, h * HD, h_ok, lg);
  // The angle is formed here, ahead of the loads of the first keys: its frequency was asked for at
  // the top, and a wait for it behind those loads would be a wait for them too (loads complete in
  // order): the sines and the rotation of q, which are meant to run while the keys are on their way,
  // ran after them (2.4 us of the kernel's 11).
  float angle = (float)p * freq;
  asm volatile("" : "+v"(angle));
  __builtin_amdgcn_sched_barrier(0);
  if (early) attend_first<NT>(cursor, kpool, vpool, num_pages, KVH, kvh, kb_begin, lr, lg);
  if (SLICED) {
    // The workgroup adds the slices of its heads' q once, four neighbouring values a thread, and hands
    // the sums round through LDS (the buffer the join uses at the end); every wavefront then takes its
    // operand's values from there. Summed wavefront by wavefront the same values would be fetched
    // as many times as the workgroup has wavefronts, a round trip a slice.
    const int h0 = kvh * G + 16 * ht;
    for (int v4 = threadIdx.x; v4 < GT * (HD / 4); v4 += blockDim.x) {
      const int col = h0 * HD + 4 * v4;
      float4 sum;
      if (v4 == (int)threadIdx.x && qkv_slices <= 8) {      // the loads issued at the top
        sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (j < qkv_slices) sum.x += q_early[j].x, sum.y += q_early[j].y, sum.z += q_early[j].z, sum.w += q_early[j].w;
      } else {
        sum = slices_sum<float4>(part_row + col, qkv_slices, slice_stride);
      }
      float q4[4] = {as_bf16(sum.x), as_bf16(sum.y), as_bf16(sum.z), as_bf16(sum.w)};
      if (bias != nullptr)
        for (int i = 0; i < 4; ++i) q4[i] += load_param(bias, col + i, bias_dtype);
      *reinterpret_cast<float4*>(lds + 4 * v4) = make_float4(q4[0], q4[1], q4[2], q4[3]);
    }
    __syncthreads();
    const float* ql_row = lds + min(lr, GT - 1) * HD + 8 * lg;
#pragma unroll
    for (int ks = 0; ks < NT / 2; ++ks) {
      const float4 a = *reinterpret_cast<const float4*>(ql_row + 32 * ks);
      const float4 b = *reinterpret_cast<const float4*>(ql_row + 32 * ks + 4);
      qx[ks][0] = h_ok ? a.x : 0.f, qx[ks][1] = h_ok ? a.y : 0.f, qx[ks][2] = h_ok ? a.z : 0.f, qx[ks][3] = h_ok ? a.w : 0.f;
      qx[ks][4] = h_ok ? b.x : 0.f, qx[ks][5] = h_ok ? b.y : 0.f, qx[ks][6] = h_ok ? b.z : 0.f, qx[ks][7] = h_ok ? b.w : 0.f;
    }
    __syncthreads();     // the buffer is written again when the wavefronts' slices are joined
  }
  float sn = 0.f, c = 1.f;                   // lane j < HD / 2: angle j of position p
  if (has_keys && lane < HD / 2) sincos_angle(angle, &sn, &c);

  // ---- the new key and value go into the cache, written by the wavefront that reads them
  if (writes) {
    const int page = pt[p >> HE_PAGE_SHIFT];
    if (page >= 0 && page < num_pages) {
      const int off = p & (HE_PAGE_TOKENS - 1);
      const int half = rotary_dim >> 1;
      const int k_col = H * HD + kvh * HD, v_col = (H + KVH) * HD + kvh * HD;
      // the page in operand order (cache_layout.h)
      uint16_t* kpage = kpool + ((int64_t)page * KVH + kvh) * he_k_page_elems(HD);
      uint16_t* vpage = vpool + ((int64_t)page * KVH + kvh) * he_v_page_elems(HD);
      // SLICED: the slices of this lane's two key values and (up to) two value values, all loads
      // issued before the first sum (one after the other they were four round trips on the path the
      // launch waits for)
      float k_sl[2] = {0.f, 0.f}, v_sl[2] = {0.f, 0.f};
      if (SLICED) {
        const float* at[4] = {part_row + k_col + min(lane, half - 1), part_row + k_col + min(lane, half - 1) + half,
                              part_row + v_col + min(lane, HD - 1), part_row + v_col + min(lane + 64, HD - 1)};
        if (qkv_slices <= 8) {
          float got[4][8];
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 8; ++j) got[q][j] = at[q][(int64_t)min(j, qkv_slices - 1) * slice_stride];
          float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (j < qkv_slices)
#pragma unroll
              for (int q = 0; q < 4; ++q) sum[q] += got[q][j];
          k_sl[0] = as_bf16(sum[0]), k_sl[1] = as_bf16(sum[1]), v_sl[0] = as_bf16(sum[2]), v_sl[1] = as_bf16(sum[3]);
        } else {
          k_sl[0] = as_bf16(slices_sum<float>(at[0], qkv_slices, slice_stride));
          k_sl[1] = as_bf16(slices_sum<float>(at[1], qkv_slices, slice_stride));
          v_sl[0] = as_bf16(slices_sum<float>(at[2], qkv_slices, slice_stride));
          v_sl[1] = as_bf16(slices_sum<float>(at[3], qkv_slices, slice_stride));
        }
      }
      if (lane < half) {                     // half <= 64: one pair per lane
        const int j = lane;
        float x0 = SLICED ? k_sl[0] : bf16_bits_to_float(qkv_row[k_col + j]);
        float x1 = SLICED ? k_sl[1] : bf16_bits_to_float(qkv_row[k_col + j + half]);
        if (bias) {
          x0 += load_param(bias, k_col + j, bias_dtype);
          x1 += load_param(bias, k_col + j + half, bias_dtype);
        }
        kpage[he_k_index(off, j, KS)] = float_to_bf16_bits(fmaf(x0, c, -(x1 * sn)));
        kpage[he_k_index(off, j + half, KS)] = float_to_bf16_bits(fmaf(x0, sn, x1 * c));
      }
      for (int d = lane; d < HD; d += 64) {
        float x = SLICED ? (d >= 64 ? v_sl[1] : v_sl[0]) : bf16_bits_to_float(qkv_row[v_col + d]);
        if (bias) x += load_param(bias, v_col + d, bias_dtype);
        vpage[he_v_index(off, d, NT)] = float_to_bf16_bits(x);
      }
    }
    __threadfence_block();   // this wavefront reads the row back below
  }

  AttnState<NT> st;
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) st.o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  st.m = -INFINITY;
  st.l = 0.f;
  if (has_keys) {
    bf16x8 qf[KS];
    rotate_q<NT>(qf, qx, lg, sn, c);
    if (!early) attend_start<NT>(cursor, kpool, vpool, pt, max_blocks, num_pages, KVH, kvh, kb_begin, lr, lg);
    attend_walk<NT, false>(st, qf, cursor, pt, max_blocks, num_pages, kb_begin, (kb_end + 31) & ~31,
                           first, p, first, p, scale * 1.4426950408889634f, lr, lg);
  }
  float l = st.l;
  l = xor32_sum(xor16_sum(l));

  // ---- join the slices through LDS, in wavefront order
  float* lds_o = lds;
  float* lds_ml = lds + (int64_t)nw * GT * HD;
  if (h_ok) {
    float* o = lds_o + ((int64_t)wave * GT + lr) * HD;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt)
      *reinterpret_cast<float4*>(o + 16 * dt + 4 * lg) =
          make_float4(st.o[dt][0], st.o[dt][1], st.o[dt][2], st.o[dt][3]);
    if (lg == 0) {
      lds_ml[2 * (wave * GT + lr)] = st.m;
      lds_ml[2 * (wave * GT + lr) + 1] = l;
    }
  }
  __syncthreads();
  for (int item = threadIdx.x; item < GT * (HD / 4); item += blockDim.x) {
    const int hg = item / (HD / 4), d = 4 * (item % (HD / 4));
    float M = -INFINITY;
    for (int w = 0; w < nw; ++w) M = fmaxf(M, lds_ml[2 * (w * GT + hg)]);
    float L = 0.f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int w = 0; w < nw; ++w) {
      const float m = lds_ml[2 * (w * GT + hg)];
      if (!(m > -INFINITY)) continue;
      const float wgt = __builtin_amdgcn_exp2f(m - M);
      L += lds_ml[2 * (w * GT + hg) + 1] * wgt;
      const float4 v = *reinterpret_cast<const float4*>(lds_o + ((int64_t)w * GT + hg) * HD + d);
      acc.x += v.x * wgt;
      acc.y += v.y * wgt;
      acc.z += v.z * wgt;
      acc.w += v.w * wgt;
    }
    const int64_t head = (int64_t)row * H + kvh * G + 16 * ht + hg;
    if (Z == 1) {
      const float inv = L > 0.f ? 1.f / L : 0.f;
      uint2 w2;
      w2.x = pack2_bf16(acc.x * inv, acc.y * inv);
      w2.y = pack2_bf16(acc.z * inv, acc.w * inv);
      *reinterpret_cast<uint2*>(out_at(hg, d)) = w2;
    } else {                               // a part without keys stores (-inf, 0, zeros)
      *reinterpret_cast<float4*>(ws_o + (head * Z + z) * HD + d) = acc;
      if (d == 0) {
        ws_ml[2 * (head * Z + z)] = M;
        ws_ml[2 * (head * Z + z) + 1] = L;
      }
    }
  }
  asm volatile("" :: "v"(touched));
}

// Wavefronts per workgroup and workgroups per (sequence, kv head, head tile), measured on
// MI355X at 4 kv heads of 128 from 1 to 64 sequences and 500 to 8000 keys: with 256 or more
// (sequence, kv head) pairs one workgroup of 8 wavefronts each and no second launch; below,
// 4 wavefronts and as many workgroups per pair as bring the grid to about 256 (one per
// compute unit; at 32 sequences that is 41 us against 52 us for one workgroup per pair), at
// most 16 (32 for contexts beyond 16384), while a slice keeps 64 keys at max_keys.
// spread: the caller knows that one sequence has several times the keys of the others; the
// grid above would leave that sequence to a few workgroups (64 sequences, two of them with
// 30000 keys and the others with 500: 279 us, with 8 workgroups per pair 102; 32 sequences
// 186 -> 87; 8 sequences, one long, 56 -> 47 with 16): twice as many workgroups per pair,
// 8 to 16. A short sequence's spare workgroups find no keys and leave empty parts.
static void fused_shape(int rows, int H, int KVH, int hd, int max_keys, int spread, int* nw, int* Z) {
  const int G = H / KVH;
  const int gt = G < 16 ? G : 16;
  const int groups = rows * KVH * ((G + 15) / 16);
  int w = (int64_t)8 * gt * (hd + 2) * 4 <= 65536 ? 8 : 4, zz = 1;
  const int cus = he_cus();
  if (groups < cus) {
    w = 4;
    zz = (cus + groups - 1) / groups;
    const int cap = max_keys > 16384 ? 32 : 16;
    if (zz > cap) zz = cap;
    const int most = (max_keys + 4 * FUSED_MIN_CHUNK - 1) / (4 * FUSED_MIN_CHUNK);
    if (zz > most) zz = most;
    if (zz < 1) zz = 1;
  }
  if (spread) {
    const int most = (max_keys + 4 * FUSED_MIN_CHUNK - 1) / (4 * FUSED_MIN_CHUNK);
    int sz = 2 * zz < 8 ? 8 : 2 * zz > 16 ? (zz > 16 ? zz : 16) : 2 * zz;
    if (sz > most) sz = most;
    if (sz > zz) zz = sz, w = 4;
  }
  *nw = w;
  *Z = zz;
}

// Whether the fused kernel takes these sizes (otherwise the caller runs the separate
// q/k/v, attention and merge kernels).
extern "C" int he_attention_decode_fused_ok(int H, int KVH, int hd, int rotary_dim) {
  if (H <= 0 || KVH <= 0 || H % KVH) return 0;
  if (hd != 64 && hd != 128) return 0;   // registers: the fragments of two steps are in flight
  return rotary_dim == hd;
}

extern "C" int64_t he_attention_decode_fused_workspace_floats(int rows, int H, int KVH, int hd,
                                                              int max_keys, int spread) {
  if (rows <= 0 || !he_attention_decode_fused_ok(H, KVH, hd, hd) || max_keys <= 0) return 0;
  int nw, Z;
  fused_shape(rows, H, KVH, hd, max_keys, spread, &nw, &Z);
  return Z == 1 ? 0 : (int64_t)rows * H * Z * (hd + 2);
}

extern "C" int he_attention_decode_fused_bf16(void* out, const void* qkv, const void* qkv_part,
                                              int qkv_slices, int64_t qkv_slice_stride,
                                              int64_t qkv_stride,
                                              const void* bias, int bias_dtype, void* kpool,
                                              void* vpool, const void* positions,
                                              const void* row_seq, const void* seq_slot,
                                              const void* page_table, int max_blocks,
                                              int num_pages, const void* inv_freq, int rotary_dim,
                                              int rows, int H, int KVH, int hd, int window,
                                              float scale, int max_keys, int spread, int write_kv,
                                              int out_pieces, void* workspace_f32,
                                              int64_t workspace_floats, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && KVH > 0 && hd > 0 && max_keys > 0,
             "he_attention_decode_fused_bf16: bad sizes");
  HE_REQUIRE(scale > 0.f, "he_attention_decode_fused_bf16: the score scale must be positive");
  HE_REQUIRE(he_attention_decode_fused_ok(H, KVH, hd, rotary_dim),
             "he_attention_decode_fused_bf16: sizes H=%d KVH=%d head_dim=%d rotary_dim=%d are not "
             "taken (head_dim 64 or 128, rotated whole)", H, KVH, hd, rotary_dim);
  HE_REQUIRE(rows <= 65535, "he_attention_decode_fused_bf16: %d rows above 65535", rows);
  HE_REQUIRE((qkv != nullptr) != (qkv_part != nullptr),
             "he_attention_decode_fused_bf16: the projection rows come as bfloat16 rows or as K slices, one of the two");
  HE_REQUIRE(qkv_part == nullptr || (qkv_slices >= 1 && qkv_slices <= 64 && (((uintptr_t)qkv_part) & 15) == 0 &&
                                     qkv_slice_stride >= (int64_t)rows * qkv_stride && (qkv_slice_stride & 3) == 0),
             "he_attention_decode_fused_bf16: %d K slices (1 to 64) of %lld elements each, 16-byte aligned, for %d rows of %lld",
             qkv_slices, (long long)qkv_slice_stride, rows, (long long)qkv_stride);
  HE_REQUIRE((qkv_stride & 7) == 0 && (((uintptr_t)qkv) & 15) == 0 &&
                 (((uintptr_t)kpool) & 15) == 0 && (((uintptr_t)vpool) & 15) == 0 &&
                 (((uintptr_t)out) & 7) == 0,
             "he_attention_decode_fused_bf16: buffers must be 16-byte aligned");
  HE_REQUIRE(inv_freq != nullptr, "he_attention_decode_fused_bf16: missing inv_freq");
  if (rows == 0) return 0;
  const int G = H / KVH;
  const int head_tiles = (G + 15) / 16;
  const int gt = G < 16 ? G : 16;
  int nw, Z;
  fused_shape(rows, H, KVH, hd, max_keys, spread, &nw, &Z);
  const int64_t need = Z == 1 ? 0 : (int64_t)rows * H * Z * (hd + 2);
  HE_REQUIRE(Z == 1 || (workspace_f32 != nullptr && workspace_floats >= need &&
                        (((uintptr_t)workspace_f32) & 15) == 0),
             "he_attention_decode_fused_bf16: workspace of %lld floats, need %lld (16-byte aligned)",
             (long long)workspace_floats, (long long)need);
  float* ws_o = (float*)workspace_f32;
  float* ws_ml = ws_o ? ws_o + (int64_t)rows * H * Z * hd : nullptr;
  const size_t lds = (size_t)nw * gt * (hd + 2) * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(KVH * head_tiles, rows, Z);
#define FUSED_LAUNCH(NTV, SL)                                                                   \
    attention_decode_fused_kernel<NTV, SL><<<grid, 64 * nw, lds, s>>>(                          \
        (uint16_t*)out, ws_o, ws_ml, (const uint16_t*)qkv, (const float*)qkv_part, qkv_slices,  \
        qkv_slice_stride, qkv_stride, bias, bias_dtype,                                         \
        (uint16_t*)kpool,                                                                       \
        (uint16_t*)vpool, (const int32_t*)positions, (const int32_t*)row_seq,                   \
        (const int32_t*)seq_slot, (const int32_t*)page_table, max_blocks, num_pages,            \
        (const float*)inv_freq, rotary_dim, H, KVH, head_tiles, window, scale, write_kv,        \
        out_pieces)
#define FUSED(NTV)                                                                              \
  case NTV:                                                                                     \
    if (qkv_part != nullptr) FUSED_LAUNCH(NTV, true); else FUSED_LAUNCH(NTV, false);            \
    break;
  switch (hd / 16) {
    FUSED(4) FUSED(8)
    default:
      HE_REQUIRE(false, "he_attention_decode_fused_bf16: head_dim %d", hd);
  }
#undef FUSED
#undef FUSED_LAUNCH
  const int rc = he_check_launch("he_attention_decode_fused_bf16");
  if (rc || Z == 1) return rc;
  return he_attention_merge_parts(out, ws_o, ws_ml, row_seq, rows, H, hd, Z, out_pieces, stream);
}
