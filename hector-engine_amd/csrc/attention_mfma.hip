// bf16 attention over the paged cache on the matrix cores, for prompt steps
// (tiles of 16 queries of one sequence and head) and for one-token steps (the
// query heads of one kv group, the keys split over workgroups and merged).
// They replace the reference's attention_prefill_cached_kernel
// (kernels/attention.cu:664-773: one block per query and head, no tile reuse)
// and attention_cached_v2_kernel_dp (kernels/attention.cu:337-494); the
// online-softmax algebra and its merge are the reference's
// (kernels/attention.cu:279-314).
//
// Both kernels work on transposed tiles so that no operand ever has to change
// lanes. With v_mfma_f32_16x16x32_bf16 (A: lane l holds A[l%16][8*(l/16)..+8),
// B: lane l holds B[8*(l/16)..+8)[l%16], D: lane l holds D[4*(l/16)+i][l%16]):
//   S^T[key][q] = sum_d K[key][d] Q[q][d]      A = K rows (d contiguous), B = Q rows
//   O^T[d][q]   = sum_key V^T[d][key] P^T[key][q]   A = V^T rows, B = P^T
// The cache stores V transposed inside a page, [head_dim][64 tokens], so a V^T
// row's 8 consecutive keys are 16 contiguous bytes. The 32 keys of a step are
// assigned to the rows of the two S^T tiles as key = 8*(row/4) + 4*tile + row%4,
// which leaves lane group g with exactly the keys 8g..8g+7 that the B operand of
// the P^T V product wants from it. A query is a column (l%16), so its softmax
// statistics are reduced over registers and two lane swaps (xor 16, 32) only.
// Softmax, its running maximum and sum, and both accumulators are fp32.
// The prompt kernel here reads its operands from global memory; head sizes up to 128 and
// prompts of more than 16 tokens go to the kernel in attention_prefill_wide.hip, which shares
// pages through LDS (he_attention_prefill_bf16 chooses).
#include "common.h"
#include "hector_kernels.h"

#include "attention_tiles.h"

// ------------------------------------------------------------------ prefill
// grid (ceil(max_q_len / 64), H, num_seqs), 256 threads: wave w takes the 16
// queries q0 = 64*blockIdx.x + 16*w of the sequence.
template <int NT>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q,
    const uint16_t* __restrict__ kpool, const uint16_t* __restrict__ vpool,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ seq_start, const int32_t* __restrict__ page_table, int max_blocks,
    int num_pages, int H, int KVH, int window, float scale) {
  constexpr int HD = 16 * NT;
  constexpr int KS = (HD + 31) / 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int seq = blockIdx.z, h = blockIdx.y;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int row0 = cu_seqlens[seq];
  const int q_len = cu_seqlens[seq + 1] - row0;
  const int q0 = 64 * blockIdx.x + 16 * wave;
  if (q0 >= q_len) return;
  const int start = seq_start[seq];
  const int kvh = h / (H / KVH);
  const int32_t* pt = page_table + (int64_t)slot * max_blocks;

  const int qi = q0 + lr;                 // this lane's query (column)
  const bool q_ok = qi < q_len;
  const int pos = start + qi;             // its absolute position
  const int hi = q_ok ? pos : -1;
  const int lo = (window > 0 && q_ok) ? max(0, pos + 1 - window) : 0;
  bf16x8 qf[KS];
  load_q<NT>(qf, q + ((int64_t)(row0 + max(0, min(qi, q_len - 1))) * H + h) * HD, q_ok, lg);

  AttnState<NT> st;
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) st.o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  st.m = -INFINITY;
  st.l = 0.f;

  const int last_pos = start + min(q0 + 15, q_len - 1);
  const int first_pos = start + q0;
  const int tile_lo = window > 0 ? max(0, first_pos + 1 - window) : 0;
  // every query of a full tile sees the keys from the last query's window start to the
  // first query's position
  const bool full_tile = q0 + 15 < q_len;
  const int clear_lo = window > 0 ? max(0, last_pos + 1 - window) : 0;
  const int clear_hi = full_tile ? first_pos : -1;
  attend_range<NT, true>(st, qf, kpool, vpool, pt, max_blocks, num_pages, KVH, kvh, tile_lo & ~31,
                   (last_pos & ~31) + 32, lo, hi, clear_lo, clear_hi, scale * 1.4426950408889634f,
                   lr, lg);
  float l = st.l;
  l = xor32_sum(xor16_sum(l));
  if (!q_ok) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  uint16_t* orow = out + ((int64_t)(row0 + qi) * H + h) * HD;
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) {
    uint2 w;
    w.x = pack2_bf16(st.o[dt][0] * inv, st.o[dt][1] * inv);
    w.y = pack2_bf16(st.o[dt][2] * inv, st.o[dt][3] * inv);
    *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * lg) = w;
  }
}

// ------------------------------------------------------------------ decode
// grid (nsplit, KVH * head_tiles, rows), 64 threads. Columns are the query heads
// of one kv group (16 per head tile). The keys of a sequence are cut into slices
// of at least DECODE_MIN_CHUNK keys, at most nsplit of them; each workgroup takes
// one slice and writes (m, l, unnormalised O) for its heads; the merge kernel
// joins the slices in the order of their index:
//   out = sum_s O_s e^(m_s - M) / sum_s l_s e^(m_s - M)
// With a single slice in the grid the result is written directly.
#define DECODE_MIN_CHUNK 64

template <int NT>
__global__ __launch_bounds__(64) void attention_decode_kernel(
    uint16_t* __restrict__ out, float* __restrict__ ws_o, float* __restrict__ ws_ml,
    const uint16_t* __restrict__ q,
    const uint16_t* __restrict__ kpool, const uint16_t* __restrict__ vpool,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ page_table, int max_blocks,
    int num_pages, int H, int KVH, int head_tiles, int window, float scale) {
  constexpr int HD = 16 * NT;
  constexpr int KS = (HD + 31) / 32;
  const int lane = threadIdx.x;
  const int lr = lane & 15, lg = lane >> 4;
  const int split = blockIdx.x, nsplit = gridDim.x;
  const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y % head_tiles;
  const int row = blockIdx.z;
  const int G = H / KVH;
  const int hg = 16 * ht + lr;            // head within the group
  const bool h_ok = hg < G;
  const int h = kvh * G + min(hg, G - 1);
  uint16_t* orow = out + ((int64_t)row * H + h) * HD;
  const int seq = row_seq[row];
  if (seq < 0) {                          // padding row: zeros (the merge kernel writes them if there is one)
    if (nsplit == 1 && h_ok)
#pragma unroll
      for (int dt = 0; dt < NT; ++dt)
        *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * lg) = make_uint2(0u, 0u);
    return;
  }
  const int slot = seq_slot[seq];
  const int n_keys = positions[row] + 1;
  const int first = window > 0 ? max(0, n_keys - window) : 0;
  const int span_lo = first & ~31;
  int chunk = (n_keys - span_lo + nsplit - 1) / nsplit;
  chunk = max(DECODE_MIN_CHUNK, (chunk + 31) & ~31);
  const int active = (n_keys - span_lo + chunk - 1) / chunk;   // slices that hold keys
  if (split >= active) return;
  const int kb_begin = span_lo + split * chunk;
  const int kb_end = min(kb_begin + chunk, n_keys);
  const int32_t* pt = page_table + (int64_t)slot * max_blocks;
  bf16x8 qf[KS];
  load_q<NT>(qf, q + ((int64_t)row * H + h) * HD, h_ok, lg);
  AttnState<NT> st;
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) st.o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  st.m = -INFINITY;
  st.l = 0.f;
  const int hi = n_keys - 1;
  attend_range<NT, false>(st, qf, kpool, vpool, pt, max_blocks, num_pages, KVH, kvh, kb_begin,
                   (kb_end + 31) & ~31, first, hi, first, hi, scale * 1.4426950408889634f, lr, lg);
  float l = st.l;
  l = xor32_sum(xor16_sum(l));
  if (nsplit == 1) {                      // nothing to merge
    if (!h_ok) return;
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) {
      uint2 w;
      w.x = pack2_bf16(st.o[dt][0] * inv, st.o[dt][1] * inv);
      w.y = pack2_bf16(st.o[dt][2] * inv, st.o[dt][3] * inv);
      *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * lg) = w;
    }
    return;
  }
  const int64_t wbase = ((int64_t)row * H + h) * nsplit;
  if (h_ok) {
    if (lg == 0) {
      ws_ml[2 * (wbase + split)] = st.m;
      ws_ml[2 * (wbase + split) + 1] = l;
    }
    float* o = ws_o + (wbase + split) * HD;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt)
      *reinterpret_cast<float4*>(o + 16 * dt + 4 * lg) =
          make_float4(st.o[dt][0], st.o[dt][1], st.o[dt][2], st.o[dt][3]);
  }
}

// Joins the slices of one (row, head): grid (H, rows), four wavefronts; wavefront w adds
// the slices s = w, w + 4, ... and the four sums are added in wavefront order. The number
// of slices that hold keys is recomputed exactly as the decode kernel computes it.
// The launch is a chain of trips to memory and little else, so the loads that need no
// loaded value to know their address go out together at the start: the row's sequence, the
// slices' statistics and the first 32 slices' outputs (when every part was stored, that is
// all of them), and a row without a sequence is dealt with at the store.
#define MERGE_PER 8   // slices a wavefront holds at once
__global__ __launch_bounds__(256) void attention_merge_kernel(
    uint16_t* __restrict__ out, const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq, int H, int HD,
    int nsplit, int window, int all_parts, int out_pieces) {
  __shared__ float wgt[64];
  __shared__ float part[4][256];
  const int h = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = blockIdx.y;
  // where dim d of this row and head goes: row-major [rows, H HD], or piece-major (16-byte
  // pieces [H HD / 8][rows][8], the layout the next product reads best at up to 16 rows)
  auto at = [&](int d) {
    const int64_t c = (int64_t)h * HD + d;
    return out_pieces ? out + ((c >> 3) * gridDim.y + row) * 8 + (c & 7) : out + row * H * (int64_t)HD + c;
  };
  const bool live = row_seq == nullptr || row_seq[row] >= 0;
  int active = nsplit;                     // all_parts: every part was stored, empty ones as (-inf, 0, 0)
  if (!all_parts) {
    active = 0;
    if (live) {
      const int n_keys = positions[row] + 1;
      const int first = window > 0 ? max(0, n_keys - window) : 0;
      const int span_lo = first & ~31;
      int chunk = (n_keys - span_lo + nsplit - 1) / nsplit;
      chunk = max(DECODE_MIN_CHUNK, (chunk + 31) & ~31);
      active = (n_keys - span_lo + chunk - 1) / chunk;
    }
  }
  const int64_t base = (row * H + h) * nsplit;
  // outputs of the slices s0 + wave + 4 i at the dims d0 + lane + 64 j; what does not exist reads as 0
  auto load_slices = [&](float (&ov)[MERGE_PER][4], int d0, int s0) {
#pragma unroll
    for (int i = 0; i < MERGE_PER; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int s = s0 + wave + 4 * i, d = d0 + lane + 64 * j;
        ov[i][j] = s < active && d < HD ? ws_o[(base + s) * HD + d] : 0.f;
      }
  };
  const float m = lane < active ? ws_ml[2 * (base + lane)] : -INFINITY;
  const float l = lane < active ? ws_ml[2 * (base + lane) + 1] : 0.f;
  float ov[MERGE_PER][4];
  load_slices(ov, 0, 0);
  const float M = wave_max(m);
  const float w = m > -INFINITY ? __builtin_amdgcn_exp2f(m - M) : 0.f;   // m is in the base-2 domain
  const float L = wave_sum(l * w);          // every wavefront computes the same weights
  if (wave == 0) wgt[lane] = w;             // 0 from `active` on
  __syncthreads();
  const float inv = L > 0.f ? 1.f / L : 0.f;
  for (int d0 = 0; d0 < HD; d0 += 256) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < active; s0 += 4 * MERGE_PER) {
      if (d0 + s0 > 0) load_slices(ov, d0, s0);
#pragma unroll
      for (int i = 0; i < MERGE_PER; ++i) {
        const int s = s0 + wave + 4 * i;
        const float ws = s < active ? wgt[s] : 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] += ov[i][j] * ws;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) part[wave][lane + 64 * j] = acc[j];
    __syncthreads();
    const int d = d0 + threadIdx.x;
    if (d < HD) {
      const float sum = ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) +
                        part[3][threadIdx.x];
      *at(d) = live ? float_to_bf16_bits(sum * inv) : (uint16_t)0;
    }
    __syncthreads();
  }
}

static int decode_splits(int rows, int KVH, int head_tiles, int max_keys) {
  const int groups = rows * KVH * head_tiles;
  int s = (4096 + groups - 1) / groups;
  const int max_s = (max_keys + DECODE_MIN_CHUNK - 1) / DECODE_MIN_CHUNK;
  if (s > max_s) s = max_s;
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return s;
}

extern "C" int64_t he_attention_decode_workspace_floats(int rows, int H, int KVH, int hd,
                                                        int max_keys) {
  if (rows <= 0 || H <= 0 || KVH <= 0 || hd <= 0 || H % KVH) return 0;
  const int head_tiles = (H / KVH + 15) / 16;
  return (int64_t)rows * H * decode_splits(rows, KVH, head_tiles, max_keys) * (hd + 2);
}

#define ATTN_DISPATCH(NTV, CALL) \
  case NTV: {                    \
    constexpr int NT = NTV;      \
    CALL;                        \
    break;                       \
  }
#define ATTN_SWITCH(nt, CALL)                                                              \
  switch (nt) {                                                                            \
    ATTN_DISPATCH(1, CALL) ATTN_DISPATCH(2, CALL) ATTN_DISPATCH(3, CALL)                   \
    ATTN_DISPATCH(4, CALL) ATTN_DISPATCH(5, CALL) ATTN_DISPATCH(6, CALL)                   \
    ATTN_DISPATCH(7, CALL) ATTN_DISPATCH(8, CALL) ATTN_DISPATCH(9, CALL)                   \
    ATTN_DISPATCH(10, CALL) ATTN_DISPATCH(11, CALL) ATTN_DISPATCH(12, CALL)                \
    ATTN_DISPATCH(13, CALL) ATTN_DISPATCH(14, CALL) ATTN_DISPATCH(15, CALL)                \
    ATTN_DISPATCH(16, CALL)                                                                \
    default:                                                                               \
      he_set_error("attention: head_dim %d is not a multiple of 16 up to 256", 16 * (nt)); \
      return -1;                                                                           \
  }

extern "C" int he_attention_decode_bf16(void* out, const void* q, const void* kpool,
                                        const void* vpool, const void* positions,
                                        const void* row_seq, const void* seq_slot,
                                        const void* page_table, int max_blocks, int num_pages,
                                        int rows, int H, int KVH, int hd, int window, float scale,
                                        int max_keys, void* workspace_f32,
                                        int64_t workspace_floats, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && KVH > 0 && hd > 0 && max_keys > 0,
             "he_attention_decode_bf16: bad sizes");
  HE_REQUIRE(scale > 0.f, "he_attention_decode_bf16: the score scale must be positive");
  HE_REQUIRE(H % KVH == 0, "he_attention_decode_bf16: heads %d not a multiple of kv heads %d", H,
             KVH);
  HE_REQUIRE(hd % 16 == 0 && hd <= 256,
             "he_attention_decode_bf16: head_dim %d must be a multiple of 16 up to 256", hd);
  HE_REQUIRE(rows <= 65535, "he_attention_decode_bf16: %d rows above 65535", rows);
  if (rows == 0) return 0;
  const int G = H / KVH;
  const int head_tiles = (G + 15) / 16;
  const int nsplit = decode_splits(rows, KVH, head_tiles, max_keys);
  const int64_t need = (int64_t)rows * H * nsplit * (hd + 2);
  HE_REQUIRE(workspace_f32 != nullptr && workspace_floats >= need,
             "he_attention_decode_bf16: workspace of %lld floats, need %lld",
             (long long)workspace_floats, (long long)need);
  HE_REQUIRE((((uintptr_t)workspace_f32) & 15) == 0 && (((uintptr_t)q) & 15) == 0 &&
                 (((uintptr_t)kpool) & 15) == 0 && (((uintptr_t)vpool) & 15) == 0 &&
                 (((uintptr_t)out) & 7) == 0,
             "he_attention_decode_bf16: buffers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  float* ws_o = (float*)workspace_f32;
  float* ws_ml = ws_o + (int64_t)rows * H * nsplit * hd;
  dim3 grid(nsplit, KVH * head_tiles, rows);
  ATTN_SWITCH(hd / 16, (attention_decode_kernel<NT><<<grid, 64, 0, s>>>(
                           (uint16_t*)out, ws_o, ws_ml, (const uint16_t*)q,
                           (const uint16_t*)kpool, (const uint16_t*)vpool,
                           (const int32_t*)positions, (const int32_t*)row_seq,
                           (const int32_t*)seq_slot, (const int32_t*)page_table, max_blocks,
                           num_pages, H, KVH, head_tiles, window, scale)));
  int rc = he_check_launch("he_attention_decode_bf16");
  if (rc || nsplit == 1) return rc;
  attention_merge_kernel<<<dim3(H, rows), 256, 0, s>>>(
      (uint16_t*)out, ws_o, ws_ml, (const int32_t*)positions, (const int32_t*)row_seq, H, hd,
      nsplit, window, 0, 0);
  return he_check_launch("he_attention_decode_bf16 merge");
}

// The same join for many rows (the parts of a prompt step): one wavefront per (row, head), four
// of them a workgroup, no LDS and no barrier; a lane has the dims 2 lane, 2 lane + 1 (+ 128, ...).
// Parts are added in their order. Every part was stored; out is row-major.
__global__ __launch_bounds__(256) void attention_merge_rows_kernel(
    uint16_t* __restrict__ out, const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    int64_t pairs, int HD, int nsplit) {
  const int lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);   // row * H + h
  if (pair >= pairs) return;
  const int64_t base = pair * nsplit;
  const float2 ml = lane < nsplit ? *reinterpret_cast<const float2*>(ws_ml + 2 * (base + lane))
                                  : make_float2(-INFINITY, 0.f);
  auto load_parts = [&](float2 (&ov)[MERGE_PER], int d0, int s0) {
#pragma unroll
    for (int i = 0; i < MERGE_PER; ++i)
      ov[i] = s0 + i < nsplit && d0 < HD ? *reinterpret_cast<const float2*>(ws_o + (base + s0 + i) * HD + d0)
                                         : make_float2(0.f, 0.f);
  };
  float2 ov[MERGE_PER];
  load_parts(ov, 2 * lane, 0);   // on their way while the weights are made
  // lane s has the weight of part s (0 from nsplit on); all lanes take part in the sums
  const float M = wave_max(ml.x);
  const float w = ml.x > -INFINITY ? __builtin_amdgcn_exp2f(ml.x - M) : 0.f;   // base-2 domain
  const float L = wave_sum(ml.y * w);
  const float inv = L > 0.f ? 1.f / L : 0.f;
  for (int d0 = 2 * lane; d0 < HD; d0 += 128) {
    float2 acc = make_float2(0.f, 0.f);
    for (int s0 = 0; s0 < nsplit; s0 += MERGE_PER) {
      if (d0 >= 128 || s0 > 0) load_parts(ov, d0, s0);
#pragma unroll
      for (int i = 0; i < MERGE_PER; ++i) {
        // v_readlane: the lane is the same for all, and it need not be active
        const float w_s = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), (s0 + i) & 63));
        acc.x += ov[i].x * w_s;
        acc.y += ov[i].y * w_s;
      }
    }
    *reinterpret_cast<uint32_t*>(out + pair * HD + d0) = pack2_bf16(acc.x * inv, acc.y * inv);
  }
}

int he_attention_merge_rows(void* out, const float* ws_o, const float* ws_ml, int rows, int H, int hd,
                            int parts, void* stream) {
  HE_REQUIRE(parts >= 1 && parts <= 64 && hd % 2 == 0, "he_attention_merge_rows: %d parts (at most 64), head_dim %d", parts, hd);
  const int64_t pairs = (int64_t)rows * H;
  HE_REQUIRE((pairs + 3) / 4 < (1ll << 31), "he_attention_merge_rows: too many rows for one launch");
  if (pairs == 0) return 0;
  attention_merge_rows_kernel<<<(unsigned)((pairs + 3) / 4), 256, 0, (hipStream_t)stream>>>(
      (uint16_t*)out, ws_o, ws_ml, pairs, hd, parts);
  return he_check_launch("he_attention_merge_rows");
}

// Joins parts [rows][H][parts] of (O fp32 [hd], then (m, l) pairs) that were all stored.
int he_attention_merge_parts(void* out, const float* ws_o, const float* ws_ml, const void* row_seq,
                             int rows, int H, int hd, int parts, int out_pieces, void* stream) {
  HE_REQUIRE(parts >= 1 && parts <= 64, "he_attention_merge_parts: %d parts, at most 64", parts);
  attention_merge_kernel<<<dim3(H, rows), 256, 0, (hipStream_t)stream>>>(
      (uint16_t*)out, ws_o, ws_ml, nullptr, (const int32_t*)row_seq, H, hd, parts, 0, 1, out_pieces);
  return he_check_launch("he_attention_merge_parts");
}

// Parts the keys of a prompt step are cut into (he_attention_prefill_bf16's `parts`): a step with few
// blocks of 128 queries and many keys (a short continuation of a long sequence) would leave most of the
// chip idle, each of its workgroups walking all the pages alone. As many parts as bring the launch to two
// workgroups a compute unit, each of at least 4 pages, at most 16; none for a step whose sequences have
// fewer than four keys a query (a whole prompt has workgroups enough, and the join would cost more than the
// parts save: 2048 tokens 47 us whole, 71 in two parts). most_keys: the most keys a sequence of the step
// has (or a bound). Measured at 28 heads of 128, 4 kv heads (us without parts -> with, join included):
// 8 tokens after 8000 108 -> 18, 64 after 8000 114 -> 27, 200 after 8000 129 -> 45, 512 after 7680 130 -> 76,
// 4 x 128 after 4000 74 -> 51, 512 after 30000 457 -> 233, 1024 after 7168 144 -> 134.
extern "C" int he_attention_prefill_parts(int num_seqs, int max_q_len, int H, int hd, int most_keys) {
  if (num_seqs <= 0 || H <= 0 || hd <= 0 || hd > 128 || hd % 16 || max_q_len <= 0) return 1;
  if ((int64_t)most_keys < 4 * (int64_t)max_q_len) return 1;
  const int64_t blocks = (int64_t)((max_q_len + 127) / 128) * H * num_seqs;
  int64_t parts = 2 * he_cus() / blocks;
  const int pages = (most_keys + HE_PAGE_TOKENS - 1) / HE_PAGE_TOKENS;
  if (parts > pages / 4) parts = pages / 4;
  if (parts > 16) parts = 16;
  return parts < 1 ? 1 : (int)parts;
}

extern "C" int64_t he_attention_prefill_workspace_floats(int total_rows, int H, int hd, int parts) {
  return parts > 1 ? (int64_t)total_rows * H * parts * (hd + 2) : 0;
}

extern "C" int he_attention_prefill_bf16(void* out, const void* q, const void* kpool,
                                         const void* vpool, const void* cu_seqlens,
                                         const void* seq_slot, const void* seq_start,
                                         const void* page_table, int max_blocks, int num_pages,
                                         int num_seqs, int max_q_len, int H, int KVH, int hd,
                                         int window, float scale, int kernel, int total_rows,
                                         int parts, void* workspace_f32, int64_t workspace_floats,
                                         void* stream) {
  HE_REQUIRE(num_seqs >= 0 && max_q_len >= 0 && H > 0 && KVH > 0 && hd > 0 && total_rows >= 0,
             "he_attention_prefill_bf16: bad sizes");
  HE_REQUIRE(kernel >= 0 && kernel <= 2,
             "he_attention_prefill_bf16: kernel %d (0 = the library's choice; 1: 16 queries a wavefront, "
             "operands from global memory; 2: 32 queries a wavefront, pages shared through LDS)", kernel);
  HE_REQUIRE(kernel < 2 || hd <= 128,
             "he_attention_prefill_bf16: kernel %d needs head_dim %d <= 128", kernel, hd);
  HE_REQUIRE(scale > 0.f, "he_attention_prefill_bf16: the score scale must be positive");
  HE_REQUIRE(H % KVH == 0, "he_attention_prefill_bf16: heads %d not a multiple of kv heads %d", H,
             KVH);
  HE_REQUIRE(hd % 16 == 0 && hd <= 256,
             "he_attention_prefill_bf16: head_dim %d must be a multiple of 16 up to 256", hd);
  HE_REQUIRE(num_seqs <= 65535 && H <= 65535, "he_attention_prefill_bf16: grid too large");
  HE_REQUIRE((((uintptr_t)q) & 15) == 0 && (((uintptr_t)kpool) & 15) == 0 &&
                 (((uintptr_t)vpool) & 15) == 0 && (((uintptr_t)out) & 7) == 0,
             "he_attention_prefill_bf16: buffers must be 16-byte aligned");
  if (num_seqs == 0 || max_q_len == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (kernel == 0) kernel = hd > 128 ? 1 : 2;
  if (parts < 1) parts = 1;
  HE_REQUIRE(parts == 1 || kernel == 2,
             "he_attention_prefill_bf16: keys in %d parts are for kernel 2 (head sizes up to 128)", parts);
  if (kernel == 2) {
    float* ws_o = (float*)workspace_f32;
    float* ws_ml = ws_o + (int64_t)total_rows * H * parts * hd;
    if (parts > 1) {
      const int64_t need = he_attention_prefill_workspace_floats(total_rows, H, hd, parts);
      HE_REQUIRE(parts <= 64 && ws_o != nullptr && workspace_floats >= need && (((uintptr_t)ws_o) & 15) == 0,
                 "he_attention_prefill_bf16: %d parts (at most 64) need %lld floats of workspace (16-byte aligned), %lld given",
                 parts, (long long)need, (long long)workspace_floats);
    }
    int rc = he_attention_prefill_wide(out, q, kpool, vpool, cu_seqlens, seq_slot, seq_start, page_table,
                                       max_blocks, num_pages, num_seqs, max_q_len, H, KVH, hd, window, scale,
                                       parts, ws_o, ws_ml, stream);
    if (rc || parts == 1) return rc;
    return he_attention_merge_rows(out, ws_o, ws_ml, total_rows, H, hd, parts, stream);
  }
  dim3 grid((max_q_len + 63) / 64, H, num_seqs);
  ATTN_SWITCH(hd / 16, (attention_prefill_kernel<NT><<<grid, 256, 0, s>>>(
                           (uint16_t*)out, (const uint16_t*)q, (const uint16_t*)kpool,
                           (const uint16_t*)vpool, (const int32_t*)cu_seqlens,
                           (const int32_t*)seq_slot, (const int32_t*)seq_start,
                           (const int32_t*)page_table, max_blocks, num_pages, H, KVH, window,
                           scale)));
  return he_check_launch("he_attention_prefill_bf16");
}
