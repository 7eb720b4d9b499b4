// Device code shared by the MFMA attention kernels: the operand fragments of one step
// of 32 keys, the online-softmax state of 16 queries (one per column), and the loop that
// walks a key range one step ahead with its loads. The layout notes are in
// attention_mfma.hip.
#pragma once
#include "cache_layout.h"

// Online softmax keeps, per query, a reference point m (base-2 domain) and sums of
// 2^(s - m). Any m gives the same quotient; m need only be close enough to the running
// maximum that 2^(s - m) stays small. Following the maximum exactly makes one of the 16
// queries of a tile move it in most steps, and every move rescales all accumulators.
#define HE_SOFTMAX_SLACK 8.0f

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 ld8(const uint16_t* p, bool ok) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if (ok) v = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, v);
}

template <int NT>
struct AttnState {
  floatx4 o[NT];  // O^T[16*dt + 4*lg + i][q], unnormalised
  float m;        // reference point (near the running maximum) of the query of this lane's column
  float l;        // this lane's share of the running sum
};

// The K and V^T operands of one step of 32 keys, loaded ahead of their use so that the
// loads of step i+1 are in flight while step i computes.
template <int NT>
struct KVFrag {
  bf16x8 k[2][(16 * NT + 31) / 32];
  bf16x8 v[NT];
  int ok;   // the page exists (always, for an admitted batch)
};

// kpool/vpool of this kv head; page: physical page of the 32 keys; koff: 0 or 32. The pages
// are stored in operand order (cache_layout.h): every load below is one contiguous KiB.
template <int NT>
__device__ __forceinline__ void load_frag(KVFrag<NT>& f, const uint16_t* __restrict__ kpool,
                                          const uint16_t* __restrict__ vpool, int page,
                                          int num_pages, int64_t k_page_stride,
                                          int64_t v_page_stride, int koff, int lr, int lg) {
  constexpr int HD = 16 * NT;
  constexpr int KS = (HD + 31) / 32;
  f.ok = page >= 0 && page < num_pages;
  const int lane = 16 * lg + lr, h = koff >> 5;
  const uint16_t* kpage = kpool + (int64_t)(f.ok ? page : 0) * k_page_stride + ((h * 2) * KS * 64 + lane) * 8;
  const uint16_t* vpage = vpool + (int64_t)(f.ok ? page : 0) * v_page_stride + (h * NT * 64 + lane) * 8;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      f.k[t][ks] = ld8(kpage + (t * KS + ks) * 512, 32 * ks + 8 * lg < HD);
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) f.v[dt] = ld8(vpage + dt * 512, true);
}

// One step of 32 keys starting at absolute position key_base (a multiple of 32).
// The lane's query sees the keys in [lo, hi]; with MASK false the caller has checked
// that all 32 keys are visible to every query of the tile. Scores are kept in the
// base-2 domain: s2 = (q . k) * scale * log2(e), p = 2^(s2 - m), so the exponential is
// the bare hardware instruction; m is the reference point of s2 (see HE_SOFTMAX_SLACK). When
// no query's reference point moves, the rescaling of the accumulators is skipped.
template <int NT, bool MASK>
__device__ __forceinline__ void attend_frag(AttnState<NT>& st, const bf16x8* qf,
                                            const KVFrag<NT>& f, int key_base, int lo, int hi,
                                            float scale_log2, int lg) {
  constexpr int HD = 16 * NT;
  constexpr int KS = (HD + 31) / 32;
  if (MASK && !f.ok) hi = -1;
  floatx4 s[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[t][ks], qf[ks], s[t], 0, 0, 0);
  }
  // raw scores (masked ones at -inf), their maximum, then p = 2^(raw * scale - m) with the
  // scale folded into the subtraction (scale > 0, so the maximum commutes with it)
  float p[2][4];
  float mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = s[t][r];
      if (MASK) {
        const int key = key_base + 8 * lg + 4 * t + r;
        v = (key >= lo && key <= hi) ? v : -INFINITY;
      }
      p[t][r] = v;
      mx = fmaxf(mx, v);
    }
  mx = xor32_max(xor16_max(mx)) * scale_log2;
  // the reference point follows the maximum only when that has grown by more than
  // 2^HE_SOFTMAX_SLACK: p stays below that factor, and the accumulators are rarely rescaled
  const float m_new = mx > st.m + HE_SOFTMAX_SLACK ? mx : st.m;
  const bool moved = __builtin_amdgcn_ballot_w64(m_new != st.m) != 0;   // wave-uniform
  const float m_use = m_new == -INFINITY ? 0.f : m_new;
  float sum = 0.f;
  uint32_t packed[4];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 4; r += 2) {
      const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(p[t][r], scale_log2, -m_use));
      const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(p[t][r + 1], scale_log2, -m_use));
      sum += e0 + e1;
      packed[2 * t + (r >> 1)] = pack2_bf16(e0, e1);
    }
  if (moved) {
    const float alpha = __builtin_amdgcn_exp2f(st.m - m_use);
    st.l = st.l * alpha + sum;
    st.m = m_new;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) st.o[dt] *= alpha;
  } else {
    st.l += sum;
  }
  const bf16x8 pb =
      __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
#pragma unroll
  for (int dt = 0; dt < NT; ++dt)
    st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.v[dt], pb, st.o[dt], 0, 0, 0);
}

// Runs the steps kb = kb_begin, kb_begin + 32, ... < kb_end (all multiples of 32) of one
// (sequence, kv head) against the state, one step ahead with its loads and one page
// ahead with its page-table entry.
// Where a walk over the keys stands: the page of the current step, the entry of the page
// after it, and the fragments of the step to come, already on their way.
template <int NT>
struct AttendCursor {
  const uint16_t* kp;
  const uint16_t* vp;
  int64_t k_stride, v_stride;
  int block, page, page_ahead;
  KVFrag<NT> cur;
};

// Starts the walk at key kb_begin (a multiple of 32) in two parts, so that a caller can put
// work between them: attend_pages asks for the page-table entries, attend_first issues the loads
// of the first step. A caller with other work to do (a query to rotate) does it between
// attend_first and attend_walk, while the fragments are on their way.
template <int NT>
__device__ __forceinline__ void attend_pages(AttendCursor<NT>& c, const int32_t* __restrict__ pt,
                                             int max_blocks, int kb_begin) {
  c.block = kb_begin >> HE_PAGE_SHIFT;
  c.page = pt[c.block];
  c.page_ahead = pt[min(c.block + 1, max_blocks - 1)];
}

template <int NT>
__device__ __forceinline__ void attend_first(AttendCursor<NT>& c, const uint16_t* __restrict__ kpool,
                                             const uint16_t* __restrict__ vpool, int num_pages, int KVH,
                                             int kvh, int kb_begin, int lr, int lg) {
  constexpr int HD = 16 * NT;
  c.k_stride = (int64_t)KVH * he_k_page_elems(HD);
  c.v_stride = (int64_t)KVH * he_v_page_elems(HD);
  c.kp = kpool + (int64_t)kvh * he_k_page_elems(HD);
  c.vp = vpool + (int64_t)kvh * he_v_page_elems(HD);
  load_frag<NT>(c.cur, c.kp, c.vp, c.page, num_pages, c.k_stride, c.v_stride, kb_begin & 32, lr, lg);
}

template <int NT>
__device__ __forceinline__ void attend_start(AttendCursor<NT>& c, const uint16_t* __restrict__ kpool,
                                             const uint16_t* __restrict__ vpool,
                                             const int32_t* __restrict__ pt, int max_blocks,
                                             int num_pages, int KVH, int kvh, int kb_begin, int lr,
                                             int lg) {
  attend_pages<NT>(c, pt, max_blocks, kb_begin);
  attend_first<NT>(c, kpool, vpool, num_pages, KVH, kvh, kb_begin, lr, lg);
}

// Runs the keys [kb_begin, kb_end) (multiples of 32) of one (sequence, kv head) against the
// state, one step ahead with its loads and one page ahead with its page-table entry.
template <int NT, bool UNMASKED_STEPS>
__device__ __forceinline__ void attend_walk(AttnState<NT>& st, const bf16x8* qf, AttendCursor<NT>& c,
                                            const int32_t* __restrict__ pt, int max_blocks,
                                            int num_pages, int kb_begin, int kb_end, int lo, int hi,
                                            int clear_lo, int clear_hi, float scale_log2, int lr,
                                            int lg) {
  KVFrag<NT> nxt;
  for (int kb = kb_begin; kb < kb_end; kb += 32) {
    const int kn = kb + 32;
    if (kn < kb_end) {
      if ((kn & 32) == 0) {   // the next step starts a new page
        ++c.block;
        c.page = c.page_ahead;
        c.page_ahead = pt[min(c.block + 1, max_blocks - 1)];
      }
      load_frag<NT>(nxt, c.kp, c.vp, c.page, num_pages, c.k_stride, c.v_stride, kn & 32, lr, lg);
    }
    // keys in [clear_lo, clear_hi] are visible to every query of the tile
    if (UNMASKED_STEPS && kb >= clear_lo && kb + 31 <= clear_hi && c.cur.ok)
      attend_frag<NT, false>(st, qf, c.cur, kb, lo, hi, scale_log2, lg);
    else
      attend_frag<NT, true>(st, qf, c.cur, kb, lo, hi, scale_log2, lg);
    c.cur = nxt;
  }
}

template <int NT, bool UNMASKED_STEPS>
__device__ __forceinline__ void attend_range(AttnState<NT>& st, const bf16x8* qf,
                                             const uint16_t* __restrict__ kpool,
                                             const uint16_t* __restrict__ vpool,
                                             const int32_t* __restrict__ pt, int max_blocks,
                                             int num_pages, int KVH, int kvh, int kb_begin,
                                             int kb_end, int lo, int hi, int clear_lo,
                                             int clear_hi, float scale_log2, int lr, int lg) {
  if (kb_begin >= kb_end) return;
  AttendCursor<NT> c;
  attend_start<NT>(c, kpool, vpool, pt, max_blocks, num_pages, KVH, kvh, kb_begin, lr, lg);
  attend_walk<NT, UNMASKED_STEPS>(st, qf, c, pt, max_blocks, num_pages, kb_begin, kb_end, lo, hi,
                                  clear_lo, clear_hi, scale_log2, lr, lg);
}

template <int NT>
__device__ __forceinline__ void load_q(bf16x8* qf, const uint16_t* qrow, bool valid, int lg) {
  constexpr int HD = 16 * NT;
  constexpr int KS = (HD + 31) / 32;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    // no branch around the load (qrow is a row that may be read, whether or not the lane's query
    // or head counts; a piece beyond the head reads the head's start): the loads of a tile go
    // out together, and what does not count becomes zero
    const int d = 32 * ks + 8 * lg;
    const uint4 v = *reinterpret_cast<const uint4*>(qrow + (d < HD ? d : 0));
    qf[ks] = __builtin_bit_cast(bf16x8, (valid && d < HD) ? v : make_uint4(0, 0, 0, 0));
  }
}

