// Plain attention over the paged cache in fp32, in one fixed order per (query, head): the keys
// are taken page by page (64 positions, by absolute position), inside a page one by one in
// ascending position with an online softmax begun afresh, and the pages' results (m, l, sums)
// are joined one after the other in ascending position. The result for a query depends only on
// its own position and the cache rows [first, p], never on how the step was cut or batched, so
// prompt steps and one-token steps give identical bits. It is the 32-bit path's attention and
// the reference beside the MFMA kernels.
//
// For the query at absolute position p: first = window > 0 ? max(0, p+1-window) : 0,
// s_j = (q . k_j) * scale for j in [first, p], out = sum_j softmax(s)_j v_j,
// kv head = h / (H / KVH)   (reference: kernels/attention.cu:155-316, :664-773, :60).
//
// Three launches keep that order and give the same bits: one wavefront per (query, head) that walks
// the pages itself (or, in a step of many queries, per four neighbouring queries, which share what
// they fetch); or, for steps of few queries over many keys (one-token steps), a wavefront
// per (query, head, page) that leaves its page's result in a workspace, and a second kernel that
// joins them in order (one wavefront alone would walk thousands of keys while the chip idles:
// a one-token step of 28 heads over 2,048 keys took 2.4 ms so).
// No multiply and add of this file is fused unless it is written as an fma: the same lines are
// compiled into several kernels that must give the same bits.
#pragma clang fp contract(off)
#include "cache_layout.h"
#include "hector_kernels.h"

#define AP_MAX_PER_LANE 8

// NPL: head elements a lane holds (head_dim / 64 rounded up to 1, 2, 4 or 8)
template <int NPL>
struct ApState {
  float m, l;
  float acc[NPL];
};

// The score of one key: k holds this lane's elements of the key. It does not depend on the keys
// before it, so the scores of a group of keys are computed side by side ahead of the chain below.
template <int NPL>
__device__ __forceinline__ float ap_score(const float (&qv)[NPL], const float (&k)[NPL], float scale, int lane,
                                          int npl, int hd) {
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int d = lane + i * HE_WAVE;
    if (i < npl && d < hd) part = fmaf(qv[i], k[i], part);
  }
  return wave_sum(part) * scale;
}

// One key joins the running softmax of a page: s is its score, v this lane's elements of its value.
// Of the two weights exp(m - m_new) and exp(s - m_new) one is exp(0) = 1: one exponential a key.
template <int NPL>
__device__ __forceinline__ void ap_update(ApState<NPL>& st, float s, const float (&v)[NPL], int lane, int npl,
                                          int hd) {
  const bool up = s > st.m;                 // the reference point moves to s
  const float m_new = up ? s : st.m;
  const float e = expf(up ? st.m - s : s - st.m);
  const float alpha = up ? e : 1.f;
  const float w = up ? 1.f : e;
  st.l = fmaf(st.l, alpha, w);
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int d = lane + i * HE_WAVE;
    if (i < npl && d < hd) st.acc[i] = fmaf(st.acc[i], alpha, w * v[i]);
  }
  st.m = m_new;
}

#define AP_GROUP 4
// The key and value elements of this lane for the AP_GROUP keys from j0 on (positions beyond j_hi
// read key j_hi again: no load stands behind a condition, so the compiler counts what is in flight).
template <typename T, int NPL>
__device__ __forceinline__ void ap_fetch(float (&kv)[AP_GROUP][NPL], float (&vv)[AP_GROUP][NPL], const T* kpage,
                                         const T* vpage, int j0, int j_hi, int KS, int NT, int lane, int npl,
                                         int hd) {
#pragma unroll
  for (int g = 0; g < AP_GROUP; ++g) {
    const int off = min(j0 + g, j_hi) & (HE_PAGE_TOKENS - 1);
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int d = lane + i * HE_WAVE;
      const bool has = i < npl && d < hd;
      kv[g][i] = has ? to_float(kpage[he_k_index(off, d, KS)]) : 0.f;
      vv[g][i] = has ? to_float(vpage[he_v_index(off, d, NT)]) : 0.f;
    }
  }
}

// The online softmax of the keys [j_lo, j_hi] of one page (they lie in the same page), begun afresh.
// Every multiply-add is written out as an fma: these lines are compiled into several kernels,
// and the compiler would otherwise be free to fuse each copy its own way.
template <typename T, int NPL>
__device__ __forceinline__ void ap_page(ApState<NPL>& st, const float (&qv)[NPL], const T* kpool,
                                        const T* vpool, int page, int num_pages, int KVH, int kvh, int hd,
                                        int j_lo, int j_hi, float scale, int lane, int npl) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) st.acc[i] = 0.f;
  if (page < 0 || page >= num_pages) return;  // never for an admitted batch
  // the pages are stored in the MFMA kernels' operand order (cache_layout.h)
  const T* kpage = kpool + ((int64_t)page * KVH + kvh) * he_k_page_elems(hd);
  const T* vpage = vpool + ((int64_t)page * KVH + kvh) * he_v_page_elems(hd);
  const int KS = he_k_steps(hd), NT = he_v_tiles(hd);
  // Four keys at a time, in two sets of registers: while the chain of the softmax takes the keys of
  // one set one by one in ascending position, the elements of the next four are on their way (a key
  // at a time, each load was waited for before the next was asked for: 1 us a key; four at a time
  // without the second set, a wait of its own for every four: a page of 64 keys 39 us).
  float ka[AP_GROUP][NPL], va[AP_GROUP][NPL], kb[AP_GROUP][NPL], vb[AP_GROUP][NPL];
  ap_fetch<T, NPL>(ka, va, kpage, vpage, j_lo, j_hi, KS, NT, lane, npl, hd);
  for (int j0 = j_lo; j0 <= j_hi; j0 += 2 * AP_GROUP) {
    ap_fetch<T, NPL>(kb, vb, kpage, vpage, j0 + AP_GROUP, j_hi, KS, NT, lane, npl, hd);
    float sc[AP_GROUP];
#pragma unroll
    for (int g = 0; g < AP_GROUP; ++g) sc[g] = ap_score<NPL>(qv, ka[g], scale, lane, npl, hd);
#pragma unroll
    for (int g = 0; g < AP_GROUP; ++g)
      if (j0 + g <= j_hi) ap_update<NPL>(st, sc[g], va[g], lane, npl, hd);
    ap_fetch<T, NPL>(ka, va, kpage, vpage, j0 + 2 * AP_GROUP, j_hi, KS, NT, lane, npl, hd);
#pragma unroll
    for (int g = 0; g < AP_GROUP; ++g) sc[g] = ap_score<NPL>(qv, kb[g], scale, lane, npl, hd);
#pragma unroll
    for (int g = 0; g < AP_GROUP; ++g)
      if (j0 + AP_GROUP + g <= j_hi) ap_update<NPL>(st, sc[g], vb[g], lane, npl, hd);
  }
}

// total <- total joined with the result of the next page (one that had keys).
template <int NPL>
__device__ __forceinline__ void ap_join(ApState<NPL>& total, const ApState<NPL>& st) {
  if (!(st.m > -INFINITY)) return;
  const float m_new = fmaxf(total.m, st.m);
  const float a = total.m > -INFINITY ? expf(total.m - m_new) : 0.f;
  const float b = expf(st.m - m_new);
  total.l = fmaf(total.l, a, st.l * b);
#pragma unroll
  for (int i = 0; i < NPL; ++i) total.acc[i] = fmaf(total.acc[i], a, st.acc[i] * b);
  total.m = m_new;
}

// grid (rows, ceil(H / 4), pages): pages == 1: the wavefront walks all pages of its query and stores
// the result; pages > 1: it takes the page (first >> 6) + blockIdx.z alone and stores (m, l, sums)
// into ws [row][head][pages][hd + 2], if the query has such a page.
template <typename T, int NPL>
__global__ __launch_bounds__(256) void attention_plain_kernel(
    T* __restrict__ out, float* __restrict__ ws, const T* __restrict__ q, const T* __restrict__ kpool,
    const T* __restrict__ vpool, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ page_table, int max_blocks, int num_pages, int H, int KVH, int hd,
    int window, float scale) {
  const int lane = threadIdx.x & (HE_WAVE - 1);
  const int h = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int64_t row = blockIdx.x;
  if (h >= H) return;
  const bool split = gridDim.z > 1;
  T* o = out + (row * H + h) * (int64_t)hd;
  const int seq = row_seq[row];
  const int npl = (hd + HE_WAVE - 1) / HE_WAVE;
  if (seq < 0) {
    if (!split)
      for (int i = 0; i < npl; ++i) {
        const int d = lane + i * HE_WAVE;
        if (d < hd) o[d] = from_float<T>(0.f);
      }
    return;
  }
  const int p = positions[row];
  const int slot = seq_slot[seq];
  const int kvh = h / (H / KVH);
  const int first = window > 0 ? max(0, p + 1 - window) : 0;
  const int32_t* pt = page_table + (int64_t)slot * max_blocks;
  const int c_first = first >> HE_PAGE_SHIFT, c_last = p >> HE_PAGE_SHIFT;
  if (split && c_first + (int)blockIdx.z > c_last) return;

  float qv[NPL];
  const T* qrow = q + (row * H + h) * (int64_t)hd;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int d = lane + i * HE_WAVE;
    qv[i] = (i < npl && d < hd) ? to_float(qrow[d]) : 0.f;
  }
  ApState<NPL> st;
  if (split) {
    const int c = c_first + blockIdx.z;
    ap_page<T, NPL>(st, qv, kpool, vpool, pt[c], num_pages, KVH, kvh, hd, max(first, c << HE_PAGE_SHIFT),
               min(p, (c << HE_PAGE_SHIFT) + HE_PAGE_TOKENS - 1), scale, lane, npl);
    float* w = ws + ((row * H + h) * (int64_t)gridDim.z + blockIdx.z) * (hd + 2);
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int d = lane + i * HE_WAVE;
      if (i < npl && d < hd) w[d] = st.acc[i];
    }
    if (lane == 0) w[hd] = st.m, w[hd + 1] = st.l;
    return;
  }
  ApState<NPL> total;
  total.m = -INFINITY;
  total.l = 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) total.acc[i] = 0.f;
  for (int c = c_first; c <= c_last; ++c) {
    ap_page<T, NPL>(st, qv, kpool, vpool, pt[c], num_pages, KVH, kvh, hd, max(first, c << HE_PAGE_SHIFT),
               min(p, (c << HE_PAGE_SHIFT) + HE_PAGE_TOKENS - 1), scale, lane, npl);
    ap_join(total, st);
  }
  const float inv = total.l > 0.f ? 1.f / total.l : 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int d = lane + i * HE_WAVE;
    if (i < npl && d < hd) o[d] = from_float<T>(total.acc[i] * inv);
  }
}

// Four neighbouring queries of one sequence and head in one wavefront (whole prompts): every key
// and value is fetched once for the four, and each query still takes its own keys [first, p] page by
// page in the order above, so the bits are those of the kernel that takes a query at a time. A
// group of four rows that is not four consecutive positions of one sequence (the end of a
// sequence, padding) is taken query by query. grid (ceil(rows / 4), ceil(H / 4)).
#define AP_ROWS 4
template <typename T, int NPL>
__global__ __launch_bounds__(256) void attention_plain_rows_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kpool, const T* __restrict__ vpool,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ page_table, int max_blocks,
    int num_pages, int rows, int H, int KVH, int hd, int window, float scale) {
  const int lane = threadIdx.x & (HE_WAVE - 1);
  const int h = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (h >= H) return;
  const int64_t row0 = (int64_t)blockIdx.x * AP_ROWS;
  const int npl = (hd + HE_WAVE - 1) / HE_WAVE;
  const int kvh = h / (H / KVH);
  const int n_rows = (int)min((int64_t)AP_ROWS, rows - row0);
  const int seq0 = row_seq[row0], p0 = positions[row0];
  bool together = n_rows == AP_ROWS && seq0 >= 0;
  for (int r = 1; r < n_rows; ++r) together = together && row_seq[row0 + r] == seq0 && positions[row0 + r] == p0 + r;
  auto store = [&](int64_t row, const ApState<NPL>& total) {
    T* o = out + (row * H + h) * (int64_t)hd;
    const float inv = total.l > 0.f ? 1.f / total.l : 0.f;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int d = lane + i * HE_WAVE;
      if (i < npl && d < hd) o[d] = from_float<T>(total.acc[i] * inv);
    }
  };
  auto load_q = [&](float (&qv)[NPL], int64_t row) {
    const T* qrow = q + (row * H + h) * (int64_t)hd;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int d = lane + i * HE_WAVE;
      qv[i] = (i < npl && d < hd) ? to_float(qrow[d]) : 0.f;
    }
  };
  if (!together) {
    for (int r = 0; r < n_rows; ++r) {
      const int64_t row = row0 + r;
      ApState<NPL> total, st;
      total.m = -INFINITY;
      total.l = 0.f;
#pragma unroll
      for (int i = 0; i < NPL; ++i) total.acc[i] = 0.f;
      const int seq = row_seq[row];
      if (seq >= 0) {
        const int p = positions[row];
        const int first = window > 0 ? max(0, p + 1 - window) : 0;
        const int32_t* pt = page_table + (int64_t)seq_slot[seq] * max_blocks;
        float qv[NPL];
        load_q(qv, row);
        for (int c = first >> HE_PAGE_SHIFT; c <= (p >> HE_PAGE_SHIFT); ++c) {
          ap_page<T, NPL>(st, qv, kpool, vpool, pt[c], num_pages, KVH, kvh, hd, max(first, c << HE_PAGE_SHIFT),
                          min(p, (c << HE_PAGE_SHIFT) + HE_PAGE_TOKENS - 1), scale, lane, npl);
          ap_join(total, st);
        }
      }
      store(row, total);
    }
    return;
  }
  const int32_t* pt = page_table + (int64_t)seq_slot[seq0] * max_blocks;
  float qv[AP_ROWS][NPL];
  ApState<NPL> total[AP_ROWS], st[AP_ROWS];
  int first[AP_ROWS];
#pragma unroll
  for (int r = 0; r < AP_ROWS; ++r) {
    load_q(qv[r], row0 + r);
    first[r] = window > 0 ? max(0, p0 + r + 1 - window) : 0;
    total[r].m = -INFINITY;
    total[r].l = 0.f;
#pragma unroll
    for (int i = 0; i < NPL; ++i) total[r].acc[i] = 0.f;
  }
  const int KS = he_k_steps(hd), NT = he_v_tiles(hd);
  const int p_last = p0 + AP_ROWS - 1;
  for (int c = first[0] >> HE_PAGE_SHIFT; c <= (p_last >> HE_PAGE_SHIFT); ++c) {
#pragma unroll
    for (int r = 0; r < AP_ROWS; ++r) {
      st[r].m = -INFINITY;
      st[r].l = 0.f;
#pragma unroll
      for (int i = 0; i < NPL; ++i) st[r].acc[i] = 0.f;
    }
    const int page = pt[c];
    if (page >= 0 && page < num_pages) {
      const int64_t base = ((int64_t)page * KVH + kvh) * he_k_page_elems(hd);
      const int64_t vbase = ((int64_t)page * KVH + kvh) * he_v_page_elems(hd);
      const int j_lo = max(first[0], c << HE_PAGE_SHIFT), j_hi = min(p_last, (c << HE_PAGE_SHIFT) + HE_PAGE_TOKENS - 1);
      const T* kpage = kpool + base;
      const T* vpage = vpool + vbase;
      // two sets of registers, as in ap_page: the next four keys are on their way while these are taken
      float ka[AP_GROUP][NPL], va[AP_GROUP][NPL], kb[AP_GROUP][NPL], vb[AP_GROUP][NPL];
      ap_fetch<T, NPL>(ka, va, kpage, vpage, j_lo, j_hi, KS, NT, lane, npl, hd);
      for (int j0 = j_lo; j0 <= j_hi; j0 += 2 * AP_GROUP) {
        ap_fetch<T, NPL>(kb, vb, kpage, vpage, j0 + AP_GROUP, j_hi, KS, NT, lane, npl, hd);
        float sc[AP_GROUP][AP_ROWS];
#pragma unroll
        for (int g = 0; g < AP_GROUP; ++g)
#pragma unroll
          for (int r = 0; r < AP_ROWS; ++r) sc[g][r] = ap_score<NPL>(qv[r], ka[g], scale, lane, npl, hd);
#pragma unroll
        for (int g = 0; g < AP_GROUP; ++g) {
          const int j = j0 + g;
#pragma unroll
          for (int r = 0; r < AP_ROWS; ++r)
            if (j <= j_hi && j >= first[r] && j <= p0 + r) ap_update<NPL>(st[r], sc[g][r], va[g], lane, npl, hd);
        }
        ap_fetch<T, NPL>(ka, va, kpage, vpage, j0 + 2 * AP_GROUP, j_hi, KS, NT, lane, npl, hd);
#pragma unroll
        for (int g = 0; g < AP_GROUP; ++g)
#pragma unroll
          for (int r = 0; r < AP_ROWS; ++r) sc[g][r] = ap_score<NPL>(qv[r], kb[g], scale, lane, npl, hd);
#pragma unroll
        for (int g = 0; g < AP_GROUP; ++g) {
          const int j = j0 + AP_GROUP + g;
#pragma unroll
          for (int r = 0; r < AP_ROWS; ++r)
            if (j <= j_hi && j >= first[r] && j <= p0 + r) ap_update<NPL>(st[r], sc[g][r], vb[g], lane, npl, hd);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < AP_ROWS; ++r) ap_join(total[r], st[r]);
  }
#pragma unroll
  for (int r = 0; r < AP_ROWS; ++r) store(row0 + r, total[r]);
}

// Joins the pages' results of a split launch in ascending position. grid (rows, ceil(H / 4)).
template <typename T, int NPL>
__global__ __launch_bounds__(256) void attention_plain_join_kernel(
    T* __restrict__ out, const float* __restrict__ ws, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_seq, int H, int hd, int window, int pages) {
  const int lane = threadIdx.x & (HE_WAVE - 1);
  const int h = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int64_t row = blockIdx.x;
  if (h >= H) return;
  T* o = out + (row * H + h) * (int64_t)hd;
  const int npl = (hd + HE_WAVE - 1) / HE_WAVE;
  ApState<NPL> total;
  total.m = -INFINITY;
  total.l = 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) total.acc[i] = 0.f;
  if (row_seq[row] >= 0) {
    const int p = positions[row];
    const int first = window > 0 ? max(0, p + 1 - window) : 0;
    const int count = (p >> HE_PAGE_SHIFT) - (first >> HE_PAGE_SHIFT) + 1;
    if (count > pages) {
      // the caller's bound on the keys was too low: no part of the result may pass for one
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        const int d = lane + i * HE_WAVE;
        if (i < npl && d < hd) o[d] = from_float<T>(NAN);
      }
      return;
    }
    // eight pages' results are asked for together and then joined one after the other in order
    // (one at a time, every page waited for its own loads: 17 us for 33 pages)
    constexpr int AHEAD = 8;
    for (int z0 = 0; z0 < count; z0 += AHEAD) {
      ApState<NPL> part[AHEAD];
#pragma unroll
      for (int u = 0; u < AHEAD; ++u) {
        const float* w = ws + ((row * H + h) * (int64_t)pages + min(z0 + u, count - 1)) * (hd + 2);
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
          const int d = lane + i * HE_WAVE;
          part[u].acc[i] = (i < npl && d < hd) ? w[d] : 0.f;
        }
        part[u].m = w[hd];
        part[u].l = w[hd + 1];
      }
#pragma unroll
      for (int u = 0; u < AHEAD; ++u)
        if (z0 + u < count) ap_join(total, part[u]);
    }
  }
  const float inv = total.l > 0.f ? 1.f / total.l : 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int d = lane + i * HE_WAVE;
    if (i < npl && d < hd) o[d] = from_float<T>(total.acc[i] * inv);
  }
}

// Pages a query of this step has at most (what a split launch needs room for), given the most keys
// a sequence holds after the step.
static int ap_pages(int most_keys, int window) {
  int pages = (most_keys + HE_PAGE_TOKENS - 1) / HE_PAGE_TOKENS;
  if (window > 0) pages = min(pages, (window + HE_PAGE_TOKENS - 2) / HE_PAGE_TOKENS + 1);
  return max(pages, 1);
}

// Floats of workspace with which the step's attention runs page by page in parallel (0: one
// wavefront per query and head walks the pages itself; that is the better launch for a step with
// many queries).
extern "C" int64_t he_attention_plain_workspace_floats(int rows, int H, int hd, int most_keys, int window) {
  if (rows <= 0 || H <= 0 || hd <= 0 || most_keys <= 0) return 0;
  const int pages = ap_pages(most_keys, window);
  if (pages < 2 || (int64_t)rows * H > 8 * he_cus()) return 0;
  return (int64_t)rows * H * pages * (hd + 2);
}

extern "C" int he_attention_plain(void* out, const void* q, const void* kpool, const void* vpool,
                                  const void* positions, const void* row_seq, const void* seq_slot,
                                  const void* page_table, int max_blocks, int num_pages, int rows,
                                  int H, int KVH, int hd, int window, float scale, int dtype,
                                  int most_keys, void* workspace_f32, int64_t workspace_floats,
                                  void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && KVH > 0 && hd > 0, "he_attention_plain: bad sizes");
  HE_REQUIRE(H % KVH == 0, "he_attention_plain: heads %d not a multiple of kv heads %d", H, KVH);
  HE_REQUIRE(hd <= AP_MAX_PER_LANE * HE_WAVE, "he_attention_plain: head_dim %d above %d", hd,
             AP_MAX_PER_LANE * HE_WAVE);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_attention_plain: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  // page by page in parallel when the caller brought room for it (the same bits either way)
  const int64_t need = he_attention_plain_workspace_floats(rows, H, hd, most_keys, window);
  const bool split = need > 0 && workspace_f32 != nullptr && workspace_floats >= need;
  const int pages = split ? ap_pages(most_keys, window) : 1;
  HE_REQUIRE(pages <= 65535, "he_attention_plain: %d pages of keys are too many for one launch", pages);
  dim3 grid(rows, (H + 3) / 4, pages);
  float* ws = (float*)workspace_f32;
  hipStream_t s = (hipStream_t)stream;
#define AP_LAUNCH(T, NPL)                                                                      \
  attention_plain_kernel<T, NPL><<<grid, 256, 0, s>>>(                                         \
      (T*)out, ws, (const T*)q, (const T*)kpool, (const T*)vpool, (const int32_t*)positions,   \
      (const int32_t*)row_seq, (const int32_t*)seq_slot, (const int32_t*)page_table,           \
      max_blocks, num_pages, H, KVH, hd, window, scale)
#define AP_JOIN(T, NPL)                                                                        \
  attention_plain_join_kernel<T, NPL><<<dim3(rows, (H + 3) / 4), 256, 0, s>>>(                 \
      (T*)out, ws, (const int32_t*)positions, (const int32_t*)row_seq, H, hd, window, pages)
  const int npl = (hd + HE_WAVE - 1) / HE_WAVE;   // elements a lane holds: 1, 2, up to 4, up to 8
#define AP_BY_SIZE(WHAT)                                  \
  if (dtype == HE_BF16) {                                 \
    if (npl <= 1) WHAT(bf16_t, 1);                        \
    else if (npl <= 2) WHAT(bf16_t, 2);                   \
    else if (npl <= 4) WHAT(bf16_t, 4);                   \
    else WHAT(bf16_t, 8);                                 \
  } else {                                                \
    if (npl <= 1) WHAT(float, 1);                         \
    else if (npl <= 2) WHAT(float, 2);                    \
    else if (npl <= 4) WHAT(float, 4);                    \
    else WHAT(float, 8);                                  \
  }
#define AP_ROWS_LAUNCH(T, NPL)                                                                          \
  attention_plain_rows_kernel<T, NPL><<<dim3((rows + AP_ROWS - 1) / AP_ROWS, (H + 3) / 4), 256, 0, s>>>(   \
      (T*)out, (const T*)q, (const T*)kpool, (const T*)vpool, (const int32_t*)positions,               \
      (const int32_t*)row_seq, (const int32_t*)seq_slot, (const int32_t*)page_table, max_blocks,       \
      num_pages, rows, H, KVH, hd, window, scale)
  if (!split && rows >= 64) {      // a step of many queries: four neighbours a wavefront share their keys
    AP_BY_SIZE(AP_ROWS_LAUNCH)
    return he_check_launch("he_attention_plain");
  }
  AP_BY_SIZE(AP_LAUNCH)
  int rc = he_check_launch("he_attention_plain");
  if (rc || !split) return rc;
  AP_BY_SIZE(AP_JOIN)
#undef AP_BY_SIZE
#undef AP_ROWS_LAUNCH
#undef AP_LAUNCH
#undef AP_JOIN
  return he_check_launch("he_attention_plain");
}
