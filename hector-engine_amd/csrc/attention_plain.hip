// Plain attention over the paged cache: one wavefront per (query row, head),
// keys visited one by one in ascending position with an online softmax in
// fp32. The result for a query depends only on its own position and the cache
// rows [first, p], never on how the step was cut or batched, so prompt steps
// and one-token steps give identical bits. It is the 32-bit path's attention
// and the reference beside the MFMA kernels.
//
// For the query at absolute position p: first = window > 0 ? max(0, p+1-window) : 0,
// s_j = (q . k_j) * scale for j in [first, p], out = sum_j softmax(s)_j v_j,
// kv head = h / (H / KVH)   (reference: kernels/attention.cu:155-316, :664-773, :60).
#include "cache_layout.h"
#include "hector_kernels.h"

#define AP_MAX_PER_LANE 8

template <typename T>
__global__ __launch_bounds__(256) void attention_plain_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kpool,
    const T* __restrict__ vpool, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ page_table, int max_blocks, int num_pages, int H, int KVH, int hd,
    int window, float scale) {
  const int lane = threadIdx.x & (HE_WAVE - 1);
  const int h = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int64_t row = blockIdx.x;
  if (h >= H) return;
  T* o = out + (row * H + h) * (int64_t)hd;
  const int seq = row_seq[row];
  const int npl = (hd + HE_WAVE - 1) / HE_WAVE;
  if (seq < 0) {
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

  float qv[AP_MAX_PER_LANE], acc[AP_MAX_PER_LANE];
  const T* qrow = q + (row * H + h) * (int64_t)hd;
#pragma unroll
  for (int i = 0; i < AP_MAX_PER_LANE; ++i) {
    const int d = lane + i * HE_WAVE;
    qv[i] = (i < npl && d < hd) ? to_float(qrow[d]) : 0.f;
    acc[i] = 0.f;
  }
  float m = -INFINITY, l = 0.f;
  for (int j = first; j <= p; ++j) {
    const int page = pt[j >> HE_PAGE_SHIFT];
    if (page < 0 || page >= num_pages) continue;  // never for an admitted batch
    const int off = j & (HE_PAGE_TOKENS - 1);
    // the pages are stored in the MFMA kernels' operand order (cache_layout.h)
    const int64_t base = ((int64_t)page * KVH + kvh) * he_k_page_elems(hd);
    const int64_t vbase = ((int64_t)page * KVH + kvh) * he_v_page_elems(hd);
    const int KS = he_k_steps(hd), NT = he_v_tiles(hd);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < AP_MAX_PER_LANE; ++i) {
      const int d = lane + i * HE_WAVE;
      if (i < npl && d < hd) part = fmaf(qv[i], to_float(kpool[base + he_k_index(off, d, KS)]), part);
    }
    const float s = wave_sum(part) * scale;
    const float m_new = fmaxf(m, s);
    const float alpha = expf(m - m_new);
    const float w = expf(s - m_new);
    l = l * alpha + w;
#pragma unroll
    for (int i = 0; i < AP_MAX_PER_LANE; ++i) {
      const int d = lane + i * HE_WAVE;
      if (i < npl && d < hd) acc[i] = acc[i] * alpha + w * to_float(vpool[vbase + he_v_index(off, d, NT)]);
    }
    m = m_new;
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int i = 0; i < AP_MAX_PER_LANE; ++i) {
    const int d = lane + i * HE_WAVE;
    if (i < npl && d < hd) o[d] = from_float<T>(acc[i] * inv);
  }
}

extern "C" int he_attention_plain(void* out, const void* q, const void* kpool, const void* vpool,
                                  const void* positions, const void* row_seq, const void* seq_slot,
                                  const void* page_table, int max_blocks, int num_pages, int rows,
                                  int H, int KVH, int hd, int window, float scale, int dtype,
                                  void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && KVH > 0 && hd > 0, "he_attention_plain: bad sizes");
  HE_REQUIRE(H % KVH == 0, "he_attention_plain: heads %d not a multiple of kv heads %d", H, KVH);
  HE_REQUIRE(hd <= AP_MAX_PER_LANE * HE_WAVE, "he_attention_plain: head_dim %d above %d", hd,
             AP_MAX_PER_LANE * HE_WAVE);
  if (rows == 0) return 0;
  dim3 grid(rows, (H + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
#define AP_LAUNCH(T)                                                                       \
  attention_plain_kernel<T><<<grid, 256, 0, s>>>(                                          \
      (T*)out, (const T*)q, (const T*)kpool, (const T*)vpool, (const int32_t*)positions,   \
      (const int32_t*)row_seq, (const int32_t*)seq_slot, (const int32_t*)page_table,       \
      max_blocks, num_pages, H, KVH, hd, window, scale)
  if (dtype == HE_BF16)
    AP_LAUNCH(bf16_t);
  else if (dtype == HE_F32)
    AP_LAUNCH(float);
  else
    HE_REQUIRE(false, "he_attention_plain: unknown dtype %d", dtype);
#undef AP_LAUNCH
  return he_check_launch("he_attention_plain");
}
