// One pass over the projected q/k/v rows of a step: add the projection bias,
// rotate q and k by each row's own position, write q out densely and scatter
// k and v into the paged cache at (slot, position). It replaces the reference's
// add_bias, rope and kv_cache_update launches (kernels/elementwise.cu:307-323,
// kernels/attention.cu:516-558, kernels/attention.cu:1067-1097).
//
// Rotation (half-split pairing): for i < r/2, a = pos * inv_freq[i],
//   y[i]       = x[i] * cos a - x[i + r/2] * sin a
//   y[i + r/2] = x[i] * sin a + x[i + r/2] * cos a
// and dims >= r pass through. All of it in fp32.
#include "cache_layout.h"
#include "hector_kernels.h"

#define ROPE_MAX_HALF 256

template <typename T, typename TI>
__global__ void qkv_rope_cache_kernel(
    T* __restrict__ q_out, T* __restrict__ kpool, T* __restrict__ vpool,
    const TI* __restrict__ q_in, const TI* __restrict__ k_in, const TI* __restrict__ v_in,
    int64_t in_stride, const void* __restrict__ q_bias, const void* __restrict__ k_bias,
    const void* __restrict__ v_bias, int bias_dtype, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ seq_slot,
    const int32_t* __restrict__ page_table, int max_blocks, int num_pages,
    const float* __restrict__ inv_freq, int rotary_dim, int H, int KVH, int hd) {
  __shared__ float cs[2][ROPE_MAX_HALF];
  const int64_t row = blockIdx.x;
  const int seq = row_seq[row];
  if (seq < 0) return;  // padding row
  const int pos = positions[row];
  const int half = rotary_dim >> 1;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float a = (float)pos * inv_freq[i];
    float sn, c;
    sincos_angle(a, &sn, &c);
    cs[0][i] = c;
    cs[1][i] = sn;
  }
  __syncthreads();

  // ---- q: rotate and store densely
  {
    const TI* in = q_in + row * in_stride;
    T* out = q_out + row * (int64_t)H * hd;
    const int per_head = half + (hd - rotary_dim);
    for (int it = threadIdx.x; it < H * per_head; it += blockDim.x) {
      const int h = it / per_head;
      const int j = it - h * per_head;
      const int base = h * hd;
      if (j < half) {
        float x0 = to_float((in + base + j)[0]);
        float x1 = to_float((in + base + j + half)[0]);
        if (q_bias) {
          x0 += load_param(q_bias, base + j, bias_dtype);
          x1 += load_param(q_bias, base + j + half, bias_dtype);
        }
        const float c = cs[0][j], sn = cs[1][j];
        out[base + j] = from_float<T>(x0 * c - x1 * sn);
        out[base + j + half] = from_float<T>(x0 * sn + x1 * c);
      } else {
        const int d = rotary_dim + (j - half);
        float x = to_float((in + base + d)[0]);
        if (q_bias) x += load_param(q_bias, base + d, bias_dtype);
        out[base + d] = from_float<T>(x);
      }
    }
  }
  if (k_in == nullptr) return;  // this layer reads another layer's cache

  const int slot = seq_slot[seq];
  const int page = page_table[(int64_t)slot * max_blocks + (pos >> HE_PAGE_SHIFT)];
  if (page < 0 || page >= num_pages) return;  // never for a batch the host has admitted
  const int off = pos & (HE_PAGE_TOKENS - 1);
  // ---- k: rotate and scatter
  {
    const TI* in = k_in + row * in_stride;
    const int per_head = half + (hd - rotary_dim);
    for (int it = threadIdx.x; it < KVH * per_head; it += blockDim.x) {
      const int h = it / per_head;
      const int j = it - h * per_head;
      const int base = h * hd;
      T* out = kpool + ((int64_t)page * KVH + h) * he_k_page_elems(hd);   // the page, in operand order
      const int KS = he_k_steps(hd);
      if (j < half) {
        float x0 = to_float((in + base + j)[0]);
        float x1 = to_float((in + base + j + half)[0]);
        if (k_bias) {
          x0 += load_param(k_bias, base + j, bias_dtype);
          x1 += load_param(k_bias, base + j + half, bias_dtype);
        }
        const float c = cs[0][j], sn = cs[1][j];
        out[he_k_index(off, j, KS)] = from_float<T>(x0 * c - x1 * sn);
        out[he_k_index(off, j + half, KS)] = from_float<T>(x0 * sn + x1 * c);
      } else {
        const int d = rotary_dim + (j - half);
        float x = to_float((in + base + d)[0]);
        if (k_bias) x += load_param(k_bias, base + d, bias_dtype);
        out[he_k_index(off, d, KS)] = from_float<T>(x);
      }
    }
  }
  // ---- v: bias and scatter
  {
    const TI* in = v_in + row * in_stride;
    for (int it = threadIdx.x; it < KVH * hd; it += blockDim.x) {
      const int h = it / hd;
      const int d = it - h * hd;
      float x = to_float((in + it)[0]);
      if (v_bias) x += load_param(v_bias, it, bias_dtype);
      vpool[((int64_t)page * KVH + h) * he_v_page_elems(hd) + he_v_index(off, d, he_v_tiles(hd))] =
          from_float<T>(x);
    }
  }
}

// bf16 rows, eight elements per access: one thread rotates the pairs (j..j+7, j+half..)
// of one head, or copies eight v elements. Needs rotary_dim/2, head_dim - rotary_dim and
// the row stride in multiples of 8.
__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint4 pack8(const float* f) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = (uint32_t)float_to_bf16_bits(f[2 * i]) | ((uint32_t)float_to_bf16_bits(f[2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// grid: one workgroup per 8 rows for v, then one per row for q and k.
// V lies transposed in a page (8 keys of one dim are 16 contiguous bytes), so the v values of
// a run of tokens that share such a group are gathered dim by dim and stored together: 16
// bytes a store when the run is a whole group (a prompt), 2 bytes a token otherwise.
__global__ __launch_bounds__(1024) void qkv_rope_cache_vec_kernel(
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ kpool, uint16_t* __restrict__ vpool,
    const uint16_t* __restrict__ q_in, const uint16_t* __restrict__ k_in,
    const uint16_t* __restrict__ v_in, int64_t in_stride, const uint16_t* __restrict__ q_bias,
    const uint16_t* __restrict__ k_bias, const uint16_t* __restrict__ v_bias,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ page_table, int max_blocks,
    int num_pages, const float* __restrict__ inv_freq, int rotary_dim, int rows, int H, int KVH,
    int hd) {
  __shared__ float cs[2][ROPE_MAX_HALF];
  const int v_blocks = (int)gridDim.x - rows;   // they come first: theirs is the longest chain of dependent loads
  if ((int)blockIdx.x < v_blocks) {
    // ---- v: the runs of tokens that begin in rows [r0, r0 + 8)
    const int r0 = 8 * (int)blockIdx.x;
    const int NT = he_v_tiles(hd);
    for (int r = r0; r < min(r0 + 8, rows); ++r) {
      const int seq = row_seq[r];
      if (seq < 0) continue;
      const int pos = positions[r];
      const bool begins = (pos & 7) == 0 || r == 0 || row_seq[r - 1] != seq || positions[r - 1] != pos - 1;
      if (!begins) continue;
      int n = 1;   // tokens of the run: the same sequence, consecutive positions, one group of 8 keys
      while (n < 8 - (pos & 7) && r + n < rows && row_seq[r + n] == seq && positions[r + n] == pos + n) ++n;
      const int page = page_table[(int64_t)seq_slot[seq] * max_blocks + (pos >> HE_PAGE_SHIFT)];
      if (page < 0 || page >= num_pages) continue;
      const int off = pos & (HE_PAGE_TOKENS - 1);
      for (int e = threadIdx.x; e < KVH * hd; e += blockDim.x) {
        const int h = e / hd, d = e - h * hd;
        const float b = v_bias ? bf16_bits_to_float(v_bias[e]) : 0.f;
        uint16_t vals[8];
        // eight loads with no branch around them (a token beyond the run reads the run's last
        // row and is dropped): they go out together
#pragma unroll
        for (int i = 0; i < 8; ++i) vals[i] = v_in[(int64_t)(r + min(i, n - 1)) * in_stride + e];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (v_bias) vals[i] = float_to_bf16_bits(bf16_bits_to_float(vals[i]) + b);
          if (i >= n) vals[i] = 0;
        }
        uint16_t* out = vpool + ((int64_t)page * KVH + h) * he_v_page_elems(hd) + he_v_index(off, d, NT);
        if (n == 8) {
          *reinterpret_cast<uint4*>(out) =
              make_uint4(vals[0] | ((uint32_t)vals[1] << 16), vals[2] | ((uint32_t)vals[3] << 16),
                         vals[4] | ((uint32_t)vals[5] << 16), vals[6] | ((uint32_t)vals[7] << 16));
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (i < n) out[i] = vals[i];
        }
      }
    }
    return;
  }
  // ---- q and k of one row
  const int64_t row = (int)blockIdx.x - v_blocks;
  const int seq = row_seq[row];
  if (seq < 0) return;  // padding row
  const int half = rotary_dim >> 1;
  const int rot8 = half >> 3;                 // groups of 8 pairs per head
  const int pass8 = (hd - rotary_dim) >> 3;   // groups of 8 pass-through dims per head
  const int per_head = rot8 + pass8;
  const int q_items = H * per_head;
  const int items = q_items + (k_in ? KVH * per_head : 0);
  // an item: eight pairs (j.., j + half..) of one head, or eight pass-through dims from d on
  struct Item {
    const uint16_t* in;
    const uint16_t* bias;
    int h, j;
    bool is_q, rotated;
  };
  auto item = [&](int it) {
    Item im;
    im.is_q = it < q_items;
    const int idx = im.is_q ? it : it - q_items;
    im.h = idx / per_head;
    const int g = idx - im.h * per_head;
    im.rotated = g < rot8;
    im.j = im.rotated ? 8 * g : rotary_dim + 8 * (g - rot8);
    im.in = (im.is_q ? q_in : k_in) + row * in_stride + im.h * hd;
    const uint16_t* bias = im.is_q ? q_bias : k_bias;
    im.bias = bias ? bias + im.h * hd : nullptr;
    return im;
  };
  const uint4 zero = make_uint4(0, 0, 0, 0);
  // four loads with no branch around them, so that they go out together: an item without a
  // partner, or a row without a bias, reads its own eight elements again and drops them
  auto load = [&](const Item& im, uint4 (&raw)[4]) {
    const int partner = im.rotated ? im.j + half : im.j;
    const uint16_t* b = im.bias ? im.bias : im.in;
    const uint4 x0 = *reinterpret_cast<const uint4*>(im.in + im.j);
    const uint4 x1 = *reinterpret_cast<const uint4*>(im.in + partner);
    const uint4 b0 = *reinterpret_cast<const uint4*>(b + im.j);
    const uint4 b1 = *reinterpret_cast<const uint4*>(b + partner);
    raw[0] = x0;
    raw[1] = im.rotated ? x1 : zero;
    raw[2] = im.bias ? b0 : zero;
    raw[3] = im.bias && im.rotated ? b1 : zero;
  };
  // the loads of a thread's first item are on their way while the angles are computed
  Item first;
  uint4 first_raw[4];
  const bool has_first = (int)threadIdx.x < items;
  if (has_first) {
    first = item(threadIdx.x);
    load(first, first_raw);
  }
  const int pos = positions[row];
  int page = -1;
  if (k_in != nullptr) page = page_table[(int64_t)seq_slot[seq] * max_blocks + (pos >> HE_PAGE_SHIFT)];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float sn, c;
    sincos_angle((float)pos * inv_freq[i], &sn, &c);
    cs[0][i] = c;
    cs[1][i] = sn;
  }
  __syncthreads();
  const bool cache_ok = page >= 0 && page < num_pages;
  const int off = pos & (HE_PAGE_TOKENS - 1);
  const int KS = he_k_steps(hd);
  auto finish = [&](const Item& im, const uint4 (&raw)[4]) {
    // where the eight elements from dim d on go: the q row, or the cache page in operand order
    uint16_t* out;
    if (im.is_q) {
      out = q_out + row * (int64_t)H * hd + im.h * hd;
    } else {
      if (!cache_ok) return;
      out = kpool + ((int64_t)page * KVH + im.h) * he_k_page_elems(hd);
    }
    auto at = [&](int d) { return out + (im.is_q ? d : he_k_index(off, d, KS)); };
    float x0[8], x1[8], b0[8], b1[8];
    unpack8(raw[0], x0);
    unpack8(raw[2], b0);
    if (im.rotated) {
      unpack8(raw[1], x1);
      unpack8(raw[3], b1);
      float y0[8], y1[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float a0 = x0[i] + b0[i], a1 = x1[i] + b1[i];
        const float c = cs[0][im.j + i], sn = cs[1][im.j + i];
        y0[i] = a0 * c - a1 * sn;
        y1[i] = a0 * sn + a1 * c;
      }
      *reinterpret_cast<uint4*>(at(im.j)) = pack8(y0);
      *reinterpret_cast<uint4*>(at(im.j + half)) = pack8(y1);
    } else {
      if (im.bias) {
#pragma unroll
        for (int i = 0; i < 8; ++i) x0[i] += b0[i];
        *reinterpret_cast<uint4*>(at(im.j)) = pack8(x0);
      } else {
        *reinterpret_cast<uint4*>(at(im.j)) = raw[0];
      }
    }
  };
  if (has_first) finish(first, first_raw);
  for (int it = threadIdx.x + blockDim.x; it < items; it += blockDim.x) {
    const Item im = item(it);
    uint4 raw[4];
    load(im, raw);
    finish(im, raw);
  }
}

extern "C" int he_qkv_rope_cache(void* q_out, void* kpool, void* vpool, const void* q_in,
                                 const void* k_in, const void* v_in, int64_t in_stride,
                                 const void* q_bias, const void* k_bias, const void* v_bias,
                                 int bias_dtype, const void* positions, const void* row_seq,
                                 const void* seq_slot, const void* page_table, int max_blocks,
                                 int num_pages, const void* inv_freq, int rotary_dim, int rows,
                                 int H, int KVH, int hd, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && KVH >= 0 && hd > 0, "he_qkv_rope_cache: bad sizes");
  HE_REQUIRE(rotary_dim >= 0 && rotary_dim <= hd && (rotary_dim & 1) == 0,
             "he_qkv_rope_cache: rotary_dim %d must be even and at most head_dim %d", rotary_dim,
             hd);
  HE_REQUIRE(rotary_dim / 2 <= ROPE_MAX_HALF, "he_qkv_rope_cache: rotary_dim %d above %d",
             rotary_dim, 2 * ROPE_MAX_HALF);
  HE_REQUIRE(rotary_dim == 0 || inv_freq != nullptr, "he_qkv_rope_cache: missing inv_freq");
  HE_REQUIRE((k_in == nullptr) == (v_in == nullptr), "he_qkv_rope_cache: k and v go together");
  HE_REQUIRE(k_in == nullptr || (kpool && vpool && page_table && max_blocks > 0 && KVH > 0),
             "he_qkv_rope_cache: cache arguments missing");
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_qkv_rope_cache: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = 256;
#define ROPE_LAUNCH(T, TI)                                                                      \
  qkv_rope_cache_kernel<T, TI><<<rows, threads, 0, s>>>(                                        \
      (T*)q_out, (T*)kpool, (T*)vpool, (const TI*)q_in, (const TI*)k_in, (const TI*)v_in,       \
      in_stride, q_bias, k_bias, v_bias, bias_dtype,                                            \
      (const int32_t*)positions, (const int32_t*)row_seq, (const int32_t*)seq_slot,             \
      (const int32_t*)page_table, max_blocks, num_pages, (const float*)inv_freq, rotary_dim, H, \
      KVH, hd)
  const bool vec_ok = dtype == HE_BF16 &&
                      (q_bias == nullptr || bias_dtype == HE_BF16) &&
                      ((rotary_dim >> 1) & 7) == 0 && ((hd - rotary_dim) & 7) == 0 &&
                      (in_stride & 7) == 0 && (hd & 7) == 0 &&
                      ((((uintptr_t)q_in) | ((uintptr_t)k_in) | ((uintptr_t)v_in) |
                        ((uintptr_t)q_bias) | ((uintptr_t)k_bias) | ((uintptr_t)v_bias) |
                        ((uintptr_t)q_out) | ((uintptr_t)kpool)) & 15) == 0;
  if (vec_ok) {
    const int items = (H + (k_in ? KVH : 0)) * ((rotary_dim >> 4) + ((hd - rotary_dim) >> 3));
    const int vec_threads = min(1024, max(64, (items + 63) / 64 * 64));
    const int v_blocks = k_in ? (rows + 7) / 8 : 0;
    qkv_rope_cache_vec_kernel<<<rows + v_blocks, vec_threads, 0, s>>>(
        (uint16_t*)q_out, (uint16_t*)kpool, (uint16_t*)vpool, (const uint16_t*)q_in,
        (const uint16_t*)k_in, (const uint16_t*)v_in, in_stride, (const uint16_t*)q_bias,
        (const uint16_t*)k_bias, (const uint16_t*)v_bias, (const int32_t*)positions,
        (const int32_t*)row_seq, (const int32_t*)seq_slot, (const int32_t*)page_table, max_blocks,
        num_pages, (const float*)inv_freq, rotary_dim, rows, H, KVH, hd);
  } else if (dtype == HE_BF16) {
    ROPE_LAUNCH(bf16_t, bf16_t);
  } else {
    ROPE_LAUNCH(float, float);
  }
#undef ROPE_LAUNCH
  return he_check_launch("he_qkv_rope_cache");
}
