// C ABI of the gfx950 kernel library. Every function launches on the given HIP
// stream and returns 0, or non-zero after recording a message for
// he_last_error(). Pointers are device pointers unless named host_*. Shapes
// are validated on the host before any launch. dtype codes: 0 = float32,
// 1 = bfloat16 (2 = float16, as the input of he_cast only).
#pragma once
#include <stdint.h>

#define HE_ABI_VERSION 20

#ifdef __cplusplus
extern "C" {
#endif

const char* he_last_error(void);
int he_abi_version(void);

// ---- weight preparation ----------------------------------------------------
// out[i] = bf16(quantiles[16 bits of the counter-based word of (key, i)] * std + mean), stored as
// `dtype`; quantiles_f32: 65536 quantiles of the standard normal distribution (device pointer).
int he_fill_random(void* out, int64_t n, int dtype, uint64_t key, const void* quantiles_f32,
                   float mean, float std, void* stream);
// out[i] = uniform integer in [0, high) from the counter-based word of (key, i).
int he_fill_random_integers(void* out_i32, int64_t n, uint64_t key, int64_t high, void* stream);
// out = in converted (in: float32, bfloat16 or float16; out: float32 or bfloat16, nearest even).
int he_cast(void* out, const void* in, int64_t n, int in_dtype, int out_dtype, void* stream);

// ---- row-wise ------------------------------------------------------------
int he_embedding(void* out_f32, const void* table, const void* ids, int rows, int D, int V,
                 int table_dtype, void* stream);
int he_gather_rows_f32(void* out, const void* src, const void* rows, int n_out, int D, int n_src,
                       void* stream);
int he_residual_add(void* resid_f32, const void* delta, int64_t n, int delta_dtype, void* stream);
// splits > 0: gate_up is fp32 [splits][rows][2I], the K slices of the product.
int he_silu_mul(void* out, const void* gate_up, int rows, int I, int interleaved, int splits,
                int dtype, void* stream);

// ---- norms ---------------------------------------------------------------
// resid (fp32, in place) += delta (may be null); out (may be null) = rmsnorm(resid) * weight.
int he_add_rmsnorm(void* resid_f32, const void* delta, const void* weight, void* out, int rows, int D,
                   float eps, int act_dtype, int w_dtype, void* stream);
int he_rmsnorm_rows(void* out, const void* x, const void* weight, int rows, int D,
                    int64_t x_stride, int64_t out_stride, float eps, int dtype, int w_dtype,
                    void* stream);

// ---- matrix products: C[M,N] = A[M,K] * W[N,K]^T (+ bias) -------------------
// he_gemm_plain: fp32 FMA sums in one fixed order per element (segments of 128 k, each a chain in
// ascending k, added in segment order). With a workspace of he_gemm_plain_workspace_floats(M, N, K)
// floats (0 for more than 8 rows) a product of few rows runs through kernels made for it; the
// result is the same bit for bit.
int64_t he_gemm_plain_workspace_floats(int M, int N, int K);
int he_gemm_plain(void* C, const void* A, const void* W, const void* bias, int M, int N, int K,
                  int64_t lda, int64_t ldw, int64_t ldc, int in_dtype, int out_dtype,
                  int bias_dtype, void* workspace_f32, int64_t workspace_floats, void* stream);
// bf16 MFMA product for M <= HE_BLOCKSPLIT_MAX_M with K cut inside the workgroup (NW
// wavefronts, one slice each, added in LDS): complete in one launch.
#define HE_BLOCKSPLIT_MAX_M 32
int he_gemm_blocksplit_bf16(void* C, const void* A, const void* W, const void* bias, int M, int N,
                            int K, int out_dtype, int bias_dtype, int gated, int R, int U, int NW,
                            void* stream);
// The same with an RMS norm carried across a pair of products. resid != null: the residual
// epilogue (resid[M,N] fp32 += result in place, xg[M,N] bf16 = resid * gain, sq_out[M, sq_count]
// = sums of resid^2 per workgroup, sq_count = he_gemm_blocksplit_blocks). scale_partials != null:
// the rows of A are such xg rows; the result is scaled by 1/sqrt(sum(partials)/K + eps) per row.
// x_pieces / out_pieces (M <= 16): A, or the bf16 output (C, or xg), lies piece-major: a [M, D] tensor as
// 16-byte pieces [D / 8][M][8], element (m, d) at ((d / 8) M + m) 8 + d % 8.
int he_gemm_blocksplit_blocks(int M, int N, int K);
int he_gemm_blocksplit_fused_bf16(void* C, const void* A, const void* W, const void* bias, int M,
                                  int N, int K, int out_dtype, int bias_dtype, int gated, int R,
                                  int U, int NW, const void* scale_partials, int scale_count,
                                  float scale_eps, void* resid, const void* gain, int gain_dtype,
                                  void* xg, void* sq_out, int sq_count, int x_pieces, int out_pieces,
                                  void* stream);
// out = x / sqrt(sum(partials of the row)/D + eps): such xg rows as a normalised tensor
// (row-major; x_pieces: x lies piece-major for exactly `rows` rows).
int he_scale_rows_bf16(void* out, const void* x, const void* partials, int count, int rows, int D,
                       float eps, int x_pieces, void* stream);
// C[M,N] = the slices of partial_f32 [splits][M][N] added in index order (+ bias).
int he_splitk_reduce(void* C, const void* partial_f32, const void* bias, int M, int N, int splits,
                     int out_dtype, int bias_dtype, void* stream);
// bf16 MFMA product for M <= HE_GEMM_ROWS_MAX_M rows whose activation rows are shared through LDS
// by the wavefronts of a workgroup (made for 17 to 64 rows), with the epilogues of
// he_gemm_blocksplit_fused_bf16 (x_pieces / out_pieces for any M here). R (1, 2), NWV (4, 8),
// splits <= 0: the heuristic. A product the plan cuts into several K slices (he_gemm_rows_plan
// says how many) writes fp32 [slices][M][N] into partial_f32 (each slice already scaled by the owed
// row scale) and takes no other epilogue; he_splitk_reduce or he_splitk_reduce_residual adds them.
// With one slice and resid != null, sq_count must be the plan's `groups`.
#define HE_GEMM_ROWS_MAX_M 64
int he_gemm_rows_plan(int M, int N, int K, int* groups, int* splits);
int he_gemm_rows_bf16(void* C, void* partial_f32, int64_t partial_floats, const void* A, const void* W,
                      const void* bias, int M, int N, int K, int out_dtype, int bias_dtype, int gated,
                      int R, int NWV, int splits, const void* scale_partials, int scale_count,
                      float scale_eps, void* resid, const void* gain, int gain_dtype, void* xg,
                      void* sq_out, int sq_count, int x_pieces, int out_pieces, int* splits_used,
                      void* stream);
// resid[M,N] (fp32, in place) += the slices of partial_f32 [splits][M][N] in index order (+ bias);
// xg = bf16(resid * gain) (piece-major with out_pieces); sq_out[M, sq_count] = sums of resid^2 per
// block of 1024 columns (sq_count = he_splitk_reduce_residual_blocks(N)): the rows a residual
// epilogue leaves for the next norm.
int he_splitk_reduce_residual_blocks(int N);
int he_splitk_reduce_residual(void* resid_f32, const void* partial_f32, const void* bias, int bias_dtype,
                              const void* gain, int gain_dtype, void* xg, void* sq_out, int sq_count,
                              int M, int N, int splits, int out_pieces, void* stream);

// ---- position encoding + cache write -------------------------------------
int he_qkv_rope_cache(void* q_out, void* kpool, void* vpool, const void* q_in, const void* k_in,
                      const void* v_in, int64_t in_stride, const void* q_bias, const void* k_bias,
                      const void* v_bias, int bias_dtype, const void* positions,
                      const void* row_seq, const void* seq_slot, const void* page_table,
                      int max_blocks, int num_pages, const void* inv_freq, int rotary_dim, int rows,
                      int H, int KVH, int hd, int dtype, void* stream);

// ---- attention over the paged cache ----------------------------------------
// he_attention_plain: fp32 sums in one fixed order per (query, head): page by page (64 positions),
// inside a page key by key with an online softmax begun afresh, the pages joined in ascending
// position. most_keys: no sequence holds more keys after the step. With a workspace of
// he_attention_plain_workspace_floats floats (0 for a step of many queries) the pages of a query
// run in parallel and a second kernel joins them; the result is the same bit for bit.
int64_t he_attention_plain_workspace_floats(int rows, int H, int hd, int most_keys, int window);
int he_attention_plain(void* out, const void* q, const void* kpool, const void* vpool,
                       const void* positions, const void* row_seq, const void* seq_slot,
                       const void* page_table, int max_blocks, int num_pages, int rows, int H,
                       int KVH, int hd, int window, float scale, int dtype, int most_keys,
                       void* workspace_f32, int64_t workspace_floats, void* stream);
// bf16, one query row per sequence (decode): split over the keys, then merged.
int he_attention_decode_bf16(void* out, const void* q, const void* kpool, const void* vpool,
                             const void* positions, const void* row_seq, const void* seq_slot,
                             const void* page_table, int max_blocks, int num_pages, int rows,
                             int H, int KVH, int hd, int window, float scale, int max_keys,
                             void* workspace_f32, int64_t workspace_floats, void* stream);
int64_t he_attention_decode_workspace_floats(int rows, int H, int KVH, int hd, int max_keys);
// bf16, one query row per sequence, one launch for bias + rotary + cache write + attention +
// merge (a second launch joins the parts where few sequences are cut across workgroups).
// qkv: the un-biased projection rows [rows, (H + 2 KVH) hd]. he_attention_decode_fused_ok: 1
// when the sizes are taken (head_dim 64 or 128, rotated whole). out_pieces: out lies piece-major
// (as he_gemm_blocksplit_fused_bf16 reads it with x_pieces). spread: one sequence of the step has
// several times the keys of the others; every sequence's keys are then cut across more workgroups.
// seq_slot null: page_table has a row per row of the step ([rows, max_blocks], the page numbers of
// the row's sequence) instead of a row per slot. qkv null: the projection rows come as the fp32
// sums of their K slices, qkv_part [qkv_slices][.][qkv_stride] with qkv_slice_stride elements from
// slice to slice (what he_gemm_rows_bf16 leaves when it cuts a product along K); the kernel adds
// them in slice order and rounds to bfloat16, the bits he_splitk_reduce would have written.
int he_attention_decode_fused_ok(int H, int KVH, int hd, int rotary_dim);
int64_t he_attention_decode_fused_workspace_floats(int rows, int H, int KVH, int hd, int max_keys,
                                                   int spread);
int he_attention_decode_fused_bf16(void* out, const void* qkv, const void* qkv_part, int qkv_slices,
                                   int64_t qkv_slice_stride, int64_t qkv_stride, const void* bias,
                                   int bias_dtype, void* kpool, void* vpool, const void* positions,
                                   const void* row_seq, const void* seq_slot,
                                   const void* page_table, int max_blocks, int num_pages,
                                   const void* inv_freq, int rotary_dim, int rows, int H, int KVH,
                                   int hd, int window, float scale, int max_keys, int spread,
                                   int write_kv, int out_pieces, void* workspace_f32,
                                   int64_t workspace_floats,
                                   void* stream);
// bf16, prompt steps: tiles of queries of one sequence against its cache rows. kernel: 0 leaves
// the choice to the library; 1: 16 queries a wavefront, operands straight from global memory
// (any head size up to 256); 2: 32 queries a wavefront, pages shared through LDS, the softmax
// beside the matrix products (head sizes up to 128). parts > 1 (kernel 2 only): the keys of a
// block of queries are cut into that many parts that run side by side and are joined by a
// second launch; the workspace holds he_attention_prefill_workspace_floats() floats.
// he_attention_prefill_parts() is the number the library would take for a step.
int he_attention_prefill_parts(int num_seqs, int max_q_len, int H, int hd, int most_keys);
int64_t he_attention_prefill_workspace_floats(int total_rows, int H, int hd, int parts);
int he_attention_prefill_bf16(void* out, const void* q, const void* kpool, const void* vpool,
                              const void* cu_seqlens, const void* seq_slot, const void* seq_start,
                              const void* page_table, int max_blocks, int num_pages, int num_seqs,
                              int max_q_len, int H, int KVH, int hd, int window, float scale,
                              int kernel, int total_rows, int parts, void* workspace_f32,
                              int64_t workspace_floats, void* stream);

// ---- sampling ------------------------------------------------------------
int64_t he_argmax_workspace_bytes(int rows, int V);
int he_argmax_rows(void* out_i32, const void* logits_f32, int rows, int V, int64_t row_stride,
                   void* workspace, int64_t workspace_bytes, void* stream);
// Not in the reference: an argmax for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). The same kernels as
// he_argmax_rows, with the parts of the rows in a static device array of
// HE_ARGMAX_STATIC_SCRATCH_BYTES per GPU in place of a workspace; it calls no hipMalloc / hipFree
// and no allocating library routine. Inputs needing more scratch (rows * ceil(V / 8192) * 8
// bytes) are refused with an error. All calls on one GPU share that GPU's array: calls that
// overlap on one GPU (two streams, two threads) race; calls on one stream do not.
// he_argmax_rows_static_setup looks up the current device's copy of the array (once per device;
// the first call of he_argmax_rows_static on a device does the same), e.g. before a capture.
#define HE_ARGMAX_STATIC_SCRATCH_BYTES 65536
int he_argmax_rows_static_setup(void);
int he_argmax_rows_static(void* out_i32, const void* logits_f32, int rows, int V,
                          int64_t row_stride, void* stream);
int he_apply_penalties(void* logits_f32, int rows, int V, int64_t row_stride, const void* ids,
                       const void* counts, const void* offsets, float rep, float freq, float pres,
                       void* stream);
// The penalties of he_apply_penalties from a ring of recent tokens on the device: window [rows][W]
// (token number n at n % W), appended [rows] = tokens ever appended. last_ids (or null) are appended
// first, one a row. W up to 4096.
int he_apply_penalties_window(void* logits_f32, int rows, int V, int64_t row_stride, void* window_i32,
                              void* appended_i32, int W, const void* last_ids_i32, float rep, float freq,
                              float pres, void* stream);
int he_sample_rows(void* out_i32, const void* logits_f32, int rows, int V, int64_t row_stride,
                   const void* uniforms_u32, float temperature, int top_k, float top_p,
                   void* stream);

#ifdef __cplusplus
}
#endif
