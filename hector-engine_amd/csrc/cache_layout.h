// Where a key or value element lies inside a cache page of 64 tokens of one kv head.
//
// A page is stored in the order in which the MFMA attention kernels read it: for a step of
// 32 keys, the K operand of key tile t and k step ks (16 keys x 32 head dims) and the V^T
// operand of dim tile dt (16 head dims x 32 keys) are each one contiguous KiB, lane l's
// eight elements at 16 l bytes. A wavefront's operand load is then one fully coalesced
// access and every 128-byte line is asked for once; with pages stored as tokens x head
// size, a load touches 16 rows x 64 bytes and every line is asked for twice (measured:
// 7-9 % of the one-token attention's time). A page can also be copied into LDS as it is.
//
//   K: [half h][key tile t][k step ks][lane = 16 lg + lr][e]   key = 32 h + 8 (lr / 4) + 4 t + lr % 4
//                                                              dim = 32 ks + 8 lg + e
//   V: [half h][dim tile dt][lane = 16 lg + lr][e]             dim = 16 dt + lr, key = 32 h + 8 lg + e
//
// (the keys of a K tile are interleaved so that the scores a lane holds after the first
// product are the eight consecutive keys its V^T operand needs). Head sizes that are no
// multiple of 32 (K) or 16 (V) leave the rest of their last step or tile unused.
#pragma once
#include "common.h"

__host__ __device__ __forceinline__ int he_k_steps(int hd) { return (hd + 31) >> 5; }
__host__ __device__ __forceinline__ int he_v_tiles(int hd) { return (hd + 15) >> 4; }
// elements of one page of one kv head
__host__ __device__ __forceinline__ int he_k_page_elems(int hd) { return HE_PAGE_TOKENS * 32 * he_k_steps(hd); }
__host__ __device__ __forceinline__ int he_v_page_elems(int hd) { return HE_PAGE_TOKENS * 16 * he_v_tiles(hd); }

// token: 0..63 inside the page, d: head dim; KS = he_k_steps(hd). Eight dims from a multiple
// of 8 on are contiguous.
__host__ __device__ __forceinline__ int he_k_index(int token, int d, int KS) {
  const int h = token >> 5, kl = token & 31;
  const int t = (kl >> 2) & 1, lr = ((kl >> 3) << 2) | (kl & 3);
  const int ks = d >> 5, lg = (d >> 3) & 3, e = d & 7;
  return ((((h * 2 + t) * KS + ks) * 64) + 16 * lg + lr) * 8 + e;
}
// NT = he_v_tiles(hd). Eight tokens from a multiple of 8 on are contiguous.
__host__ __device__ __forceinline__ int he_v_index(int token, int d, int NT) {
  const int h = token >> 5, lg = (token >> 3) & 3, e = token & 7;
  const int dt = d >> 4, lr = d & 15;
  return ((h * NT + dt) * 64 + 16 * lg + lr) * 8 + e;
}
