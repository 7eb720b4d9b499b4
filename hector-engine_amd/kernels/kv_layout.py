"""Sizes and indices of a cache page (64 tokens of one kv head) as the attention kernels of
this library keep it (the attention part asks the cache for pages of these sizes through its
KVNeed; the cache itself knows no layout): in the order in which the MFMA kernels read their operands, so that every operand
load is one contiguous KiB (csrc/cache_layout.h holds the same formulas for the device).

  K: [half h][key tile t][k step ks][lane = 16 lg + lr][e]   key = 32 h + 8 (lr // 4) + 4 t + lr % 4
                                                             dim = 32 ks + 8 lg + e
  V: [half h][dim tile dt][lane = 16 lg + lr][e]             dim = 16 dt + lr, key = 32 h + 8 lg + e

Head sizes that are no multiple of 32 (K) or 16 (V) leave the rest of their last step or
tile unused."""
from __future__ import annotations

PAGE_TOKENS = 64


def k_steps(head_dim: int) -> int:
    return (head_dim + 31) // 32


def v_tiles(head_dim: int) -> int:
    return (head_dim + 15) // 16


def k_page_elems(head_dim: int) -> int:
    return PAGE_TOKENS * 32 * k_steps(head_dim)


def v_page_elems(head_dim: int) -> int:
    return PAGE_TOKENS * 16 * v_tiles(head_dim)


def k_index(token: int, d: int, head_dim: int) -> int:
    h, kl = token >> 5, token & 31
    t, lr = (kl >> 2) & 1, ((kl >> 3) << 2) | (kl & 3)
    ks, lg, e = d >> 5, (d >> 3) & 3, d & 7
    return ((((h * 2 + t) * k_steps(head_dim) + ks) * 64) + 16 * lg + lr) * 8 + e


def v_index(token: int, d: int, head_dim: int) -> int:
    h, lg, e = token >> 5, (token >> 3) & 3, token & 7
    dt, lr = d >> 4, d & 15
    return ((h * v_tiles(head_dim) + dt) * 64 + 16 * lg + lr) * 8 + e
