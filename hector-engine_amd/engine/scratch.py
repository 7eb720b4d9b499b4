"""Bump allocator for the activations of one step (the reference's scratch pool:
one arena, a moving offset, 256-byte alignment, reset - src/memory.cpp:135-161).
Tensors handed out are views into the arena and are valid until the next
reset(). When a step needs more than the arena holds, a larger arena replaces
it (views of the old one stay valid through their own references); a pool that
backs a captured graph is frozen and must not grow."""
from __future__ import annotations

import torch

ALIGN = 256


class ScratchPool:
    def __init__(self, device, initial_bytes: int = 1 << 20):
        self.device = device
        self.capacity = 0
        self.offset = 0
        self.peak = 0
        self.step_total = 0
        self.frozen = False
        self._arena: torch.Tensor | None = None
        self._grow(initial_bytes)

    def _grow(self, need: int) -> None:
        if self.frozen:
            raise RuntimeError("scratch pool of a captured graph cannot grow")
        self.capacity = max(need, 2 * self.capacity)
        self._arena = torch.empty(self.capacity, dtype=torch.uint8, device=self.device)
        self.offset = 0

    def reset(self) -> None:
        """Starts a new step. If the last step outgrew the arena on its way, the arena
        is made large enough to hold a whole such step in one piece."""
        if self.step_total > self.capacity and not self.frozen:
            self.capacity = 0
            self._grow(self.step_total + self.step_total // 8)
        self.offset = 0
        self.step_total = 0

    def alloc(self, shape, dtype: torch.dtype) -> torch.Tensor:
        numel = 1
        for s in shape:
            numel *= int(s)
        nbytes = numel * torch.empty((), dtype=dtype).element_size()
        padded = (nbytes + ALIGN - 1) // ALIGN * ALIGN
        if self.offset + padded > self.capacity:
            self._grow(self.offset + padded)
        view = self._arena[self.offset:self.offset + nbytes].view(dtype).view(*shape)
        self.offset += padded
        self.step_total += padded
        self.peak = max(self.peak, self.step_total)
        return view
