"""Bump allocator for the activations of one step (the reference's scratch pool:
one arena, a moving offset, 256-byte alignment, reset - src/memory.cpp:135-161).

Three arenas: one for what lives as long as the step (its metadata, the residual rows,
the logits), and two that the layers take in turn. A layer's arena is reset when the
layer after the next begins, so what a layer hands to its successor (a branch output
not yet added, the rows prepared for the next norm) stays valid while that one runs,
and a step holds the activations of two layers, not of all of them. Inside a layer,
mark() / release() give back the temporaries of a loop's turn.

Tensors handed out are views into an arena and are valid until it is reset. When an
arena is too small, a larger one replaces it (views of the old one stay valid through
their own references) and at the next step it is sized to hold the whole need in one
piece; a pool that backs a captured graph is frozen and must not grow."""
from __future__ import annotations

import torch

ALIGN = 256


class _Arena:
    def __init__(self, device, initial_bytes: int):
        self.device = device
        self.capacity = 0
        self.offset = 0
        self.high = 0            # most bytes in use since the last step began
        self.spilled = 0         # bytes left behind in arenas that were replaced this step
        self.generation = 0
        self.buffer: torch.Tensor | None = None
        self.grow(initial_bytes)

    def grow(self, need: int) -> None:
        self.spilled += self.offset
        self.capacity = max(need, 2 * self.capacity)
        self.buffer = torch.empty(self.capacity, dtype=torch.uint8, device=self.device)
        self.offset = 0
        self.generation += 1

    def clear(self) -> None:
        self.offset = 0

    def new_step(self, may_grow: bool) -> None:
        need = self.high + self.spilled
        if need > self.capacity and may_grow:
            self.capacity = 0
            self.offset = 0
            self.spilled = 0
            self.grow(need + need // 8)
        self.offset = 0
        self.high = 0
        self.spilled = 0


class ScratchPool:
    def __init__(self, device, initial_bytes: int = 1 << 20):
        self.device = device
        self.frozen = False
        self.peak = 0
        self._arenas = [_Arena(device, initial_bytes) for _ in range(3)]   # step, layers in turn
        self._current = 0
        self._turn = 0

    @property
    def capacity(self) -> int:
        return sum(a.capacity for a in self._arenas)

    def reset(self) -> None:
        """Starts a new step."""
        for a in self._arenas:
            a.new_step(not self.frozen)
        self._current = 0
        self._turn = 0

    def begin_layer(self) -> None:
        """Allocations from here on belong to a layer: they live until the layer after the
        next one begins."""
        self._turn ^= 1
        self._current = 1 + self._turn
        self._arenas[self._current].clear()

    def end_layers(self) -> None:
        """Back to allocations that live as long as the step."""
        self._current = 0

    def mark(self):
        a = self._arenas[self._current]
        return (self._current, a.generation, a.offset)

    def release(self, mark) -> None:
        """Gives back everything allocated since mark() (nothing, if the arena was replaced)."""
        index, generation, offset = mark
        a = self._arenas[index]
        if index == self._current and a.generation == generation:
            a.offset = offset

    def alloc(self, shape, dtype: torch.dtype) -> torch.Tensor:
        numel = 1
        for s in shape:
            numel *= int(s)
        nbytes = numel * torch.empty((), dtype=dtype).element_size()
        padded = (nbytes + ALIGN - 1) // ALIGN * ALIGN
        a = self._arenas[self._current]
        if a.offset + padded > a.capacity:
            if self.frozen:
                raise RuntimeError("scratch pool of a captured graph cannot grow")
            a.grow(a.offset + padded)
        view = a.buffer[a.offset:a.offset + nbytes].view(dtype).view(*shape)
        a.offset += padded
        a.high = max(a.high, a.offset)
        self.peak = max(self.peak, sum(x.high + x.spilled for x in self._arenas))
        return view
