"""Counter-based uniforms: one 32-bit draw per (seed, sequence, step), so what a
sequence samples does not depend on the batch it runs in or on the order of the
batch. (The reference draws one uniform per token from a host mt19937_64:
src/sampler.hpp:129-130, src/sampler.cpp:186.)"""
from __future__ import annotations

_M = (1 << 64) - 1


def uniform_u32(seed: int, sequence: int, step: int) -> int:
    z = (seed * 0x9E3779B97F4A7C15 + sequence * 0xBF58476D1CE4E5B9
         + step * 0x94D049BB133111EB + 0x2545F4914F6CDD1D) & _M
    z ^= z >> 30
    z = (z * 0xBF58476D1CE4E5B9) & _M
    z ^= z >> 27
    z = (z * 0x94D049BB133111EB) & _M
    z ^= z >> 31
    return z >> 32
