"""xoshiro256** seeded through SplitMix64, the reference's generator
(crates/runtime/src/sampling.rs:112-149): ``next_f32 = (next_u64 >> 40) / 2^24`` in [0, 1)."""
from __future__ import annotations

_MASK = (1 << 64) - 1


def _rotl(x: int, k: int) -> int:
    return ((x << k) | (x >> (64 - k))) & _MASK


class Xoshiro256:
    __slots__ = ("s",)

    def __init__(self, seed: int):
        x = (seed + 0x9E3779B97F4A7C15) & _MASK
        s = []
        for _ in range(4):
            x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
            x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
            s.append(x ^ (x >> 31))
        if not any(s):
            s[0] = 1
        self.s = s

    def next_u64(self) -> int:
        s0, s1, s2, s3 = self.s
        result = (_rotl((s1 * 5) & _MASK, 7) * 9) & _MASK
        t = (s1 << 17) & _MASK
        s2 ^= s0
        s3 ^= s1
        s1 ^= s2
        s0 ^= s3
        s2 ^= t
        s3 = _rotl(s3, 45)
        self.s = [s0, s1, s2, s3]
        return result

    def next_f32(self) -> float:
        return (self.next_u64() >> 40) * (1.0 / (1 << 24))
