"""Writes tests/golden/rng_fixture.json: known answers of this project's own seeded
generators and 16-bit conversions, produced by the pure-Python/numpy restatement below (not
by the C library they pin).  Nothing here touches the reference tree: the reference holds no
golden vectors for this path, and its generators are unseeded.

    python tests/golden/make_fixtures.py
"""
import json
import math
import struct
from pathlib import Path

MASK = (1 << 64) - 1


def mix64(z):
    z = (z + 0x9E3779B97F4A7C15) & MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return z ^ (z >> 31)


def rng_u64(seed, stream, index):
    return mix64((mix64(seed ^ ((stream * 0xD1342543DE82EF95) & MASK)) + index) & MASK)


def f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def bf16_bits(x):
    """float -> bfloat16 bits, round to nearest even, from the binary32 pattern."""
    u = struct.unpack("<I", struct.pack("<f", x))[0]
    if (u & 0x7FFFFFFF) > 0x7F800000:
        return ((u >> 16) | 0x40) & 0xFFFF
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFFFFFF
    return u >> 16


def uniform(seed, stream, i):
    r = rng_u64(seed, stream, i)
    u = f32((r >> 40) * (1.0 / 16777216.0))
    return bf16_bits(f32(2.0 * u - 1.0))


def normal(seed, stream, i, sigma):
    r = rng_u64(seed, stream, i)
    u1 = ((r >> 40) + 1.0) * (1.0 / 16777216.0)
    u2 = (r & 0xFFFFFF) * (1.0 / 16777216.0)
    z = math.sqrt(-2.0 * math.log(u1)) * math.cos(6.283185307179586476925 * u2)
    return bf16_bits(f32(z * float(f32(sigma))))


def randint(seed, stream, i):
    r = rng_u64(seed, stream, i) >> 33
    return bf16_bits(float(r % 1000 * 1 // 100 % 10 - 5.0))


def main():
    n = 64
    out = {
        "seed": 69,
        "u64": [[s, i, rng_u64(69, s, i)] for s in (0, 1, 2) for i in (0, 1, 2, 1 << 20, (1 << 32) + 5)],
        "uniform_stream1": [uniform(69, 1, i) for i in range(n)],
        "uniform_stream2": [uniform(69, 2, i) for i in range(n)],
        "normal_stream1_sigma1": [normal(69, 1, i, 1.0) for i in range(n)],
        "normal_stream2_sigma002": [normal(69, 2, i, 0.02) for i in range(n)],
        "randint_stream1": [randint(69, 1, i) for i in range(n)],
        # bf16 rounding ties and specials: (float32 bits, expected bf16 bits)
        "bf16_cases": [[0x3F808000, 0x3F80], [0x3F818000, 0x3F82], [0x3F808001, 0x3F81],
                       [0x3F80FFFF, 0x3F81], [0x7F800000, 0x7F80], [0xFF800000, 0xFF80],
                       [0x7FC00000, 0x7FC0], [0x7F800001, 0x7FC0], [0x80000000, 0x8000],
                       [0x7F7FFFFF, 0x7F80], [0x00008000, 0x0000], [0x00018000, 0x0002]],
    }
    path = Path(__file__).with_name("rng_fixture.json")
    path.write_text(json.dumps(out, indent=1))
    print("wrote", path)


if __name__ == "__main__":
    main()
