"""TEST INFRASTRUCTURE: XXH3-128 (seed 0, default secret), restated in numpy (long inputs) and plain integers (the
forms for 0..240 bytes).

The reference's delta publisher digests every changed tensor with ``checksum("xxh3-128", new)``
(slime/utils/disk_delta.py:40-58, default of --update-weight-delta-checksum, slime/utils/arguments.py:186-188), i.e.
``xxhash.xxh3_128(data).hexdigest()`` from the third-party ``xxhash`` package (xxHash 0.8.x).  The algorithm restated
here is the published one (xxhash.h: XXH3_hashLong_128b, XXH3_accumulate_512 / XXH3_scrambleAcc scalar forms,
XXH3_mergeAccs, XXH3_avalanche).  Pinned against the ``xxhash`` package itself, which is installed
(tests/test_oracle_xxh3.py): every length around the block and stripe boundaries and random inputs.

The point of the restatement is its shape: the accumulation over the 16 stripes of a 1 KiB block is a plain sum
(``block_sums``: parallel over blocks), only the scramble between blocks is sequential (``chain``) - the split the
GPU kernels use.
"""

from __future__ import annotations

import numpy as np

SECRET = bytes([
    0xb8, 0xfe, 0x6c, 0x39, 0x23, 0xa4, 0x4b, 0xbe, 0x7c, 0x01, 0x81, 0x2c, 0xf7, 0x21, 0xad, 0x1c,
    0xde, 0xd4, 0x6d, 0xe9, 0x83, 0x90, 0x97, 0xdb, 0x72, 0x40, 0xa4, 0xa4, 0xb7, 0xb3, 0x67, 0x1f,
    0xcb, 0x79, 0xe6, 0x4e, 0xcc, 0xc0, 0xe5, 0x78, 0x82, 0x5a, 0xd0, 0x7d, 0xcc, 0xff, 0x72, 0x21,
    0xb8, 0x08, 0x46, 0x74, 0xf7, 0x43, 0x24, 0x8e, 0xe0, 0x35, 0x90, 0xe6, 0x81, 0x3a, 0x26, 0x4c,
    0x3c, 0x28, 0x52, 0xbb, 0x91, 0xc3, 0x00, 0xcb, 0x88, 0xd0, 0x65, 0x8b, 0x1b, 0x53, 0x2e, 0xa3,
    0x71, 0x64, 0x48, 0x97, 0xa2, 0x0d, 0xf9, 0x4e, 0x38, 0x19, 0xef, 0x46, 0xa9, 0xde, 0xac, 0xd8,
    0xa8, 0xfa, 0x76, 0x3f, 0xe3, 0x9c, 0x34, 0x3f, 0xf9, 0xdc, 0xbb, 0xc7, 0xc7, 0x0b, 0x4f, 0x1d,
    0x8a, 0x51, 0xe0, 0x4b, 0xcd, 0xb4, 0x59, 0x31, 0xc8, 0x9f, 0x7e, 0xc9, 0xd9, 0x78, 0x73, 0x64,
    0xea, 0xc5, 0xac, 0x83, 0x34, 0xd3, 0xeb, 0xc3, 0xc5, 0x81, 0xa0, 0xff, 0xfa, 0x13, 0x63, 0xeb,
    0x17, 0x0d, 0xdd, 0x51, 0xb7, 0xf0, 0xda, 0x49, 0xd3, 0x16, 0x55, 0x26, 0x29, 0xd4, 0x68, 0x9e,
    0x2b, 0x16, 0xbe, 0x58, 0x7d, 0x47, 0xa1, 0xfc, 0x8f, 0xf8, 0xb8, 0xd1, 0x7a, 0xd0, 0x31, 0xce,
    0x45, 0xcb, 0x3a, 0x8f, 0x95, 0x16, 0x04, 0x28, 0xaf, 0xd7, 0xfb, 0xca, 0xbb, 0x4b, 0x40, 0x7e,
])
P32_1, P32_2, P32_3 = 0x9E3779B1, 0x85EBCA77, 0xC2B2AE3D
P64_1, P64_2, P64_3 = 0x9E3779B185EBCA87, 0xC2B2AE3D27D4EB4F, 0x165667B19E3779F9
P64_4, P64_5 = 0x85EBCA77C2B2AE63, 0x27D4EB2F165667C5
PRIME_MX1 = 0x165667919E3779F9
INIT_ACC = (P32_3, P64_1, P64_2, P64_3, P64_4, P32_2, P64_5, P32_1)
STRIPE, BLOCK, STRIPES_PER_BLOCK = 64, 1024, 16
M64 = (1 << 64) - 1


def secret64(offset: int, count: int = 8) -> np.ndarray:
    """``count`` little-endian u64 read from the secret at ``offset`` (any alignment)."""
    return np.frombuffer(SECRET[offset:offset + 8 * count], dtype="<u8").copy()


def stripe_terms(stripe: np.ndarray, key: np.ndarray) -> np.ndarray:
    """What one 64-byte stripe adds to the eight accumulators (XXH3_scalarRound): lane i gets the product of the two
    halves of data[i] ^ key[i], and the data word of its neighbour i ^ 1.  stripe, key: u64 [..., 8]."""
    mixed = stripe ^ key
    prod = (mixed & np.uint64(0xFFFFFFFF)) * (mixed >> np.uint64(32))
    return prod + stripe[..., [1, 0, 3, 2, 5, 4, 7, 6]]


def block_sums(data: np.ndarray, n_blocks: int) -> np.ndarray:
    """Sum of the stripe terms of each of the first ``n_blocks`` 1 KiB blocks -> u64 [n_blocks, 8].  No dependence
    between blocks: this is the part a GPU does at memory speed."""
    words = np.frombuffer(data[:n_blocks * BLOCK].tobytes(), dtype="<u8").reshape(n_blocks, STRIPES_PER_BLOCK, 8)
    keys = np.stack([secret64(8 * s) for s in range(STRIPES_PER_BLOCK)])          # stripe s reads the secret at 8 s
    with np.errstate(over="ignore"):
        return stripe_terms(words, keys[None]).sum(axis=1, dtype=np.uint64)


def chain(sums: np.ndarray) -> np.ndarray:
    """acc <- scramble(acc + sums[k]) for every block in order (XXH3_scalarScrambleRound with the secret at 128)."""
    acc = np.array(INIT_ACC, dtype=np.uint64)
    key = secret64(len(SECRET) - STRIPE)
    with np.errstate(over="ignore"):
        for s in sums:
            acc = acc + s
            acc = ((acc ^ (acc >> np.uint64(47))) ^ key) * np.uint64(P32_1)
    return acc


def _mul128_fold64(a: int, b: int) -> int:
    p = a * b
    return (p & M64) ^ (p >> 64)


def _avalanche(h: int) -> int:
    h ^= h >> 37
    h = (h * PRIME_MX1) & M64
    return h ^ (h >> 32)


def _merge(acc, offset: int, start: int) -> int:
    key = secret64(offset)
    r = start
    for i in range(4):
        r = (r + _mul128_fold64(int(acc[2 * i]) ^ int(key[2 * i]), int(acc[2 * i + 1]) ^ int(key[2 * i + 1]))) & M64
    return _avalanche(r)


PRIME_MX2 = 0x9FB21C651E98DF25


def _s64(off: int) -> int:
    return int.from_bytes(SECRET[off:off + 8], "little")


def _s32(off: int) -> int:
    return int.from_bytes(SECRET[off:off + 4], "little")


def _le(b: bytes, off: int, size: int) -> int:
    return int.from_bytes(b[off:off + size], "little")


def _xxh64_avalanche(h: int) -> int:
    h ^= h >> 33
    h = (h * P64_2) & M64
    h ^= h >> 29
    h = (h * P64_3) & M64
    return h ^ (h >> 32)


def _mix16(b: bytes, off: int, soff: int) -> int:
    return _mul128_fold64(_le(b, off, 8) ^ _s64(soff), _le(b, off + 8, 8) ^ _s64(soff + 8))


def _mix32(acc, b: bytes, o1: int, o2: int, soff: int):
    low, high = acc
    low = (low + _mix16(b, o1, soff)) & M64
    low ^= (_le(b, o2, 8) + _le(b, o2 + 8, 8)) & M64
    high = (high + _mix16(b, o2, soff + 16)) & M64
    high ^= (_le(b, o1, 8) + _le(b, o1 + 8, 8)) & M64
    return low, high


def _finish_mid(acc, n: int) -> tuple[int, int]:
    low, high = acc
    h_low = (low + high) & M64
    h_high = (low * P64_1 + high * P64_4 + n * P64_2) & M64
    return _avalanche(h_low), (-_avalanche(h_high)) & M64


def xxh3_128_short(b: bytes) -> tuple[int, int]:
    """The forms for inputs of 0..240 bytes (XXH3_len_0to16_128b, _17to128_128b, _129to240_128b; seed 0)."""
    n = len(b)
    if n == 0:
        return _xxh64_avalanche(_s64(64) ^ _s64(72)), _xxh64_avalanche(_s64(80) ^ _s64(88))
    if n <= 3:
        lo = (b[0] << 16) | (b[n >> 1] << 24) | b[n - 1] | (n << 8)
        swapped = int.from_bytes(lo.to_bytes(4, "little"), "big")
        hi = ((swapped << 13) | (swapped >> 19)) & 0xFFFFFFFF
        return _xxh64_avalanche(lo ^ (_s32(0) ^ _s32(4))), _xxh64_avalanche(hi ^ (_s32(8) ^ _s32(12)))
    if n <= 8:
        keyed = (_le(b, 0, 4) + (_le(b, n - 4, 4) << 32)) ^ (_s64(16) ^ _s64(24))
        p = keyed * (P64_1 + (n << 2))
        low, high = p & M64, p >> 64
        high = (high + (low << 1)) & M64
        low ^= high >> 3
        low ^= low >> 35
        low = (low * PRIME_MX2) & M64
        low ^= low >> 28
        return low, _avalanche(high)
    if n <= 16:
        in_lo, in_hi = _le(b, 0, 8), _le(b, n - 8, 8)
        p = (in_lo ^ in_hi ^ (_s64(32) ^ _s64(40))) * P64_1
        low, high = p & M64, p >> 64
        low = (low + ((n - 1) << 54)) & M64
        in_hi ^= _s64(48) ^ _s64(56)
        high = (high + in_hi + (in_hi & 0xFFFFFFFF) * (P32_2 - 1)) & M64
        low ^= int.from_bytes(high.to_bytes(8, "little"), "big")
        q = low * P64_2
        return _avalanche(q & M64), _avalanche(((q >> 64) + high * P64_2) & M64)
    acc = ((n * P64_1) & M64, 0)
    if n <= 128:
        for i in range((n - 1) // 32, -1, -1):
            acc = _mix32(acc, b, 16 * i, n - 16 * (i + 1), 32 * i)
        return _finish_mid(acc, n)
    for i in range(32, 160, 32):
        acc = _mix32(acc, b, i - 32, i - 16, i - 32)
    acc = (_avalanche(acc[0]), _avalanche(acc[1]))
    for i in range(160, n + 1, 32):
        acc = _mix32(acc, b, i - 32, i - 16, 3 + i - 160)
    acc = _mix32(acc, b, n - 16, n - 32, 136 - 17 - 16)
    return _finish_mid(acc, n)


def xxh3_128(data) -> tuple[int, int]:
    """-> (low64, high64) of XXH3_128bits(data)."""
    data = np.frombuffer(bytes(data), dtype=np.uint8)
    n = data.size
    if n <= 240:
        return xxh3_128_short(data.tobytes())
    n_blocks = (n - 1) // BLOCK
    acc = chain(block_sums(data, n_blocks))
    with np.errstate(over="ignore"):
        tail = n_blocks * BLOCK
        for s in range(((n - 1) - tail) // STRIPE):                                # whole stripes of the last block
            w = np.frombuffer(data[tail + s * STRIPE: tail + (s + 1) * STRIPE].tobytes(), dtype="<u8")
            acc = acc + stripe_terms(w, secret64(8 * s))
        w = np.frombuffer(data[n - STRIPE:].tobytes(), dtype="<u8")                # the last 64 bytes, whatever they overlap
        acc = acc + stripe_terms(w, secret64(len(SECRET) - STRIPE - 7))
    low = _merge(acc, 11, (n * P64_1) & M64)
    high = _merge(acc, len(SECRET) - STRIPE - 11, ~(n * P64_2) & M64)
    return low, high


def hexdigest(data) -> str:
    """The string ``xxhash.xxh3_128(data).hexdigest()`` returns: the 128-bit value, most significant byte first."""
    low, high = xxh3_128(data)
    return f"{high:016x}{low:016x}"
