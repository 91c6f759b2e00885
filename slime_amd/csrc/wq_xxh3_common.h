// The pieces of XXH3's long-input form that more than one kernel uses: the default secret, the primes, and the sums of
// one 1 KiB block held by one wavefront (lane l = words 2j, 2j+1 of stripe l / 4, j = l % 4).
#pragma once

#include "wq_common.h"

namespace wq {

static __constant__ __align__(16) uint8_t kXxh3Secret[192] = {
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
};

constexpr uint64_t kP32_1 = 0x9E3779B1ull, kP32_2 = 0x85EBCA77ull, kP32_3 = 0xC2B2AE3Dull;
constexpr uint64_t kP64_1 = 0x9E3779B185EBCA87ull, kP64_2 = 0xC2B2AE3D27D4EB4Full, kP64_3 = 0x165667B19E3779F9ull;
constexpr uint64_t kP64_4 = 0x85EBCA77C2B2AE63ull, kP64_5 = 0x27D4EB2F165667C5ull, kMx1 = 0x165667919E3779F9ull;
constexpr int kXxhBlock = 1024, kXxhStripe = 64;

// little-endian u64 of the secret at any byte offset
__device__ __forceinline__ uint64_t secret64(int off)
{
    uint64_t v = 0;
#pragma unroll
    for (int b = 0; b < 8; ++b) v |= (uint64_t)kXxh3Secret[off + b] << (8 * b);
    return v;
}

__device__ __forceinline__ uint64_t load64_bytes(const uint8_t* p)
{
    uint64_t v = 0;
#pragma unroll
    for (int b = 0; b < 8; ++b) v |= (uint64_t)ldg<uint8_t>(p + b) << (8 * b);
    return v;
}

__device__ __forceinline__ uint64_t mul_halves(uint64_t x) { return (x & 0xFFFFFFFFull) * (x >> 32); }

__device__ __forceinline__ int64_t scrambled_blocks(int64_t n) { return (n - 1) / kXxhBlock; }

// The two secret words a lane of a block meets: stripe s reads the secret at 8 s, so word i of the stripe meets the
// secret's u64 number s + i - an aligned load.
__device__ __forceinline__ void xxh3_lane_keys(int lane, uint64_t& k0, uint64_t& k1)
{
    const uint64_t* words = (const uint64_t*)kXxh3Secret;
    const int first = (lane >> 2) + 2 * (lane & 3);
    k0 = words[first];
    k1 = words[first + 1];
}

// v + (v of the lane 4 further on in the 16-lane row) + ... : the sum over the four lanes of a row that share lane % 4,
// by two rotations of the row (DPP row_ror:4, row_ror:8)
__device__ __forceinline__ uint64_t row_sum_stride4_u64(uint64_t v)
{
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    v += ((uint64_t)dpp_u32<0x124>(hi) << 32) | dpp_u32<0x124>(lo);
    lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    v += ((uint64_t)dpp_u32<0x128>(hi) << 32) | dpp_u32<0x128>(lo);
    return v;
}

// v + (v of the lane 32 away), then + (v of the lane 16 away): with the rotations above, the sum over all sixteen lanes
// of the wavefront that share lane % 4, in every lane.  v_permlane32_swap / v_permlane16_swap exchange half-waves /
// odd and even rows between two registers, so each step is two moves and an add, with no trip through LDS.
__device__ __forceinline__ uint64_t rows_sum_u64(uint64_t v)
{
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    auto l = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
    auto h = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
    v = (((uint64_t)h[0] << 32) | l[0]) + (((uint64_t)h[1] << 32) | l[1]);
    lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    l = __builtin_amdgcn_permlane16_swap(lo, lo, false, false);
    h = __builtin_amdgcn_permlane16_swap(hi, hi, false, false);
    return (((uint64_t)h[0] << 32) | l[0]) + (((uint64_t)h[1] << 32) | l[1]);
}

// What the 16 bytes of a lane (words d0 = 2j, d1 = 2j + 1 of its stripe) add to accumulators 2j and 2j + 1.
__device__ __forceinline__ void xxh3_lane_terms(uint64_t d0, uint64_t d1, uint64_t k0, uint64_t k1, uint64_t& s0, uint64_t& s1)
{
    s0 = d1 + mul_halves(d0 ^ k0);
    s1 = d0 + mul_halves(d1 ^ k1);
}

// The eight sums of the block a wavefront holds: lanes 0..3 leave with accumulators 2 lane and 2 lane + 1 (every lane
// with those of its lane % 4).
__device__ __forceinline__ void xxh3_block_reduce(uint64_t& s0, uint64_t& s1)
{
    s0 = rows_sum_u64(row_sum_stride4_u64(s0));
    s1 = rows_sum_u64(row_sum_stride4_u64(s1));
}

// The digest walk over tensors described by wq_delta_desc (new_bytes, n, xxh3_sums -> xxh3_digest), for the delta pass
// that has already left the block sums; a tensor whose result[0] is zero gets {0, 0}.  One of `single` (host pointer,
// passed by value to the kernel) and `descs` (device array of n_desc) is given.  Defined beside the walk itself.
int xxh3_chain_for_delta(const wq_delta_desc* single, const wq_delta_desc* descs, int n_desc, hipStream_t st);

}  // namespace wq
