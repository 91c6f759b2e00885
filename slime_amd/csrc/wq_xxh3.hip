// XXH3-128 (seed 0, default secret) of tensors in HBM, for gfx950: the digest the delta publisher attaches to every
// changed tensor (checksum("xxh3-128", new), slime/utils/disk_delta.py:40-58 - the default of
// --update-weight-delta-checksum).  The reference hashes on the host, which means copying every changed tensor there;
// here the tensor stays where it is and sixteen bytes come back.
//
// XXH3's long-input form keeps eight 64-bit accumulators.  A 1 KiB block adds, for each of its sixteen 64-byte
// stripes, lo32(d ^ k) * hi32(d ^ k) of the stripe's word i to accumulator i and word i ^ 1 itself to it - a plain sum
// mod 2^64, in any order - and only then are the accumulators scrambled (xor-shift, xor, multiply): the one step that
// makes blocks sequential.  So the work splits in two:
//   xxh3_block_sums_kernel   the eight sums of every block, at memory speed: a wavefront takes a block with one
//                            16-byte load per lane (lane l holds words 2j, 2j+1 of stripe l / 4, j = l % 4), multiplies
//                            in place and adds across the sixteen lanes that share j; 64 bytes of sums per KiB.
//   xxh3_chain_kernel        per tensor, eight lanes walk acc <- scramble(acc + sums[k]) (about 50 clocks a block), add
//                            the tail - the stripes of the last partial block and the last 64 bytes, read straight from
//                            the tensor - and one lane folds the accumulators into the two 64-bit halves.
// Inputs of 240 bytes or less use XXH3's short forms: one lane of the second kernel computes those.
// The delta pass can leave the block sums itself (it reads the same bytes); then only the walk runs, over its descriptors.

#include "wq_common.h"
#include "wq_xxh3_common.h"

namespace wq {

constexpr int kXxhBlocksPerItem = 16;      // a work item of the sums kernel: 16 KiB, four blocks per wavefront
constexpr int kXxhItemsPerXcdRun = 32;

struct Xxh3Args {
    wq_xxh3_desc d;
    const wq_xxh3_desc* descs;
    const int64_t* item_start;
    int32_t n_desc;
};

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask)
{
    const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask), hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask);
    return ((uint64_t)hi << 32) | lo;
}

template <int GROUPED>
__global__ __launch_bounds__(256) void xxh3_block_sums_kernel(const Xxh3Args a, const int64_t total_items)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_items) return;
    const int64_t item = xcd_chunked_item(slot, total_items, kXxhItemsPerXcdRun);
    wq_xxh3_desc d;
    int64_t local = item;
    if (GROUPED) {
        const int di = find_owner(a.item_start, a.n_desc, item, total_items);
        d = a.descs[di];
        local = item - a.item_start[di];
    } else {
        d = a.d;
    }
    const int64_t nb = scrambled_blocks(d.n);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    uint64_t k0, k1;
    xxh3_lane_keys(lane, k0, k1);
    const uint8_t* base = (const uint8_t*)d.data;
    const bool aligned = ((uintptr_t)base & 15) == 0;
    constexpr int PER_WAVE = kXxhBlocksPerItem / 4;

    uint64_t d0[PER_WAVE], d1[PER_WAVE];
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
        // blocks past the end re-read the tensor's first block instead of branching around the load
        const int64_t b = local * kXxhBlocksPerItem + wave + 4 * i;
        const uint8_t* p = base + (b < nb ? b : 0) * kXxhBlock + lane * 16;
        if (aligned) {
            const u32x4 v = ldg_nt<u32x4>(p);
            d0[i] = ((uint64_t)v.y << 32) | v.x;
            d1[i] = ((uint64_t)v.w << 32) | v.z;
        } else {
            d0[i] = load64_bytes(p);
            d1[i] = load64_bytes(p + 8);
        }
    }
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
        const int64_t b = local * kXxhBlocksPerItem + wave + 4 * i;
        uint64_t s0, s1;
        xxh3_lane_terms(d0[i], d1[i], k0, k1, s0, s1);
        xxh3_block_reduce(s0, s1);
        if (lane < 4 && b < nb) {
            uint64_t* out = d.sums + b * 8 + 2 * lane;
            out[0] = s0;
            out[1] = s1;
        }
    }
}

__device__ __forceinline__ uint64_t mul128_fold64(uint64_t x, uint64_t y) { return (x * y) ^ __umul64hi(x, y); }

__device__ __forceinline__ uint64_t avalanche(uint64_t h)
{
    h ^= h >> 37;
    h *= kMx1;
    return h ^ (h >> 32);
}

// ---- inputs of 0..240 bytes: XXH3's short forms, one lane (a few hundred dependent operations at most) --------------

constexpr uint64_t kMx2 = 0x9FB21C651E98DF25ull;

__device__ __forceinline__ uint32_t secret32(int off)
{
    return (uint32_t)kXxh3Secret[off] | ((uint32_t)kXxh3Secret[off + 1] << 8) | ((uint32_t)kXxh3Secret[off + 2] << 16) |
           ((uint32_t)kXxh3Secret[off + 3] << 24);
}

__device__ __forceinline__ uint64_t xxh64_avalanche(uint64_t h)
{
    h ^= h >> 33;
    h *= kP64_2;
    h ^= h >> 29;
    h *= kP64_3;
    return h ^ (h >> 32);
}

__device__ __forceinline__ uint64_t bswap64(uint64_t v)
{
    return ((uint64_t)__builtin_bswap32((uint32_t)v) << 32) | __builtin_bswap32((uint32_t)(v >> 32));
}

__device__ __forceinline__ uint64_t mix16(const uint8_t* p, int soff)
{
    return mul128_fold64(load64_bytes(p) ^ secret64(soff), load64_bytes(p + 8) ^ secret64(soff + 8));
}

__device__ __forceinline__ void mix32(uint64_t& low, uint64_t& high, const uint8_t* p1, const uint8_t* p2, int soff)
{
    low += mix16(p1, soff);
    low ^= load64_bytes(p2) + load64_bytes(p2 + 8);
    high += mix16(p2, soff + 16);
    high ^= load64_bytes(p1) + load64_bytes(p1 + 8);
}

__device__ void xxh3_short(const uint8_t* p, int n, uint64_t& out_low, uint64_t& out_high)
{
    if (n == 0) {
        out_low = xxh64_avalanche(secret64(64) ^ secret64(72));
        out_high = xxh64_avalanche(secret64(80) ^ secret64(88));
    } else if (n <= 3) {
        const uint32_t lo = ((uint32_t)ldg<uint8_t>(p) << 16) | ((uint32_t)ldg<uint8_t>(p + (n >> 1)) << 24) | (uint32_t)ldg<uint8_t>(p + n - 1) | ((uint32_t)n << 8);
        const uint32_t sw = __builtin_bswap32(lo), hi = (sw << 13) | (sw >> 19);
        out_low = xxh64_avalanche((uint64_t)lo ^ (uint64_t)(secret32(0) ^ secret32(4)));
        out_high = xxh64_avalanche((uint64_t)hi ^ (uint64_t)(secret32(8) ^ secret32(12)));
    } else if (n <= 8) {
        uint32_t a = 0, b = 0;
        for (int k = 0; k < 4; ++k) {
            a |= (uint32_t)ldg<uint8_t>(p + k) << (8 * k);
            b |= (uint32_t)ldg<uint8_t>(p + n - 4 + k) << (8 * k);
        }
        const uint64_t keyed = ((uint64_t)a + ((uint64_t)b << 32)) ^ (secret64(16) ^ secret64(24));
        const uint64_t mult = kP64_1 + ((uint64_t)n << 2);
        uint64_t low = keyed * mult, high = __umul64hi(keyed, mult);
        high += low << 1;
        low ^= high >> 3;
        low ^= low >> 35;
        low *= kMx2;
        low ^= low >> 28;
        out_low = low;
        out_high = avalanche(high);
    } else if (n <= 16) {
        const uint64_t in_lo = load64_bytes(p);
        uint64_t in_hi = load64_bytes(p + n - 8);
        const uint64_t x = in_lo ^ in_hi ^ (secret64(32) ^ secret64(40));
        uint64_t low = x * kP64_1, high = __umul64hi(x, kP64_1);
        low += (uint64_t)(n - 1) << 54;
        in_hi ^= secret64(48) ^ secret64(56);
        high += in_hi + (in_hi & 0xFFFFFFFFull) * (kP32_2 - 1);
        low ^= bswap64(high);
        out_low = avalanche(low * kP64_2);
        out_high = avalanche(__umul64hi(low, kP64_2) + high * kP64_2);
    } else {
        uint64_t low = (uint64_t)n * kP64_1, high = 0;
        if (n <= 128) {
            for (int i = (n - 1) / 32; i >= 0; --i) mix32(low, high, p + 16 * i, p + n - 16 * (i + 1), 32 * i);
        } else {
            for (int i = 32; i < 160; i += 32) mix32(low, high, p + i - 32, p + i - 16, i - 32);
            low = avalanche(low);
            high = avalanche(high);
            for (int i = 160; i <= n; i += 32) mix32(low, high, p + i - 32, p + i - 16, 3 + i - 160);
            mix32(low, high, p + n - 16, p + n - 32, 136 - 17 - 16);
        }
        out_low = avalanche(low + high);
        out_high = 0 - avalanche(low * kP64_1 + high * kP64_4 + (uint64_t)n * kP64_2);
    }
}

// XXH3's scramble of one accumulator, ((a ^ a >> 47) ^ key) * PRIME32_1 mod 2^64, plus `add`.  The two halves of the
// product are kept independent: the low word's 32 x 32 -> 64 multiply-add (which takes `add` along) and the high word's
// 32 x 32 -> 32 multiply can be in flight together, and one 32-bit add joins them.  Written as a 64-bit multiply the
// compiler chains two v_mad_u64_u32, the second waiting for the first - and the walk is nothing but that dependency.
__device__ __forceinline__ uint64_t scramble_then_add(uint64_t a, uint64_t key, uint64_t add)
{
    const uint32_t lo = (uint32_t)a, hi = (uint32_t)(a >> 32);
    const uint32_t xh = hi ^ (uint32_t)(key >> 32);
    const uint32_t xl = lo ^ (hi >> 15) ^ (uint32_t)key;
    uint32_t top = xh * (uint32_t)kP32_1;
    asm volatile("" : "+v"(top));                       // keep it a product of its own
    const uint64_t low = (uint64_t)xl * (uint32_t)kP32_1 + add;
    return (((uint64_t)((uint32_t)(low >> 32) + top)) << 32) | (uint32_t)low;
}

// one wavefront per tensor; lanes 0..7 own one accumulator each
__device__ __forceinline__ wq_xxh3_desc chain_view(const wq_xxh3_desc& d, bool& skip)
{
    skip = false;
    return d;
}
// after a delta pass: the digest of a tensor that did not change is not wanted (nothing is published for it)
__device__ __forceinline__ wq_xxh3_desc chain_view(const wq_delta_desc& d, bool& skip)
{
    skip = ldg<uint64_t>(d.result) == 0;
    return wq_xxh3_desc{d.new_bytes, d.n, d.xxh3_sums, d.xxh3_digest};
}

template <typename Desc>
__global__ __launch_bounds__(64) void xxh3_chain_kernel(const Desc single, const Desc* __restrict__ descs, int n_desc)
{
    const int t = blockIdx.x;
    if (t >= n_desc) return;
    bool skip;
    const wq_xxh3_desc d = chain_view(descs ? descs[t] : single, skip);
    const int lane = threadIdx.x, i = lane & 7;
    if (skip) {                               // uniform per wavefront
        if (lane < 2) stg<uint64_t>(d.digest + lane, 0);
        return;
    }
    if (d.n <= 240) {                         // uniform per wavefront
        if (lane == 0) {
            uint64_t low, high;
            xxh3_short((const uint8_t*)d.data, (int)d.n, low, high);
            stg<uint64_t>(d.digest, low);
            stg<uint64_t>(d.digest + 1, high);
        }
        return;
    }
    const uint64_t init[8] = {kP32_3, kP64_1, kP64_2, kP64_3, kP64_4, kP32_2, kP64_5, kP32_1};
    uint64_t acc = init[0];
#pragma unroll
    for (int k = 1; k < 8; ++k) acc = i == k ? init[k] : acc;
    const uint64_t scramble_key = secret64(192 - kXxhStripe + 8 * i);
    const int64_t nb = scrambled_blocks(d.n);
    const uint64_t* s = d.sums + i;

    // The walk, acc <- scramble(acc + sums[k]) for every block, carried as b_k = acc_k + sums[k]:
    // b_k = scramble(b_{k-1}) + sums[k], so that the addition rides on the multiply-add of the scramble.  A block costs
    // about 50 clocks of dependent arithmetic (20 ns) and a load from HBM takes well over a microsecond, so the sums are
    // fetched 64 blocks ahead: eight batches of eight are in flight, and the batch just consumed is refilled at once with
    // the blocks 64 further on.  Measured per block on a 256 MiB tensor: 32 ahead 23.9 ns, 48: 21.2, 64: 20.2, 80: 21.9,
    // 96: 22.7, 128: 27.2 (the ring no longer fits the registers).
    if (nb > 0) {
        constexpr int U = 8, DEPTH = 8;
        uint64_t ring[DEPTH][U];
        acc += ldg<uint64_t>(s);
        const uint64_t* rest = s + 8;          // sums[1 ..]
        const int64_t m = nb - 1;
        int64_t k = 0;
        if (m >= DEPTH * U) {
#pragma unroll
            for (int b = 0; b < DEPTH; ++b)
#pragma unroll
                for (int u = 0; u < U; ++u) ring[b][u] = ldg<uint64_t>(rest + (b * U + u) * 8);
            for (; k + 2 * DEPTH * U <= m; k += DEPTH * U) {
#pragma unroll
                for (int b = 0; b < DEPTH; ++b) {
#pragma unroll
                    for (int u = 0; u < U; ++u) acc = scramble_then_add(acc, scramble_key, ring[b][u]);
#pragma unroll
                    for (int u = 0; u < U; ++u) ring[b][u] = ldg<uint64_t>(rest + (k + (DEPTH + b) * U + u) * 8);
                }
            }
#pragma unroll
            for (int b = 0; b < DEPTH; ++b)
#pragma unroll
                for (int u = 0; u < U; ++u) acc = scramble_then_add(acc, scramble_key, ring[b][u]);
            k += DEPTH * U;
        }
        for (; k < m; ++k) acc = scramble_then_add(acc, scramble_key, ldg<uint64_t>(rest + k * 8));
        acc = scramble_then_add(acc, scramble_key, 0);
    }

    // the last partial block: its whole stripes, then the last 64 bytes of the input under their own key
    const uint8_t* data = (const uint8_t*)d.data;
    const int64_t tail = nb * kXxhBlock;
    const int n_stripes = (int)(((d.n - 1) - tail) / kXxhStripe);
    for (int st = 0; st <= n_stripes; ++st) {
        const bool last = st == n_stripes;
        const uint8_t* p = last ? data + d.n - kXxhStripe : data + tail + (int64_t)st * kXxhStripe;
        const uint64_t w = load64_bytes(p + 8 * i);
        const uint64_t key = secret64(last ? 192 - kXxhStripe - 7 + 8 * i : 8 * st + 8 * i);
        acc += shfl_xor_u64(w, 1) + mul_halves(w ^ key);
    }

    // fold: lane 0 collects the eight accumulators
    uint64_t all[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t lo = (uint32_t)__shfl((int)(uint32_t)acc, j), hi = (uint32_t)__shfl((int)(uint32_t)(acc >> 32), j);
        all[j] = ((uint64_t)hi << 32) | lo;
    }
    if (lane == 0) {
        uint64_t low = (uint64_t)d.n * kP64_1, high = ~((uint64_t)d.n * kP64_2);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            low += mul128_fold64(all[2 * j] ^ secret64(11 + 16 * j), all[2 * j + 1] ^ secret64(11 + 16 * j + 8));
            high += mul128_fold64(all[2 * j] ^ secret64(192 - kXxhStripe - 11 + 16 * j),
                                  all[2 * j + 1] ^ secret64(192 - kXxhStripe - 11 + 16 * j + 8));
        }
        stg<uint64_t>(d.digest, avalanche(low));
        stg<uint64_t>(d.digest + 1, avalanche(high));
    }
}

int xxh3_chain_for_delta(const wq_delta_desc* single, const wq_delta_desc* descs, int n_desc, hipStream_t st)
{
    xxh3_chain_kernel<wq_delta_desc><<<n_desc, 64, 0, st>>>(single ? *single : wq_delta_desc{}, descs, n_desc);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

static inline int64_t xxh3_items(int64_t n) { return cdiv64(n > 0 ? (n - 1) / kXxhBlock : 0, kXxhBlocksPerItem); }

}  // namespace wq

using namespace wq;

WQ_EXPORT int64_t wq_xxh3_workspace_bytes(int64_t n) { return n > 0 ? ((n - 1) / kXxhBlock) * 64 + 64 : 64; }

WQ_EXPORT int wq_xxh3_128(const void* data, int64_t n, uint64_t* workspace, uint64_t* digest, void* stream)
{
    if (n < 0) return WQ_ERR_SHAPE;
    if ((n > 0 && !data) || !workspace || !digest) return WQ_ERR_NULL;
    if (((uintptr_t)workspace & 15) || ((uintptr_t)digest & 7)) return WQ_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    Xxh3Args a{};
    a.d = wq_xxh3_desc{data, n, workspace, digest};
    const int64_t items = xxh3_items(n);
    if (items) {
        xxh3_block_sums_kernel<0><<<grid_for_items(items), 256, 0, st>>>(a, items);
        WQ_LAUNCH_CHECK();
    }
    xxh3_chain_kernel<wq_xxh3_desc><<<1, 64, 0, st>>>(a.d, nullptr, 1);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_xxh3_128_grouped(const wq_xxh3_desc* descs, const int64_t* item_start, int n_desc, int64_t total_items,
                                  void* stream)
{
    if (n_desc < 0 || total_items < 0) return WQ_ERR_SHAPE;
    if (n_desc == 0) return WQ_OK;
    if (!descs || !item_start) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    Xxh3Args a{};
    a.descs = descs;
    a.item_start = item_start;
    a.n_desc = n_desc;
    if (total_items) {
        xxh3_block_sums_kernel<1><<<grid_for_items(total_items), 256, 0, st>>>(a, total_items);
        WQ_LAUNCH_CHECK();
    }
    xxh3_chain_kernel<wq_xxh3_desc><<<n_desc, 64, 0, st>>>(wq_xxh3_desc{}, descs, n_desc);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}
