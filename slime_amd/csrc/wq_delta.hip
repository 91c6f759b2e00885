// Byte-level delta of a weight tensor against its snapshot, for gfx950.
//
// delta_xor_kernel: one pass over the new bytes and the snapshot that produces everything the delta
// publisher needs from them: diff = new ^ old, the number of changed bytes, the two adler32 sums of the
// new bytes, and (optionally) the snapshot brought up to date.  A workgroup owns a 16 KiB chunk; every
// lane has four 16-byte pieces of both inputs in flight before first use.  Per-chunk partial results go
// to a workspace row (no atomics, nothing to clear), and a one-workgroup kernel folds the rows.  On request the pass
// also leaves XXH3's per-block sums of the new bytes (a wavefront's 64 x 16 bytes of one step are exactly one 1 KiB
// block, lane for lane in the layout those sums want), so the digest costs no second read of the tensor.
//
// adler32 over n bytes d_0..d_{n-1}:  A = 1 + sum d_i,  B = n + sum (n - i) d_i,  both mod 65521, digest
// (B << 16) | A.  Both sums are linear in the bytes, so a chunk at byte offset `base` contributes
// S = sum d_j and (n - base) * S - W with W = sum j * d_j over its local offsets j.
//
// delta_overwrite_*: the idempotent encoding - [count u32][positions u32 x count][new bytes x count] -
// as a three-step stream compaction: per-chunk counts (from the pass above), an exclusive scan of them,
// and a scatter in which each lane ranks its changed bytes with a wave prefix sum.

#include <atomic>

#include "wq_common.h"
#include "wq_xxh3_common.h"

namespace wq {

constexpr int kDeltaSteps = 4;
constexpr int kDeltaChunk = WQ_DELTA_CHUNK;          // bytes of each input per workgroup
constexpr int kDeltaItemsPerXcdRun = 32;
// Residency and bytes in flight, measured on the Qwen3-4B-shaped state dict (xor diff + snapshot update, % of the 8 TB/s
// HBM peak at 4 bytes of traffic per byte; the plain copy kernel reached 72.5 % on that box).  Workgroups per CU x steps
// in flight per lane (a step = one 16-byte piece of each input):
//   8 x 4 (everything at once, full occupancy)   70.6        4 x 4   74.3        3 x 4   76.0        2 x 4   77.2
//   8 x 2   70.2      4 x 2   74.9      3 x 2   77.4      2 x 2   75.4
//   8 x 1   70.0      7 x 1   71.3      4 x 1   74.8      3 x 1   78.1 - 78.7  <- used      2 x 1   69.2      1 x 1   40.5
// The fewer bytes a CU has in flight, the better this memory system streams - down to about 24 KiB per CU.
constexpr int kDeltaOccupancyPadBytes = 50 * 1024;   // unused dynamic LDS that caps workgroups per CU: 3
constexpr int kDeltaWindow = 1;                      // steps (a 16-byte piece of each input per lane) in flight
constexpr uint32_t kAdlerMod = 65521u;
static_assert(kDeltaChunk == 256 * 16 * kDeltaSteps, "chunk = 256 lanes x 16 bytes x steps");

// acc + number of non-zero bytes in a dword
__device__ __forceinline__ uint32_t add_nonzero_bytes(uint32_t x, uint32_t acc)
{
    uint32_t t = (x & 0x7F7F7F7Fu) + 0x7F7F7F7Fu;      // bit 7 of a byte set iff its low 7 bits are non-zero
    t = ((t | x) >> 7) & 0x01010101u;                  // one per non-zero byte
    return __builtin_amdgcn_udot4(t, 0x01010101u, acc, false);
}
// acc + sum over the four bytes of x of weight_k * d_k (v_dot4_u32_u8)
__device__ __forceinline__ uint32_t add_weighted_bytes(uint32_t x, uint32_t weights, uint32_t acc)
{
    return __builtin_amdgcn_udot4(x, weights, acc, false);
}

// Sum over the 16 lanes of a DPP row, left in every lane of the row.
__device__ __forceinline__ uint32_t row16_sum_u32(uint32_t v)
{
    v += dpp_u32<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_u32<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_u32<0x141>(v);   // row_half_mirror
    v += dpp_u32<0x140>(v);   // row_mirror
    return v;
}

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int m)
{
    const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, m);
    const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), m);
    return ((uint64_t)hi << 32) | lo;
}

// A 16-byte piece that straddles the end of the buffer: the bytes that exist, zero-extended.
__device__ __forceinline__ u32x4 load_tail(const uint8_t* p, int valid)
{
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    for (int k = 0; k < valid; ++k) w[k >> 2] |= (uint32_t)ldg<uint8_t>(p + k) << (8 * (k & 3));
    return (u32x4){w[0], w[1], w[2], w[3]};
}
__device__ __forceinline__ void store_tail(uint8_t* p, u32x4 v, int valid)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    for (int k = 0; k < valid; ++k) stg<uint8_t>(p + k, (uint8_t)(w[k >> 2] >> (8 * (k & 3))));
}

// One 16 KiB chunk of one tensor.  partials: [chunks of the tensor][3] uint64 = {changed bytes, S, W}.
template <bool DIFF, bool UPDATE, bool XXH3>
__device__ __forceinline__ void delta_xor_chunk(const uint8_t* __restrict__ nw, uint8_t* __restrict__ old,
                                                uint8_t* __restrict__ diff, int64_t n, uint64_t* __restrict__ partials,
                                                uint64_t* __restrict__ xsums, int64_t item, uint32_t (*red)[4])
{
    const int64_t base = item * kDeltaChunk;
    u32x4 a[kDeltaSteps], b[kDeltaSteps];
    uint64_t k0 = 0, k1 = 0, xs0[kDeltaSteps], xs1[kDeltaSteps];
    if (XXH3) xxh3_lane_keys(threadIdx.x & 63, k0, k1);
    const bool whole = n >= 16;
    auto issue = [&](int i) {
        // lanes past the end re-read the last whole piece instead of branching around the load
        const int64_t off = base + (int64_t)(i * 256 + threadIdx.x) * 16;
        const int64_t safe = min(off, (n / 16 - 1) * 16);
        a[i] = ldg_nt<u32x4>(nw + safe);
        b[i] = ldg_nt<u32x4>(old + safe);
    };
    if (whole) {
#pragma unroll
        for (int i = 0; i < kDeltaWindow && i < kDeltaSteps; ++i) issue(i);
    }
    // W of the chunk = P + 4096 * Q with P = sum over pieces of (16 * lane) * s + r and Q = sum of step * s:
    // both stay far below 2^32 per row, so the reduction runs on dwords
    uint32_t changed = 0, s_lane = 0, p_lane = 0, q_lane = 0;
#pragma unroll
    for (int i = 0; i < kDeltaSteps; ++i) {
        if (kDeltaWindow < kDeltaSteps) {
            // a rolling window: the pieces of step i + window are requested once those of step i are about to be used
            asm volatile("" :: "v"(a[i].x), "v"(b[i].x));
            if (whole && i + kDeltaWindow < kDeltaSteps) issue(i + kDeltaWindow);
            __builtin_amdgcn_sched_barrier(0);
        }
        const uint32_t local = (uint32_t)(i * 256 + threadIdx.x) * 16;
        const int64_t off = base + local;
        int valid = 16;
        if (off + 16 > n) {
            valid = off < n ? (int)(n - off) : 0;
            a[i] = load_tail(nw + off, valid);
            b[i] = load_tail(old + off, valid);
        }
        const u32x4 d = a[i] ^ b[i];
        changed = add_nonzero_bytes(d.x, add_nonzero_bytes(d.y, add_nonzero_bytes(d.z, add_nonzero_bytes(d.w, changed))));
        // s = sum of the 16 bytes, r = sum of k * d_k over them
        uint32_t s = add_weighted_bytes(a[i].x, 0x01010101u, 0u);
        s = add_weighted_bytes(a[i].y, 0x01010101u, s);
        s = add_weighted_bytes(a[i].z, 0x01010101u, s);
        s = add_weighted_bytes(a[i].w, 0x01010101u, s);
        uint32_t r = add_weighted_bytes(a[i].x, 0x03020100u, 0u);
        r = add_weighted_bytes(a[i].y, 0x07060504u, r);
        r = add_weighted_bytes(a[i].z, 0x0B0A0908u, r);
        r = add_weighted_bytes(a[i].w, 0x0F0E0D0Cu, r);
        s_lane += s;
        p_lane += (uint32_t)threadIdx.x * 16u * s + r;
        q_lane += (uint32_t)i * s;
        if (XXH3)
            xxh3_lane_terms(((uint64_t)a[i].y << 32) | a[i].x, ((uint64_t)a[i].w << 32) | a[i].z, k0, k1, xs0[i], xs1[i]);
        if (valid == 16) {
            if (DIFF) stg_nt_sc1<u32x4>(diff + off, d);
            if (UPDATE) stg_nt_sc1<u32x4>(old + off, a[i]);
        } else if (valid > 0) {
            if (DIFF) store_tail(diff + off, d, valid);
            if (UPDATE) store_tail(old + off, a[i], valid);
        }
    }
    if (XXH3) {
        // the wavefront's piece of step i is block 16 * item + 4 * i + wave of the tensor; only blocks that end before
        // the last byte are summed here (the rest is the digest walk's tail, read from the tensor)
        const int64_t nb = scrambled_blocks(n);
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
        for (int i = 0; i < kDeltaSteps; ++i) {
            const int64_t blk = item * (kDeltaChunk / kXxhBlock) + i * 4 + wave;
            xxh3_block_reduce(xs0[i], xs1[i]);
            if (lane < 4 && blk < nb) {
                uint64_t* out = xsums + blk * 8 + 2 * lane;
                out[0] = xs0[i];
                out[1] = xs1[i];
            }
        }
    }
    changed = row16_sum_u32(changed);
    s_lane = row16_sum_u32(s_lane);
    p_lane = row16_sum_u32(p_lane);
    q_lane = row16_sum_u32(q_lane);
    if ((threadIdx.x & 15) == 0) {
        uint32_t* r = red[threadIdx.x >> 4];
        r[0] = changed;
        r[1] = s_lane;
        r[2] = p_lane;
        r[3] = q_lane;
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        uint64_t v = 0;
        for (int k = 0; k < 16; ++k)
            v += threadIdx.x < 2 ? (uint64_t)red[k][threadIdx.x] : (uint64_t)red[k][2] + 4096ull * red[k][3];
        stg<uint64_t>(partials + item * 3 + threadIdx.x, v);
    }
}

struct DeltaArgs {
    wq_delta_desc d;                 // single-tensor launch
    const wq_delta_desc* descs;      // grouped launch: device arrays
    const int64_t* chunk_start;
    int n_desc;
    const wq_delta_chunk_item* items;   // per-chunk form
};

// GROUPED: 0 = one tensor in the kernel arguments, 1 = descriptor array + prefix sums (the owner of a chunk is
// searched), 2 = one pre-resolved descriptor per chunk
template <bool DIFF, bool UPDATE, int GROUPED, bool XXH3>
__global__ __launch_bounds__(256) void delta_xor_kernel(const DeltaArgs a, int64_t items)
{
    __shared__ uint32_t red[16][4];      // per 16-lane row: changed, S, P, Q
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= items) return;
    int64_t item = xcd_chunked_item(slot, items, kDeltaItemsPerXcdRun);
    wq_delta_desc d;
    if (GROUPED == 1) {
        const int di = find_owner(a.chunk_start, a.n_desc, item, items);
        d = a.descs[di];
        item -= a.chunk_start[di];
    } else if (GROUPED == 2) {
        const wq_delta_chunk_item it = a.items[item];
        d = wq_delta_desc{it.new_bytes, it.old_bytes, it.diff, it.n, it.workspace, nullptr, it.xxh3_sums, nullptr};
        item = it.chunk;
    } else {
        d = a.d;
    }
    delta_xor_chunk<DIFF, UPDATE, XXH3>((const uint8_t*)d.new_bytes, (uint8_t*)d.old_bytes, (uint8_t*)d.diff, d.n,
                                        (uint64_t*)d.workspace, d.xxh3_sums, item, red);
}

// result[0] = changed bytes, result[1] = adler32 of the new bytes.  One workgroup of 1024 lanes per tensor; every lane keeps
// the rows of four chunks in flight, so the pass over the partials is a few dozen memory round trips.
constexpr int kFoldThreads = 1024;
constexpr int kFoldUnroll = 4;
template <bool GROUPED>
__global__ __launch_bounds__(kFoldThreads) void delta_fold_kernel(const DeltaArgs a)
{
    __shared__ uint64_t red[kFoldThreads / 64][3];
    const wq_delta_desc d = GROUPED ? a.descs[blockIdx.x] : a.d;
    const uint64_t* __restrict__ partials = (const uint64_t*)d.workspace;
    uint64_t* __restrict__ result = d.result;
    const int64_t n = d.n;
    const int64_t items = (n + kDeltaChunk - 1) / kDeltaChunk;
    uint64_t changed = 0, s_total = 0, b_acc = 0;
    for (int64_t c0 = threadIdx.x; c0 < items; c0 += kFoldThreads * kFoldUnroll) {
        uint64_t row[kFoldUnroll][3];
#pragma unroll
        for (int u = 0; u < kFoldUnroll; ++u) {
            const int64_t c = c0 + (int64_t)u * kFoldThreads;
            const int64_t cc = c < items ? c : c0;
#pragma unroll
            for (int k = 0; k < 3; ++k) row[u][k] = ldg<uint64_t>(partials + cc * 3 + k);
        }
#pragma unroll
        for (int u = 0; u < kFoldUnroll; ++u) {
            const int64_t c = c0 + (int64_t)u * kFoldThreads;
            if (c >= items) continue;
            changed += row[u][0];
            s_total += row[u][1];                                  // <= 255 * n: no overflow
            const uint64_t weight = (uint64_t)(n - c * kDeltaChunk) % kAdlerMod;
            b_acc = (b_acc + weight * (row[u][1] % kAdlerMod) + kAdlerMod - row[u][2] % kAdlerMod) % kAdlerMod;
        }
    }
    // wave sums (b_acc stays below 64 * 65521), then one lane folds the 16 wave rows
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        changed += shfl_xor_u64(changed, m);
        s_total += shfl_xor_u64(s_total, m);
        b_acc += shfl_xor_u64(b_acc, m);
    }
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6][0] = changed;
        red[threadIdx.x >> 6][1] = s_total;
        red[threadIdx.x >> 6][2] = b_acc;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int t = 1; t < kFoldThreads / 64; ++t) {
            changed += red[t][0];
            s_total += red[t][1];
            b_acc += red[t][2];
        }
        const uint64_t A = (1 + s_total % kAdlerMod) % kAdlerMod;
        const uint64_t B = ((uint64_t)n % kAdlerMod + b_acc) % kAdlerMod;
        result[0] = changed;
        result[1] = (B << 16) | A;
    }
}

// ---- overwrite encoding -----------------------------------------------------------------------------

// offsets[c] = number of changed bytes in chunks before c (exclusive scan of partials[c][0]); one workgroup.
__global__ __launch_bounds__(256) void delta_scan_kernel(const uint64_t* __restrict__ partials, int64_t items,
                                                        uint32_t* __restrict__ offsets)
{
    __shared__ uint32_t sums[256];
    __shared__ uint32_t carry;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    for (int64_t c0 = 0; c0 < items; c0 += 256) {
        const int64_t c = c0 + threadIdx.x;
        const uint32_t v = c < items ? (uint32_t)partials[c * 3] : 0u;
        sums[threadIdx.x] = v;
        __syncthreads();
        // Hillis-Steele inclusive scan over 256 entries
        for (int d = 1; d < 256; d <<= 1) {
            const uint32_t t = threadIdx.x >= d ? sums[threadIdx.x - d] : 0u;
            __syncthreads();
            sums[threadIdx.x] += t;
            __syncthreads();
        }
        if (c < items) offsets[c] = carry + sums[threadIdx.x] - v;
        __syncthreads();
        if (threadIdx.x == 255) carry += sums[255];
        __syncthreads();
    }
}

// bit k set iff byte k of the 16-byte pieces differs
__device__ __forceinline__ uint32_t diff_mask16(u32x4 a, u32x4 b)
{
    const uint32_t d[4] = {a.x ^ b.x, a.y ^ b.y, a.z ^ b.z, a.w ^ b.w};
    uint32_t m = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        uint32_t t = (((d[k] & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | d[k]) & 0x80808080u;   // bit 7 of each changed byte
        t = (t >> 7) * 0x00204081u;                                                 // gathers them into bits 21..24
        m |= ((t >> 21) & 0xFu) << (4 * k);
    }
    return m;
}

__device__ __forceinline__ uint32_t wave_exclusive_sum(uint32_t v, uint32_t& total)
{
    const int lane = threadIdx.x & 63;
    uint32_t inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t t = (uint32_t)__shfl_up((int)inc, d);
        if (lane >= d) inc += t;
    }
    total = (uint32_t)__shfl((int)inc, 63);
    return inc - v;
}

// out = [count u32][positions u32 x count][values u8 x count].  A wave owns a contiguous quarter of the
// chunk (four steps of 64 lanes x 16 bytes, all loaded before first use); lanes rank their changed bytes
// with a wave prefix sum, waves are ordered through LDS, chunks through `offsets`.
template <bool UPDATE>
__global__ __launch_bounds__(256) void delta_overwrite_kernel(const uint8_t* __restrict__ nw, uint8_t* __restrict__ old,
                                                             int64_t n, const uint32_t* __restrict__ offsets,
                                                             uint32_t count, uint8_t* __restrict__ out, int64_t items)
{
    __shared__ uint32_t wave_count[4];
    const int64_t item = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (item >= items) return;
    if (item == 0 && threadIdx.x == 0) stg<uint32_t>(out, count);
    if (n == 0) return;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t wbase = item * kDeltaChunk + (int64_t)wave * (kDeltaChunk / 4);
    u32x4 a[kDeltaSteps], b[kDeltaSteps];
    if (n >= 16) {
#pragma unroll
        for (int i = 0; i < kDeltaSteps; ++i) {
            const int64_t off = wbase + (int64_t)(i * 64 + lane) * 16;
            const int64_t safe = min(off, (n / 16 - 1) * 16);
            a[i] = ldg_nt<u32x4>(nw + safe);
            b[i] = ldg_nt<u32x4>(old + safe);
        }
    }
    uint32_t mask[kDeltaSteps], before[kDeltaSteps], wave_total = 0;
#pragma unroll
    for (int i = 0; i < kDeltaSteps; ++i) {
        const int64_t off = wbase + (int64_t)(i * 64 + lane) * 16;
        if (off + 16 > n) {
            const int valid = off < n ? (int)(n - off) : 0;
            a[i] = load_tail(nw + off, valid);          // missing bytes read as zero on both sides: unchanged
            b[i] = load_tail(old + off, valid);
        }
        mask[i] = diff_mask16(a[i], b[i]);
        uint32_t step_total;
        before[i] = wave_total + wave_exclusive_sum((uint32_t)__builtin_popcount(mask[i]), step_total);
        wave_total += step_total;
    }
    if (lane == 0) wave_count[wave] = wave_total;
    __syncthreads();
    uint32_t rank0 = offsets[item];
    for (int w = 0; w < wave; ++w) rank0 += wave_count[w];
    uint32_t* pos_out = (uint32_t*)(out + 4);
    uint8_t* val_out = out + 4 + (int64_t)count * 4;
#pragma unroll
    for (int i = 0; i < kDeltaSteps; ++i) {
        const int64_t off = wbase + (int64_t)(i * 64 + lane) * 16;
        const uint32_t w4[4] = {a[i].x, a[i].y, a[i].z, a[i].w};
        uint32_t r = rank0 + before[i];
        for (uint32_t m = mask[i]; m; m &= m - 1) {
            const int k = __builtin_ctz(m);
            stg<uint32_t>(pos_out + r, (uint32_t)(off + k));
            stg<uint8_t>(val_out + r, (uint8_t)(w4[k >> 2] >> (8 * (k & 3))));
            ++r;
        }
        if (UPDATE && mask[i]) {                         // the snapshot catches up where it differs
            if (off + 16 <= n) stg_nt<u32x4>(old + off, a[i]);
            else store_tail(old + off, a[i], (int)(n - off));
        }
    }
}

}  // namespace wq

using namespace wq;

WQ_EXPORT int64_t wq_delta_workspace_bytes(int64_t n)
{
    if (n < 0) return WQ_ERR_SHAPE;
    return cdiv64(n > 0 ? n : 1, kDeltaChunk) * 32;      // 24 bytes of partials + a 4-byte scan slot, rounded up
}

template <int GROUPED, bool XXH3>
static void launch_delta_xor_x(const DeltaArgs& a, int64_t items, bool diff, bool update, hipStream_t st)
{
    const dim3 g = grid_for_items(items);
    if (diff && update) delta_xor_kernel<true, true, GROUPED, XXH3><<<g, 256, kDeltaOccupancyPadBytes, st>>>(a, items);
    else if (diff) delta_xor_kernel<true, false, GROUPED, XXH3><<<g, 256, kDeltaOccupancyPadBytes, st>>>(a, items);
    else if (update) delta_xor_kernel<false, true, GROUPED, XXH3><<<g, 256, kDeltaOccupancyPadBytes, st>>>(a, items);
    else delta_xor_kernel<false, false, GROUPED, XXH3><<<g, 256, kDeltaOccupancyPadBytes, st>>>(a, items);
}

template <int GROUPED>
static void launch_delta_xor(const DeltaArgs& a, int64_t items, bool diff, bool update, bool xxh3, hipStream_t st)
{
    if (xxh3) launch_delta_xor_x<GROUPED, true>(a, items, diff, update, st);
    else launch_delta_xor_x<GROUPED, false>(a, items, diff, update, st);
}

static int delta_xor_one(const void* new_bytes, void* old_bytes, void* diff, int64_t n, int update_old, void* workspace,
                         uint64_t* result, uint64_t* xxh3_workspace, uint64_t* digest, bool xxh3, hipStream_t st)
{
    if (n < 0) return WQ_ERR_SHAPE;
    if (!result || !workspace || (xxh3 && (!xxh3_workspace || !digest))) return WQ_ERR_NULL;
    if (n > 0 && (!new_bytes || !old_bytes)) return WQ_ERR_NULL;
    if (((uintptr_t)new_bytes & 15) || ((uintptr_t)old_bytes & 15) || ((uintptr_t)diff & 15) ||
        ((uintptr_t)workspace & 7) || ((uintptr_t)result & 7))
        return WQ_ERR_ALIGN;
    if (xxh3 && (((uintptr_t)xxh3_workspace & 15) || ((uintptr_t)digest & 7))) return WQ_ERR_ALIGN;
    const int64_t items = n > 0 ? cdiv64(n, kDeltaChunk) : 0;
    DeltaArgs a{};
    a.d = wq_delta_desc{new_bytes, old_bytes, diff, n, workspace, result, xxh3_workspace, digest};
    if (items > 0) {
        launch_delta_xor<0>(a, items, diff != nullptr, update_old != 0, xxh3, st);
        WQ_LAUNCH_CHECK();
    }
    delta_fold_kernel<false><<<1, kFoldThreads, 0, st>>>(a);
    WQ_LAUNCH_CHECK();
    return xxh3 ? xxh3_chain_for_delta(&a.d, nullptr, 1, st) : WQ_OK;
}

WQ_EXPORT int wq_delta_xor(const void* new_bytes, void* old_bytes, void* diff, int64_t n, int update_old,
                           void* workspace, uint64_t* result, void* stream)
{
    return delta_xor_one(new_bytes, old_bytes, diff, n, update_old, workspace, result, nullptr, nullptr, false,
                         (hipStream_t)stream);
}

WQ_EXPORT int wq_delta_xor_xxh3(const void* new_bytes, void* old_bytes, void* diff, int64_t n, int update_old,
                                void* workspace, uint64_t* result, uint64_t* xxh3_workspace, uint64_t* digest, void* stream)
{
    return delta_xor_one(new_bytes, old_bytes, diff, n, update_old, workspace, result, xxh3_workspace, digest, true,
                         (hipStream_t)stream);
}

// ---- the same pass for callers that cannot allocate ------------------------------------------------------
// The per-chunk partial sums live in a file-scope device array instead of a caller workspace.  Every GPU has its
// own copy of the array at its own address; the address is looked up once per device, with that device current,
// and only that pointer is ever handed to kernels (the array's name is a host-side handle, not a device address).
constexpr int64_t kStaticMaxBytes = WQ_DELTA_NOALLOC_MAX_BYTES;
constexpr int64_t kStaticRows = kStaticMaxBytes / kDeltaChunk;
static __device__ __align__(256) uint64_t scratch[kStaticRows * 3];

constexpr int kMaxDevices = 64;
static std::atomic<uint64_t*> g_scratch_ptr[kMaxDevices];

static int static_scratch(uint64_t** out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return WQ_ERR_UNSUPPORTED;
    uint64_t* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        void* sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!sym) return WQ_ERR_NULL;
        p = (uint64_t*)sym;
        g_scratch_ptr[dev].store(p, std::memory_order_release);   // racing threads store the same value
    }
    *out = p;
    return WQ_OK;
}

WQ_EXPORT int wq_delta_xor_noalloc(const void* new_bytes, void* old_bytes, void* diff, int64_t n, int update_old,
                                   uint64_t* result, void* stream)
{
    if (n < 0) return WQ_ERR_SHAPE;
    if (n > kStaticMaxBytes) return WQ_ERR_TOO_LARGE;
    if (!result) return WQ_ERR_NULL;
    uint64_t* ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc) return rc;
    // every chunk row that the fold reads is written by this call's first kernel: nothing to clear
    return wq_delta_xor(new_bytes, old_bytes, diff, n, update_old, ws, result, stream);
}

WQ_EXPORT int wq_delta_xor_grouped(const wq_delta_desc* descs, const int64_t* chunk_start, int n_desc,
                                   int64_t total_chunks, int write_diff, int update_old, int with_xxh3, void* stream)
{
    if (n_desc < 0 || total_chunks < 0) return WQ_ERR_SHAPE;
    if (n_desc == 0) return WQ_OK;
    if (!descs || !chunk_start) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    DeltaArgs a{};
    a.descs = descs;
    a.chunk_start = chunk_start;
    a.n_desc = n_desc;
    if (total_chunks > 0) {
        launch_delta_xor<1>(a, total_chunks, write_diff != 0, update_old != 0, with_xxh3 != 0, st);
        WQ_LAUNCH_CHECK();
    }
    delta_fold_kernel<true><<<n_desc, kFoldThreads, 0, st>>>(a);
    WQ_LAUNCH_CHECK();
    return with_xxh3 ? xxh3_chain_for_delta(nullptr, descs, n_desc, st) : WQ_OK;
}

WQ_EXPORT int wq_delta_xor_items(const wq_delta_chunk_item* items, int64_t n_items, const wq_delta_desc* descs, int n_desc,
                                 int write_diff, int update_old, int with_xxh3, void* stream)
{
    if (n_desc < 0 || n_items < 0) return WQ_ERR_SHAPE;
    if (n_desc == 0) return WQ_OK;
    if (!descs || (n_items > 0 && !items)) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    DeltaArgs a{};
    a.descs = descs;
    a.n_desc = n_desc;
    a.items = items;
    if (n_items > 0) {
        launch_delta_xor<2>(a, n_items, write_diff != 0, update_old != 0, with_xxh3 != 0, st);
        WQ_LAUNCH_CHECK();
    }
    delta_fold_kernel<true><<<n_desc, kFoldThreads, 0, st>>>(a);
    WQ_LAUNCH_CHECK();
    return with_xxh3 ? xxh3_chain_for_delta(nullptr, descs, n_desc, st) : WQ_OK;
}

WQ_EXPORT int wq_delta_overwrite_encode(const void* new_bytes, void* old_bytes, int64_t n, void* workspace,
                                        uint32_t count, void* out, int update_old, void* stream)
{
    if (n < 0 || n > 0xFFFFFFFFll) return n < 0 ? WQ_ERR_SHAPE : WQ_ERR_TOO_LARGE;   // positions are uint32
    if (!out || !workspace) return WQ_ERR_NULL;
    if (n > 0 && (!new_bytes || !old_bytes)) return WQ_ERR_NULL;
    if (((uintptr_t)out & 3) || ((uintptr_t)workspace & 7)) return WQ_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int64_t items = n > 0 ? cdiv64(n, kDeltaChunk) : 0;
    const uint64_t* partials = (const uint64_t*)workspace;
    uint32_t* offsets = (uint32_t*)((uint64_t*)workspace + items * 3);
    if (items > 0) {
        delta_scan_kernel<<<1, 256, 0, st>>>(partials, items, offsets);
        WQ_LAUNCH_CHECK();
    }
    // an empty tensor still gets its header word (count = 0) from workgroup 0
    const int64_t launch_items = items > 0 ? items : 1;
    if (update_old)
        delta_overwrite_kernel<true><<<grid_for_items(launch_items), 256, 0, st>>>(
            (const uint8_t*)new_bytes, (uint8_t*)old_bytes, n, offsets, count, (uint8_t*)out, launch_items);
    else
        delta_overwrite_kernel<false><<<grid_for_items(launch_items), 256, 0, st>>>(
            (const uint8_t*)new_bytes, (uint8_t*)old_bytes, n, offsets, count, (uint8_t*)out, launch_items);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}
