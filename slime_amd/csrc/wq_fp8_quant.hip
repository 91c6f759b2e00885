// bf16 -> block-FP8 (e4m3fn) quantisation for gfx950.
//
// Vector kernel (128x128 blocks, unit column stride, 16-byte aligned rows): one 256-thread
// workgroup owns one block.  Each lane issues eight 16-byte loads (8 bf16 each, rows rb+16*i; a
// wavefront load covers four 256-byte row segments), a few at a time (kTileWindow), and the 32 KiB block lives in
// registers from then on: amax is an integer max over the bf16
// magnitude bits (packed 16-bit max), reduced over 16 lanes with DPP and across the workgroup
// through 64 bytes of LDS; the scale is computed once; every element is divided with a
// reciprocal + two FMA refinement that equals the IEEE quotient, converted with v_cvt_pk_fp8_f32
// and stored as 8-byte pieces.  HBM traffic is exactly one read of x, one write of y and 4 bytes of
// scale per block.
//
// Generic kernel: any block shape / strides / alignment, one workgroup per block, two passes over
// the block (the second one hits L2), exact IEEE division and software conversion.

#include "wq_common.h"

namespace wq {

// Workgroup shape, work order and residency, measured on MI355X on the Qwen3-4B-shaped pass (252 tensors,
// 7.27 GB of bf16, one grouped launch; fraction of the 8 TB/s HBM peak):
//   256 threads, plain dispatch order, full occupancy (8 workgroups per CU)      69.6 %
//   256 threads, runs of 32 tiles per XCD, 4 workgroups per CU                   76.7 - 77.1 %   <- used
//   256 threads, runs of 64 tiles per XCD, 4 workgroups per CU                   76.9 %
//   256 threads, runs of 32 tiles per XCD, 3 workgroups per CU                   73.6 %
//   512 threads (4 loads per lane), runs of 16 / 32 / 64 tiles                   75.5 / 76.1 / 76.3 %
//   512 threads, plain dispatch order                                            71.1 %
// A compute-free kernel with the same tiles (128 rows x 256 bytes in, 128 x 128 out, same work order) reaches 81.5-82.9 %, one with
// the same 2:1 mix over contiguous 32 KiB pieces 83-84 %.
constexpr int kTileThreads = 256;
constexpr int kTilesPerXcdRun = 32;               // consecutive tiles handed to one XCD (xcd_chunked_item)
constexpr unsigned kOccupancyPadBytes = 36 * 1024;  // unused dynamic LDS: caps residency at 4 workgroups per CU
// 16-byte loads a lane keeps in flight while it folds the block maximum: the load of step i + window is issued when step
// i has been folded in.  On the full Qwen3-30B-A3B-shaped state dict (4 workgroups per CU): all 8 at once 79.1 %, 6: 79.5,
// 4: 79.1, 3: 79.5, 2: 80.6-80.8 (used), 1: 72.1; with 5 or more workgroups per CU a window lowers the rate, and 3 per CU
// is behind with every window (2: 77.7, 3: 80.1, 4: 80.0, 8: 78.7).  The
// Qwen3-4B-shaped pass does not move (76.3-76.6 either way).  A compute-free 2:1 stream of the same shape is fastest at 2
// workgroups per CU (84 %): fewer bytes in flight per CU suit the memory system, and the window gets part of that while
// four workgroups keep the arithmetic overlapped.
constexpr int kTileWindow = 2;
// Launches of at most kSmallLaunchTiles tiles put fewer than two workgroups on a CU: nothing else is there to overlap a
// workgroup's load latency, so these issue all eight loads of a lane at once and run without the residency pad
// ([2048, 2048], 256 tiles, launches back to back: 6.0 -> 5.1 us).  From one workgroup per CU slot upwards the windowed
// form is as fast or faster ([4096, 4096], 1024 tiles: 10.7 us windowed, 11.2 us all at once; 2048 tiles: 19.2 - 20.2 us in
// every combination of window and pad), and a launch of that size is within 1.5 us of launch gap (1.6 us between two
// empty kernels on one stream) + the time its bytes take at the rate the plain copy reaches.
constexpr int64_t kSmallLaunchTiles = 512;
constexpr int kSmallTileWindow = 8;
constexpr unsigned kSmallOccupancyPadBytes = 0;
constexpr int kRowSlots = kTileThreads / 16;   // rows covered by one load step of the workgroup
constexpr int kTileLoads = 128 / kRowSlots;    // 16-byte loads per lane
constexpr int kTileWaves = kTileThreads / 64;

struct Fp8QuantArgs {
    wq_fp8_quant_desc d;  // single-tensor launch: descriptor travels in the kernel arguments
    const wq_fp8_quant_desc* descs;
    const int64_t* tile_start;
    int32_t n_desc;
    int32_t bm, bn;
    char* out_base;       // per-tile form only: when set, y and s of every descriptor are byte offsets from here
};

__device__ __forceinline__ bool desc_vector_ok(const wq_fp8_quant_desc& d)
{
    // 128 rows of either operand must span fewer than 2^31 bytes: lane offsets are 32-bit
    return d.sx_n == 1 && (d.sx_m & 7) == 0 && (d.N & 7) == 0 && (d.sy_m & 7) == 0 &&
           ((uintptr_t)d.x & 15) == 0 && ((uintptr_t)d.y & 3) == 0 && d.sx_m >= 0 && d.sx_m < (1 << 22) &&
           d.sy_m >= 0 && d.sy_m < (1 << 22);
}

// PLAIN: plain instead of non-temporal stores of the codes (see fp8_block_quant_plain_kernel)
template <int MODE, int WINDOW, bool PLAIN = false>
__device__ __forceinline__ void quant_tile_vec128(const wq_fp8_quant_desc& d, int64_t tm, int64_t tn, int kt,
                                                  uint32_t* lds)
{
    const int t = threadIdx.x;
    const int cc = t & 15;  // which 8-element piece of the 128 columns
    const int rb = t >> 4;  // 0..kRowSlots-1
    // Workgroup-uniform tile origin (scalar registers) + 32-bit per-lane byte offsets.
    const char* xt = (const char*)d.x + (tm * 128 * d.sx_m + tn * 128) * 2;
    char* yt = (char*)d.y + (tm * 128 * d.sy_m + tn * 128);
    const uint32_t xstep = (uint32_t)d.sx_m * 2u * kRowSlots, ystep = (uint32_t)d.sy_m * kRowSlots;  // one step, in bytes
    const uint32_t xoff = (uint32_t)rb * (uint32_t)d.sx_m * 2u + (uint32_t)cc * 16u;
    const uint32_t yoff = (uint32_t)rb * (uint32_t)d.sy_m + (uint32_t)cc * 8u;
    const int rows_left = (int)min((int64_t)128, d.M - tm * 128) - rb;  // row rb + kRowSlots*i is valid iff kRowSlots*i < rows_left
    const bool col_ok = tn * 128 + cc * 8 < d.N;
    const bool full = (tm * 128 + 128 <= d.M) && (tn * 128 + 128 <= d.N);

    u32x4 v[kTileLoads];
    uint32_t m = 0;
    if (full) {
#pragma unroll
        for (int i = 0; i < WINDOW && i < kTileLoads; ++i) v[i] = ldg_nt<u32x4>(xt + (xoff + i * xstep));
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) {
            m = pk_absmax(m, v[i].x);
            m = pk_absmax(m, v[i].y);
            m = pk_absmax(m, v[i].z);
            m = pk_absmax(m, v[i].w);
            if (WINDOW < kTileLoads) {
                __builtin_amdgcn_sched_barrier(0);      // keep the next load behind this step's use of its data
                if (i + WINDOW < kTileLoads) v[i + WINDOW] = ldg_nt<u32x4>(xt + (xoff + (i + WINDOW) * xstep));
            }
        }
    } else {
        // Edge tile: every lane loads from a valid address - its row and piece clamped into the tile - and the lanes
        // outside the tensor are zeroed afterwards.  (Loads predicated per lane make the compiler wait for the earlier
        // ones before it issues the next; this way all eight are in flight together, as in a full tile.)
        const int rows = (int)min((int64_t)128, d.M - tm * 128);
        const int pieces = (int)min((int64_t)16, (d.N - tn * 128) >> 3);
        const uint32_t coff = (uint32_t)min(cc, pieces - 1) * 16u;
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) {
            const uint32_t r = (uint32_t)min(rb + kRowSlots * i, rows - 1);
            v[i] = ldg_nt<u32x4>(xt + (r * (uint32_t)d.sx_m * 2u + coff));
        }
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i)
            if (!(col_ok && kRowSlots * i < rows_left)) v[i] = (u32x4){0u, 0u, 0u, 0u};
    }

    if (!full) {
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) {
            m = pk_absmax(m, v[i].x);
            m = pk_absmax(m, v[i].y);
            m = pk_absmax(m, v[i].z);
            m = pk_absmax(m, v[i].w);
        }
    }
    m = row16_max_u32(pk_fold(m));
    if (cc == 0) lds[rb] = m;
    __syncthreads();
    m = 0;
#pragma unroll
    for (int i = 0; i < kRowSlots / 4; ++i) {
        const u32x4 a = ((const u32x4*)lds)[i];
        m = max(m, max(max(a.x, a.y), max(a.z, a.w)));
    }

    const Fp8BlockParams p = fp8_block_params<MODE>(m);
    if (t == 0) stg<float>(d.s + (tm * kt + tn), p.scale);

    if (p.fast) {
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) {
            u32x2 o;
            o.x = fp8_quant4_fast<MODE>(v[i].x, v[i].y, p);
            o.y = fp8_quant4_fast<MODE>(v[i].z, v[i].w, p);
            if (full || (col_ok && kRowSlots * i < rows_left)) {
                if (PLAIN) stg<u32x2>(yt + (yoff + i * ystep), o);
                else stg_nt_sc1<u32x2>(yt + (yoff + i * ystep), o);
            }
        }
    } else {
        // NaN/Inf block (rare): literal arithmetic.  The rows are re-read so that the register copy of
        // the block is never indexed dynamically.
#pragma nounroll
        for (int i = 0; i < kTileLoads; ++i) {
            if (!(full || (col_ok && kRowSlots * i < rows_left))) continue;
            const u32x4 w = ldg<u32x4>(xt + (xoff + i * xstep));
            u32x2 o;
            o.x = fp8_quant4_exact<MODE>(w.x, w.y, p);
            o.y = fp8_quant4_exact<MODE>(w.z, w.w, p);
            stg<u32x2>(yt + (yoff + i * ystep), o);
        }
    }
}

// Every access goes through the global-address-space helpers, here too: one flat (generic-pointer) access anywhere in a
// kernel makes the compiler wait for ALL outstanding memory operations (vmcnt(0)) wherever it waits for one, in the vector
// path as well - its rolling load window then drains after every second load.
template <int MODE>
__device__ __forceinline__ void quant_tile_generic(const wq_fp8_quant_desc& d, int64_t tm, int64_t tn, int kt,
                                                   int bm, int bn, uint32_t* lds)
{
    const int64_t r0 = tm * bm, c0 = tn * bn;
    const int rows = (int)min((int64_t)bm, d.M - r0), cols = (int)min((int64_t)bn, d.N - c0);
    const int n = rows * cols;
    const uint16_t* x = (const uint16_t*)d.x;
    uint32_t m = 0;
    for (int e = threadIdx.x; e < n; e += blockDim.x) {
        int i = e / cols, j = e - i * cols;
        m = max(m, (uint32_t)ldg<uint16_t>(x + ((r0 + i) * d.sx_m + (c0 + j) * d.sx_n)) & 0x7FFFu);
    }
    m = wave64_max_u32(m);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    m = 0;
    for (int w = 0; w < kTileWaves; ++w) m = max(m, lds[w]);
    const Fp8BlockParams p = fp8_block_params<MODE>(m);
    if (threadIdx.x == 0) stg<float>(d.s + (tm * kt + tn), p.scale);
    uint8_t* y = (uint8_t*)d.y;
    for (int e = threadIdx.x; e < n; e += blockDim.x) {
        int i = e / cols, j = e - i * cols;
        float xv = u2f((uint32_t)ldg<uint16_t>(x + ((r0 + i) * d.sx_m + (c0 + j) * d.sx_n)) << 16);
        stg<uint8_t>(y + ((r0 + i) * d.sy_m + (c0 + j)), (uint8_t)fp8_quant1_exact<MODE>(xv, p));
    }
}

// GROUPED: 0 = one tensor in the kernel arguments, 1 = descriptor array + prefix sums (the owner of a tile is
// searched), 2 = one descriptor per tile, already moved to the tile's origin (a single scalar load, no search)
// SMALL: the single-wave form (see kSmallLaunchTiles)
template <int MODE, int GROUPED, bool SMALL = false>
__global__ __launch_bounds__(kTileThreads) void fp8_block_quant_kernel(const Fp8QuantArgs a, const int64_t total_tiles)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds[kRowSlots];
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_tiles) return;  // uniform per workgroup
    const int64_t tile = xcd_chunked_item(slot, total_tiles, kTilesPerXcdRun);

    wq_fp8_quant_desc d;
    int64_t local = tile;
    if (GROUPED == 1) {
        const int di = find_owner(a.tile_start, a.n_desc, tile, total_tiles);
        d = a.descs[di];
        local = tile - a.tile_start[di];
    } else if (GROUPED == 2) {
        d = a.descs[tile];      // M, N: what is left of the tensor from this tile's origin; s: this tile's slot
        local = 0;
        if (a.out_base) {
            d.y = a.out_base + (uintptr_t)d.y;
            d.s = (float*)(a.out_base + (uintptr_t)d.s);
        }
        if (d.sx_m == WQ_BUCKET_COPY_MARK) {       // pass-through item: M bytes from x to y
            copy_item(d.x, d.y, (int)d.M);
            return;
        }
    } else {
        d = a.d;
    }
    const int kt = GROUPED == 2 ? 1 : (int)((d.N + a.bn - 1) / a.bn);
    const int64_t tm = local / kt, tn = local - tm * kt;
    if (a.bm == 128 && a.bn == 128 && desc_vector_ok(d))
        quant_tile_vec128<MODE, SMALL ? kSmallTileWindow : kTileWindow>(d, tm, tn, kt, lds);
    else
        quant_tile_generic<MODE>(d, tm, tn, kt, a.bm, a.bn, lds);
}

// The per-tile form for tiles whose code rows do not start on 64-byte boundaries.  A tile's 128 codes of a row are one
// 128-byte line only when the tensor's rows start on line boundaries; in a buffer that packs tensors back to back they may
// not (a matrix with 280 tiles - DeepSeek-V3's [576, 7168] kv_a_proj_with_mqa - is followed by 1120 bytes of scales and
// leaves every later tensor of its bucket 96 bytes off).  Every row segment is then the end of one line and the start of
// the next, the neighbouring tile holds the rest of both, and streaming stores write each line to memory twice, in parts:
// 80 % of HBM peak drops to 55 % (32 bytes off) and 44 % (4 bytes off).  Plain stores let the L2 put the parts together -
// the neighbour is the next work item of the same XCD - and hold 65-70 % wherever the rows start.  Rows 64 bytes off keep
// the streaming stores (72 %, against 67 % plain).  A kernel of its own: with both store flavours in one kernel the aligned
// tiles lost 3.5 points to the second copy of the tile function.
template <int MODE>
__global__ __launch_bounds__(kTileThreads) void fp8_block_quant_plain_kernel(const Fp8QuantArgs a, const int64_t total_tiles)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds[kRowSlots];
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_tiles) return;  // uniform per workgroup
    const int64_t tile = xcd_chunked_item(slot, total_tiles, kTilesPerXcdRun);
    wq_fp8_quant_desc d = a.descs[tile];
    if (a.out_base) {
        d.y = a.out_base + (uintptr_t)d.y;
        d.s = (float*)(a.out_base + (uintptr_t)d.s);
    }
    if (d.sx_m == WQ_BUCKET_COPY_MARK) {
        copy_item(d.x, d.y, (int)d.M);
        return;
    }
    if (a.bm == 128 && a.bn == 128 && desc_vector_ok(d))
        quant_tile_vec128<MODE, kTileWindow, true>(d, 0, 0, 1, lds);
    else
        quant_tile_generic<MODE>(d, 0, 0, 1, a.bm, a.bn, lds);
}

// Up to WQ_FP8_FEW_MAX tensors with their descriptors in the kernel arguments: no device table to build, upload or keep.
// The owner of a tile is found by comparing against the (at most three) interior prefix sums and the descriptor is
// selected field by field, so everything stays in scalar registers (indexing the argument array with a run-time value
// would move it to scratch memory).
constexpr int kFewMax = WQ_FP8_FEW_MAX;
struct Fp8FewArgs {
    wq_fp8_quant_desc d[kFewMax];
    int64_t tile_start[kFewMax + 1];
    int32_t n_desc, bm, bn;
    char* out_base;      // when set, y and s of every descriptor are byte offsets from here
};

template <int MODE, bool SMALL>
__global__ __launch_bounds__(kTileThreads) void fp8_block_quant_few_kernel(const Fp8FewArgs a, const int64_t total_tiles)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds[kRowSlots];
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_tiles) return;  // uniform per workgroup
    const int64_t tile = xcd_chunked_item(slot, total_tiles, kTilesPerXcdRun);
    wq_fp8_quant_desc d = a.d[0];
    int64_t first = 0;
#pragma unroll
    for (int k = 1; k < kFewMax; ++k) {
        if (k < a.n_desc && tile >= a.tile_start[k]) {
            d = a.d[k];
            first = a.tile_start[k];
        }
    }
    if (a.out_base) {
        d.y = a.out_base + (uintptr_t)d.y;
        d.s = (float*)(a.out_base + (uintptr_t)d.s);
    }
    const int64_t local = tile - first;
    const int kt = (int)((d.N + a.bn - 1) / a.bn);
    const int64_t tm = local / kt, tn = local - tm * kt;
    if (a.bm == 128 && a.bn == 128 && desc_vector_ok(d))
        quant_tile_vec128<MODE, SMALL ? kSmallTileWindow : kTileWindow>(d, tm, tn, kt, lds);
    else
        quant_tile_generic<MODE>(d, tm, tn, kt, a.bm, a.bn, lds);
}

// ---- per-row (channel) and per-tensor scaling -------------------------------------------------

// The row and tensor forms exist only in the torch formulation; the scale rule is a run-time choice there.
__device__ __forceinline__ Fp8BlockParams torch_params(uint32_t amax_bf16_bits, int mode)
{
    return mode == WQ_FP8_MODE_TORCH_DEVICE ? fp8_block_params<WQ_FP8_MODE_TORCH_DEVICE>(amax_bf16_bits)
                                            : fp8_block_params<WQ_FP8_MODE_TORCH>(amax_bf16_bits);
}

// One workgroup per row: amax over the row, then quantise.  Second pass re-reads the row (L2).
__global__ __launch_bounds__(256) void fp8_row_quant_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t N,
                                                           int64_t sx_m, int64_t sx_n, uint8_t* __restrict__ y,
                                                           int64_t sy_m, float* __restrict__ s, int mode)
{
    __shared__ uint32_t lds[4];
    const int64_t row = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (row >= M) return;
    const uint16_t* xr = x + row * sx_m;
    uint32_t m = 0;
    for (int64_t j = threadIdx.x; j < N; j += 256) m = max(m, (uint32_t)xr[j * sx_n] & 0x7FFFu);
    m = wave64_max_u32(m);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    m = max(max(lds[0], lds[1]), max(lds[2], lds[3]));
    const Fp8BlockParams p = torch_params(m, mode);
    if (threadIdx.x == 0) s[row] = p.scale;
    uint8_t* yr = y + row * sy_m;
    for (int64_t j = threadIdx.x; j < N; j += 256)
        yr[j] = (uint8_t)fp8_elem_exact_torch(u2f((uint32_t)xr[j * sx_n] << 16), p.scale);
}

__global__ __launch_bounds__(256) void fp8_tensor_amax_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t N,
                                                             int64_t sx_m, int64_t sx_n, uint32_t* __restrict__ ws)
{
    __shared__ uint32_t lds[4];
    const int64_t total = M * N;
    uint32_t m = 0;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        int64_t i = e / N, j = e - i * N;
        m = max(m, (uint32_t)x[i * sx_m + j * sx_n] & 0x7FFFu);
    }
    m = wave64_max_u32(m);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(ws, max(max(lds[0], lds[1]), max(lds[2], lds[3])));
}

__global__ __launch_bounds__(256) void fp8_tensor_apply_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t N,
                                                              int64_t sx_m, int64_t sx_n, uint8_t* __restrict__ y,
                                                              int64_t sy_m, float* __restrict__ s,
                                                              const uint32_t* __restrict__ ws, int mode)
{
    const Fp8BlockParams p = torch_params(*ws, mode);
    if (blockIdx.x == 0 && threadIdx.x == 0) s[0] = p.scale;
    const int64_t total = M * N;
    // The reference divides a bf16 tensor by a 0-dim fp32 tensor, which torch evaluates as a bf16
    // result: the fp32 quotient is rounded to bf16 before the clamp and the e4m3 cast.  On GPU tensors
    // torch also converts the 0-dim divisor to the result dtype first, so the division there is by
    // bf16(scale) while the scale returned stays fp32.
    const float divisor = mode == WQ_FP8_MODE_TORCH_DEVICE ? u2f(f32_to_bf16_bits(p.scale) << 16) : p.scale;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        int64_t i = e / N, j = e - i * N;
        float q = u2f((uint32_t)x[i * sx_m + j * sx_n] << 16) / divisor;
        q = u2f(f32_to_bf16_bits(q) << 16);
        if (q == q) q = fminf(fmaxf(q, -kFp8Max), kFp8Max);
        y[i * sy_m + j] = (uint8_t)f32_to_e4m3fn_sw(q);
    }
}

// ---- per-row / per-tensor scale, contiguous operands ------------------------------------------------

constexpr int kRowsPerXcdRun = 32;
constexpr int kRowPieceElems = 256 * 8;      // elements of a row one load step of the workgroup covers

// One workgroup per row, the row held in registers (STEPS 16-byte pieces per lane, rows of up to 2048 * STEPS
// elements): amax, scale, and the same division-free element function as the block kernel - the scale rule and
// the (amax, x) domain are the block quantiser's, so the same exhaustive check covers it.
template <int STEPS>
__global__ __launch_bounds__(256) void fp8_row_quant_vec_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t N,
                                                               int64_t sx_m, uint8_t* __restrict__ y, int64_t sy_m,
                                                               float* __restrict__ s, int mode)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds[16];
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= M) return;
    const int64_t row = xcd_chunked_item(slot, M, kRowsPerXcdRun);
    const char* xr = (const char*)(x + row * sx_m);
    char* yr = (char*)(y + row * sy_m);
    const int n_pieces = (int)(N / 8);
    const int t = threadIdx.x;
    u32x4 v[STEPS];
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        // lanes past the end of the row re-read its last piece instead of branching around the load
        const int piece = min(i * 256 + t, n_pieces - 1);
        v[i] = ldg_nt<u32x4>(xr + (uint32_t)piece * 16u);
    }
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        if (i * 256 + t >= n_pieces) v[i] = (u32x4){0u, 0u, 0u, 0u};
        m = pk_absmax(m, v[i].x);
        m = pk_absmax(m, v[i].y);
        m = pk_absmax(m, v[i].z);
        m = pk_absmax(m, v[i].w);
    }
    m = row16_max_u32(pk_fold(m));
    if ((t & 15) == 0) lds[t >> 4] = m;
    __syncthreads();
    m = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32x4 a = ((const u32x4*)lds)[i];
        m = max(m, max(max(a.x, a.y), max(a.z, a.w)));
    }
    const Fp8BlockParams p = torch_params(m, mode);
    if (t == 0) stg<float>(s + row, p.scale);
    if (p.fast) {
#pragma unroll
        for (int i = 0; i < STEPS; ++i) {
            const int piece = i * 256 + t;
            u32x2 o;
            o.x = fp8_quant4_fast<WQ_FP8_MODE_TORCH>(v[i].x, v[i].y, p);
            o.y = fp8_quant4_fast<WQ_FP8_MODE_TORCH>(v[i].z, v[i].w, p);
            if (piece < n_pieces) stg_nt<u32x2>(yr + (uint32_t)piece * 8u, o);
        }
    } else {
        // NaN/Inf row (rare): literal arithmetic on re-read data
#pragma nounroll
        for (int i = 0; i < STEPS; ++i) {
            const int piece = i * 256 + t;
            if (piece >= n_pieces) continue;
            const u32x4 w = ldg<u32x4>(xr + (uint32_t)piece * 16u);
            u32x2 o;
            o.x = fp8_quant4_exact<WQ_FP8_MODE_TORCH>(w.x, w.y, p);
            o.y = fp8_quant4_exact<WQ_FP8_MODE_TORCH>(w.z, w.w, p);
            stg<u32x2>(yr + (uint32_t)piece * 8u, o);
        }
    }
}

// Rows of up to 8192 elements: one wavefront per row (four rows per workgroup), so that short rows still put
// 16 - 64 KiB per workgroup in flight; no LDS, no barrier.
constexpr int kWaveRowMaxSteps = 16;
__global__ __launch_bounds__(256) void fp8_row_quant_wave_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t N,
                                                                int64_t sx_m, uint8_t* __restrict__ y, int64_t sy_m,
                                                                float* __restrict__ s, int mode, int64_t items)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= items) return;
    const int64_t item = xcd_chunked_item(slot, items, kRowsPerXcdRun);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int64_t row = item * 4 + wave;
    if (row >= M) return;                                  // uniform per wavefront
    const char* xr = (const char*)(x + row * sx_m);
    char* yr = (char*)(y + row * sy_m);
    const int n_pieces = (int)(N / 8);
    const int steps = (n_pieces + 63) / 64;
    u32x4 v[kWaveRowMaxSteps];
#pragma unroll
    for (int i = 0; i < kWaveRowMaxSteps; ++i)
        if (i < steps) v[i] = ldg_nt<u32x4>(xr + (uint32_t)min(i * 64 + lane, n_pieces - 1) * 16u);
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < kWaveRowMaxSteps; ++i) {
        if (i < steps) {
            if (i * 64 + lane >= n_pieces) v[i] = (u32x4){0u, 0u, 0u, 0u};
            m = pk_absmax(m, v[i].x);
            m = pk_absmax(m, v[i].y);
            m = pk_absmax(m, v[i].z);
            m = pk_absmax(m, v[i].w);
        }
    }
    m = wave64_max_u32(pk_fold(m));
    const Fp8BlockParams p = torch_params(m, mode);
    if (lane == 0) stg<float>(s + row, p.scale);
    if (p.fast) {
#pragma unroll
        for (int i = 0; i < kWaveRowMaxSteps; ++i) {
            if (i < steps) {
                const int piece = i * 64 + lane;
                u32x2 o;
                o.x = fp8_quant4_fast<WQ_FP8_MODE_TORCH>(v[i].x, v[i].y, p);
                o.y = fp8_quant4_fast<WQ_FP8_MODE_TORCH>(v[i].z, v[i].w, p);
                if (piece < n_pieces) stg_nt<u32x2>(yr + (uint32_t)piece * 8u, o);
            }
        }
    } else {
        for (int piece = lane; piece < n_pieces; piece += 64) {
            const u32x4 w = ldg<u32x4>(xr + (uint32_t)piece * 16u);
            u32x2 o;
            o.x = fp8_quant4_exact<WQ_FP8_MODE_TORCH>(w.x, w.y, p);
            o.y = fp8_quant4_exact<WQ_FP8_MODE_TORCH>(w.z, w.w, p);
            stg<u32x2>(yr + (uint32_t)piece * 8u, o);
        }
    }
}

// Per-tensor amax of a contiguous tensor: a bounded grid, four 16-byte pieces per lane in flight, one atomic per
// workgroup.
__global__ __launch_bounds__(256) void fp8_tensor_amax_vec_kernel(const uint16_t* __restrict__ x, int64_t n_pieces,
                                                                 uint32_t* __restrict__ ws)
{
    __shared__ uint32_t lds[4];
    uint32_t m = 0;
    const char* xb = (const char*)x;
    for (int64_t p0 = (int64_t)blockIdx.x * 1024 + threadIdx.x; p0 < n_pieces; p0 += (int64_t)gridDim.x * 1024) {
        u32x4 v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = ldg_nt<u32x4>(xb + min(p0 + i * 256, n_pieces - 1) * 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // a piece past the end was read from the last valid one: harmless for a maximum
            m = pk_absmax(m, v[i].x);
            m = pk_absmax(m, v[i].y);
            m = pk_absmax(m, v[i].z);
            m = pk_absmax(m, v[i].w);
        }
    }
    m = wave64_max_u32(pk_fold(m));
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(ws, max(max(lds[0], lds[1]), max(lds[2], lds[3])));
}

typedef float f32x2q __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2q __attribute__((ext_vector_type(2)));

// Two elements of the per-tensor form: IEEE quotient, rounded to bf16 (the reference's bf16 tensor), NaN-propagating
// clamp, e4m3fn.  Returns the two codes in the low 16 bits.  FAST: the tensor's amax is finite, so |x / divisor| stays
// near 448 and the quotient comes from the correctly rounded reciprocal and two FMAs (exact for any divisor); that
// form turns -0 into +0, so the sign of x is put back on the code.
template <bool FAST>
__device__ __forceinline__ uint32_t tensor_quant2(uint32_t w, float divisor, float rcp)
{
    const float x0 = bf16lo(w), x1 = bf16hi(w);
    f32x2q q = {FAST ? div_by_scale(x0, divisor, rcp) : x0 / divisor, FAST ? div_by_scale(x1, divisor, rcp) : x1 / divisor};
    const uint32_t b = __builtin_bit_cast(uint32_t, __builtin_convertvector(q, bf16x2q));
    float q0 = bf16lo(b), q1 = bf16hi(b);
    if (FAST) {
        q0 = fminf(fmaxf(q0, -kFp8Max), kFp8Max);
        q1 = fminf(fmaxf(q1, -kFp8Max), kFp8Max);
        const uint32_t r = cvt_pk_fp8_lo(q0, q1, 0u) & 0x7F7Fu;
        return r | ((w >> 8) & 0x80u) | ((w >> 16) & 0x8000u);
    }
    const bool nan0 = q0 != q0, nan1 = q1 != q1;
    q0 = fminf(fmaxf(q0, -kFp8Max), kFp8Max);
    q1 = fminf(fmaxf(q1, -kFp8Max), kFp8Max);
    uint32_t r = cvt_pk_fp8_lo(q0, q1, 0u) & 0xFFFFu;
    if (nan0) r = (r & 0xFF00u) | 0x7Fu;
    if (nan1) r = (r & 0x00FFu) | 0x7F00u;
    return r;
}

__global__ __launch_bounds__(256) void fp8_tensor_apply_vec_kernel(const uint16_t* __restrict__ x, int64_t n_pieces,
                                                                  uint8_t* __restrict__ y, float* __restrict__ s,
                                                                  const uint32_t* __restrict__ ws, int mode,
                                                                  int64_t items)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= items) return;
    const int64_t item = xcd_chunked_item(slot, items, kRowsPerXcdRun);
    const Fp8BlockParams p = torch_params(*ws, mode);
    if (slot == 0 && threadIdx.x == 0) s[0] = p.scale;
    const float divisor = mode == WQ_FP8_MODE_TORCH_DEVICE ? u2f(f32_to_bf16_bits(p.scale) << 16) : p.scale;
    const char* xb = (const char*)x;
    const int64_t p0 = item * 1024 + threadIdx.x;
    u32x4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ldg_nt<u32x4>(xb + min(p0 + i * 256, n_pieces - 1) * 16);
    const float rcp = 1.0f / divisor;
    if (p.fast && divisor > 0x1p-100f) {      // finite amax, reciprocal a normal number
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t piece = p0 + i * 256;
            u32x2 o;
            o.x = tensor_quant2<true>(v[i].x, divisor, rcp) | (tensor_quant2<true>(v[i].y, divisor, rcp) << 16);
            o.y = tensor_quant2<true>(v[i].z, divisor, rcp) | (tensor_quant2<true>(v[i].w, divisor, rcp) << 16);
            if (piece < n_pieces) stg_nt<u32x2>(y + piece * 8, o);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t piece = p0 + i * 256;
            u32x2 o;
            o.x = tensor_quant2<false>(v[i].x, divisor, rcp) | (tensor_quant2<false>(v[i].y, divisor, rcp) << 16);
            o.y = tensor_quant2<false>(v[i].z, divisor, rcp) | (tensor_quant2<false>(v[i].w, divisor, rcp) << 16);
            if (piece < n_pieces) stg_nt<u32x2>(y + piece * 8, o);
        }
    }
}

// ---- block quant of fp16 / fp32 weights --------------------------------------------------------------
// The reference functions take any floating dtype; checkpoints and weight-sync buckets are bf16, so these
// dtypes get a plain two-pass tile kernel (second pass from L2) with the literal arithmetic: amax in the input
// dtype, the 1e-12 floor rounded to that dtype (0 for fp16: an all-zero fp16 block divides 0 by 0 in the
// reference, and here), fp32 from there on.
template <typename T> __device__ __forceinline__ float load_any(const void* p, int64_t off);
template <> __device__ __forceinline__ float load_any<float>(const void* p, int64_t off) { return ((const float*)p)[off]; }
template <> __device__ __forceinline__ float load_any<_Float16>(const void* p, int64_t off)
{
    return (float)((const _Float16*)p)[off];
}
template <> __device__ __forceinline__ float load_any<uint16_t>(const void* p, int64_t off)
{
    return u2f((uint32_t)((const uint16_t*)p)[off] << 16);
}
template <typename T> __device__ __forceinline__ float torch_floor_1em12();
template <> __device__ __forceinline__ float torch_floor_1em12<float>() { return 1e-12f; }
template <> __device__ __forceinline__ float torch_floor_1em12<_Float16>() { return 0.0f; }
template <> __device__ __forceinline__ float torch_floor_1em12<uint16_t>() { return u2f(kBf16Floor1em12 << 16); }

template <typename T, int MODE>
__global__ __launch_bounds__(256) void fp8_block_quant_any_kernel(const void* __restrict__ x, int64_t M, int64_t N,
                                                                 int64_t sx_m, int64_t sx_n, uint8_t* __restrict__ y,
                                                                 int64_t sy_m, float* __restrict__ s, int bm, int bn,
                                                                 int64_t total_tiles)
{
    __shared__ float lds[4];
    const int64_t tile = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (tile >= total_tiles) return;
    const int64_t kt = (N + bn - 1) / bn;
    const int64_t tm = tile / kt, tn = tile - tm * kt;
    const int64_t r0 = tm * bm, c0 = tn * bn;
    const int rows = (int)min((int64_t)bm, M - r0), cols = (int)min((int64_t)bn, N - c0);
    const int n = rows * cols;
    // NaN-propagating maximum of |x| (torch.max; the Triton reduction is not specified for NaN)
    float m = 0.0f;
    bool nan = false;
    for (int e = threadIdx.x; e < n; e += 256) {
        const int i = e / cols, j = e - i * cols;
        const float v = fabsf(load_any<T>(x, (r0 + i) * sx_m + (c0 + j) * sx_n));
        nan = nan || v != v;
        m = fmaxf(m, v);
    }
    m = nan ? __builtin_nanf("") : m;
    m = wave64_max_nanprop_f32(m);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    m = lds[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) m = (m != m || lds[w] != lds[w]) ? __builtin_nanf("") : fmaxf(m, lds[w]);
    float scale, inv = 0.0f;
    if (MODE == WQ_FP8_MODE_TRITON) {
        scale = (m != m ? m : fmaxf(m, 1e-10f)) / kFp8Max;
        inv = 1.0f / scale;
    } else {
        const float a = m != m ? m : fmaxf(m, torch_floor_1em12<T>());
        scale = MODE == WQ_FP8_MODE_TORCH_DEVICE ? a * (1.0f / kFp8Max) : a / kFp8Max;
    }
    if (threadIdx.x == 0) s[tile] = scale;
    for (int e = threadIdx.x; e < n; e += 256) {
        const int i = e / cols, j = e - i * cols;
        const float xv = load_any<T>(x, (r0 + i) * sx_m + (c0 + j) * sx_n);
        y[(r0 + i) * sy_m + (c0 + j)] = (uint8_t)(MODE == WQ_FP8_MODE_TRITON ? fp8_elem_exact_triton(xv, inv)
                                                                             : fp8_elem_exact_torch(xv, scale));
    }
}

template <typename T>
static void launch_block_quant_any(const void* x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, uint8_t* y,
                                   int64_t sy_m, float* s, int bm, int bn, int mode, hipStream_t st)
{
    const int64_t tiles = cdiv64(M, bm) * cdiv64(N, bn);
    const dim3 g = grid_for_items(tiles);
    if (mode == WQ_FP8_MODE_TORCH)
        fp8_block_quant_any_kernel<T, WQ_FP8_MODE_TORCH><<<g, 256, 0, st>>>(x, M, N, sx_m, sx_n, y, sy_m, s, bm, bn, tiles);
    else if (mode == WQ_FP8_MODE_TORCH_DEVICE)
        fp8_block_quant_any_kernel<T, WQ_FP8_MODE_TORCH_DEVICE><<<g, 256, 0, st>>>(x, M, N, sx_m, sx_n, y, sy_m, s, bm, bn, tiles);
    else
        fp8_block_quant_any_kernel<T, WQ_FP8_MODE_TRITON><<<g, 256, 0, st>>>(x, M, N, sx_m, sx_n, y, sy_m, s, bm, bn, tiles);
}

// tensor_fp8 on the other floating dtypes: `weight / scale` has the weight's dtype (the 0-dim fp32 scale does not take part
// in type promotion), so the fp32 quotient is rounded to it before the clamp - no second rounding for fp32 weights - and on
// GPU tensors the divisor is converted to it first.  Workspace: the fp32 bits of the NaN-propagating max |x| (for
// non-negative floats and NaNs the unsigned order of the bits is the order torch.max uses).
template <typename T> __device__ __forceinline__ float round_to(float v);
template <> __device__ __forceinline__ float round_to<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to<_Float16>(float v) { return (float)(_Float16)v; }
template <> __device__ __forceinline__ float round_to<uint16_t>(float v) { return u2f(f32_to_bf16_bits(v) << 16); }

template <typename T>
__global__ __launch_bounds__(256) void fp8_tensor_amax_any_kernel(const void* __restrict__ x, int64_t M, int64_t N,
                                                                 int64_t sx_m, int64_t sx_n, uint32_t* __restrict__ ws)
{
    __shared__ uint32_t lds[4];
    const int64_t total = M * N;
    uint32_t m = 0;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        const int64_t i = e / N, j = e - i * N;
        m = max(m, f2u(load_any<T>(x, i * sx_m + j * sx_n)) & 0x7FFFFFFFu);
    }
    m = wave64_max_u32(m);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(ws, max(max(lds[0], lds[1]), max(lds[2], lds[3])));
}

template <typename T>
__global__ __launch_bounds__(256) void fp8_tensor_apply_any_kernel(const void* __restrict__ x, int64_t M, int64_t N,
                                                                  int64_t sx_m, int64_t sx_n, uint8_t* __restrict__ y,
                                                                  int64_t sy_m, float* __restrict__ s,
                                                                  const uint32_t* __restrict__ ws, int mode)
{
    const float m = u2f(*ws);
    const float a = m != m ? m : fmaxf(m, torch_floor_1em12<T>());
    const float scale = mode == WQ_FP8_MODE_TORCH_DEVICE ? a * (1.0f / kFp8Max) : a / kFp8Max;
    if (blockIdx.x == 0 && threadIdx.x == 0) s[0] = scale;
    const float divisor = mode == WQ_FP8_MODE_TORCH_DEVICE ? round_to<T>(scale) : scale;
    const int64_t total = M * N;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        const int64_t i = e / N, j = e - i * N;
        float q = round_to<T>(load_any<T>(x, i * sx_m + j * sx_n) / divisor);
        if (q == q) q = fminf(fmaxf(q, -kFp8Max), kFp8Max);
        y[i * sy_m + j] = (uint8_t)f32_to_e4m3fn_sw(q);
    }
}

template <typename T>
static void launch_tensor_quant_any(const void* x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, uint8_t* y,
                                    int64_t sy_m, float* s, uint32_t* ws, int mode, hipStream_t st)
{
    const int blocks = (int)min((int64_t)(256 * 16), max((int64_t)1, cdiv64(M * N, 256 * 8)));
    fp8_tensor_amax_any_kernel<T><<<blocks, 256, 0, st>>>(x, M, N, sx_m, sx_n, ws);
    fp8_tensor_apply_any_kernel<T><<<blocks, 256, 0, st>>>(x, M, N, sx_m, sx_n, y, sy_m, s, ws, mode);
}

static bool known_mode(int mode)
{
    return mode == WQ_FP8_MODE_TORCH || mode == WQ_FP8_MODE_TRITON || mode == WQ_FP8_MODE_TORCH_DEVICE ||
           mode == WQ_FP8_MODE_UE8M0;
}

template <int MODE, int GROUPED>
static void launch_block_quant_mode(const Fp8QuantArgs& a, int64_t tiles, hipStream_t st)
{
    const dim3 g = grid_for_items(tiles);
    if (tiles <= kSmallLaunchTiles)
        fp8_block_quant_kernel<MODE, GROUPED, true><<<g, kTileThreads, kSmallOccupancyPadBytes, st>>>(a, tiles);
    else
        fp8_block_quant_kernel<MODE, GROUPED, false><<<g, kTileThreads, kOccupancyPadBytes, st>>>(a, tiles);
}

template <int GROUPED>
static void launch_block_quant(const Fp8QuantArgs& a, int64_t tiles, int mode, hipStream_t st)
{
    if (mode == WQ_FP8_MODE_TORCH) launch_block_quant_mode<WQ_FP8_MODE_TORCH, GROUPED>(a, tiles, st);
    else if (mode == WQ_FP8_MODE_TORCH_DEVICE) launch_block_quant_mode<WQ_FP8_MODE_TORCH_DEVICE, GROUPED>(a, tiles, st);
    else if (mode == WQ_FP8_MODE_UE8M0) launch_block_quant_mode<WQ_FP8_MODE_UE8M0, GROUPED>(a, tiles, st);
    else launch_block_quant_mode<WQ_FP8_MODE_TRITON, GROUPED>(a, tiles, st);
}

template <int MODE>
static void launch_block_quant_few_mode(const Fp8FewArgs& a, int64_t tiles, hipStream_t st)
{
    const dim3 g = grid_for_items(tiles);
    if (tiles <= kSmallLaunchTiles)
        fp8_block_quant_few_kernel<MODE, true><<<g, kTileThreads, kSmallOccupancyPadBytes, st>>>(a, tiles);
    else
        fp8_block_quant_few_kernel<MODE, false><<<g, kTileThreads, kOccupancyPadBytes, st>>>(a, tiles);
}

static int check_desc_host(const void* x, int64_t M, int64_t N, const void* y, const float* s, int bm, int bn, int mode)
{
    if (M < 0 || N < 0 || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (!known_mode(mode)) return WQ_ERR_MODE;
    if (M > 0 && N > 0 && (!x || !y || !s)) return WQ_ERR_NULL;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    return WQ_OK;
}

}  // namespace wq

using namespace wq;

WQ_EXPORT int wq_fp8_block_quant(const void* x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, void* y,
                                 int64_t sy_m, float* s, int bm, int bn, int mode, void* stream)
{
    int rc = check_desc_host(x, M, N, y, s, bm, bn, mode);
    if (rc) return rc;
    if (M == 0 || N == 0) return WQ_OK;
    Fp8QuantArgs a{};
    a.d = wq_fp8_quant_desc{x, y, s, M, N, sx_m, sx_n, sy_m};
    a.bm = bm;
    a.bn = bn;
    const int64_t tiles = cdiv64(M, bm) * cdiv64(N, bn);
    hipStream_t st = (hipStream_t)stream;
    launch_block_quant<0>(a, tiles, mode, st);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_block_quant_grouped(const wq_fp8_quant_desc* descs, const int64_t* tile_start, int n_desc,
                                         int64_t total_tiles, int bm, int bn, int mode, void* stream)
{
    if (n_desc < 0 || total_tiles < 0 || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (!known_mode(mode)) return WQ_ERR_MODE;
    if (n_desc == 0 || total_tiles == 0) return WQ_OK;
    if (!descs || !tile_start) return WQ_ERR_NULL;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    Fp8QuantArgs a{};
    a.descs = descs;
    a.tile_start = tile_start;
    a.n_desc = n_desc;
    a.bm = bm;
    a.bn = bn;
    hipStream_t st = (hipStream_t)stream;
    launch_block_quant<1>(a, total_tiles, mode, st);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_row_quant(const void* x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, void* y,
                               int64_t sy_m, float* s, int mode, void* stream)
{
    if (M < 0 || N < 0) return WQ_ERR_SHAPE;
    if (mode != WQ_FP8_MODE_TORCH && mode != WQ_FP8_MODE_TORCH_DEVICE) return WQ_ERR_MODE;
    if (M == 0) return WQ_OK;
    if (!s || (N > 0 && (!x || !y))) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = sx_n == 1 && N > 0 && (N & 7) == 0 && N <= 8 * kRowPieceElems && (sx_m & 7) == 0 && (sy_m & 7) == 0 &&
                     ((uintptr_t)x & 15) == 0 && ((uintptr_t)y & 7) == 0;
    const uint16_t* xp = (const uint16_t*)x;
    uint8_t* yp = (uint8_t*)y;
    const dim3 g = grid_for_items(M);
    if (!vec) fp8_row_quant_kernel<<<g, 256, 0, st>>>(xp, M, N, sx_m, sx_n, yp, sy_m, s, mode);
    else if (N <= 8 * 64 * kWaveRowMaxSteps) {
        const int64_t items = cdiv64(M, 4);
        fp8_row_quant_wave_kernel<<<grid_for_items(items), 256, 0, st>>>(xp, M, N, sx_m, yp, sy_m, s, mode, items);
    }
    else if (N <= kRowPieceElems) fp8_row_quant_vec_kernel<1><<<g, 256, 0, st>>>(xp, M, N, sx_m, yp, sy_m, s, mode);
    else if (N <= 2 * kRowPieceElems) fp8_row_quant_vec_kernel<2><<<g, 256, 0, st>>>(xp, M, N, sx_m, yp, sy_m, s, mode);
    else if (N <= 4 * kRowPieceElems) fp8_row_quant_vec_kernel<4><<<g, 256, 0, st>>>(xp, M, N, sx_m, yp, sy_m, s, mode);
    else fp8_row_quant_vec_kernel<8><<<g, 256, 0, st>>>(xp, M, N, sx_m, yp, sy_m, s, mode);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_tensor_quant(const void* x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, void* y,
                                  int64_t sy_m, float* s, uint32_t* workspace, int mode, void* stream)
{
    if (M < 0 || N < 0) return WQ_ERR_SHAPE;
    if (mode != WQ_FP8_MODE_TORCH && mode != WQ_FP8_MODE_TORCH_DEVICE) return WQ_ERR_MODE;
    if (!s || !workspace || (M * N > 0 && (!x || !y))) return WQ_ERR_NULL;
    const int64_t total = M * N;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = total > 0 && sx_n == 1 && sx_m == N && sy_m == N && (total & 7) == 0 && ((uintptr_t)x & 15) == 0 &&
                     ((uintptr_t)y & 7) == 0;
    if (vec) {
        const int64_t n_pieces = total / 8;
        const int64_t items = cdiv64(n_pieces, 1024);
        const int blocks = (int)min((int64_t)2048, items);
        fp8_tensor_amax_vec_kernel<<<blocks, 256, 0, st>>>((const uint16_t*)x, n_pieces, workspace);
        WQ_LAUNCH_CHECK();
        fp8_tensor_apply_vec_kernel<<<grid_for_items(items), 256, 0, st>>>((const uint16_t*)x, n_pieces, (uint8_t*)y, s,
                                                                          workspace, mode, items);
        WQ_LAUNCH_CHECK();
        return WQ_OK;
    }
    int blocks = (int)min((int64_t)(256 * 16), max((int64_t)1, cdiv64(total, 256 * 8)));
    fp8_tensor_amax_kernel<<<blocks, 256, 0, st>>>((const uint16_t*)x, M, N, sx_m, sx_n, workspace);
    WQ_LAUNCH_CHECK();
    fp8_tensor_apply_kernel<<<blocks, 256, 0, st>>>((const uint16_t*)x, M, N, sx_m, sx_n, (uint8_t*)y, sy_m, s,
                                                   workspace, mode);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_block_quant_any(const void* x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, void* y,
                                     int64_t sy_m, float* s, int bm, int bn, int mode, void* stream)
{
    if (dtype != WQ_DTYPE_BF16 && dtype != WQ_DTYPE_F32 && dtype != WQ_DTYPE_F16) return WQ_ERR_MODE;
    int rc = check_desc_host(x, M, N, y, s, bm, bn, mode);
    if (rc) return rc;
    if (mode == WQ_FP8_MODE_UE8M0) return WQ_ERR_UNSUPPORTED;      // power-of-two scales: bf16 weights only
    if (M == 0 || N == 0) return WQ_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == WQ_DTYPE_F32) launch_block_quant_any<float>(x, M, N, sx_m, sx_n, (uint8_t*)y, sy_m, s, bm, bn, mode, st);
    else if (dtype == WQ_DTYPE_F16) launch_block_quant_any<_Float16>(x, M, N, sx_m, sx_n, (uint8_t*)y, sy_m, s, bm, bn, mode, st);
    else launch_block_quant_any<uint16_t>(x, M, N, sx_m, sx_n, (uint8_t*)y, sy_m, s, bm, bn, mode, st);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_tensor_quant_any(const void* x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, void* y,
                                      int64_t sy_m, float* s, uint32_t* workspace, int mode, void* stream)
{
    if (dtype == WQ_DTYPE_BF16) return wq_fp8_tensor_quant(x, M, N, sx_m, sx_n, y, sy_m, s, workspace, mode, stream);
    if (dtype != WQ_DTYPE_F32 && dtype != WQ_DTYPE_F16) return WQ_ERR_MODE;
    if (M < 0 || N < 0) return WQ_ERR_SHAPE;
    if (mode != WQ_FP8_MODE_TORCH && mode != WQ_FP8_MODE_TORCH_DEVICE) return WQ_ERR_MODE;
    if (!s || !workspace || (M * N > 0 && (!x || !y))) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == WQ_DTYPE_F32) launch_tensor_quant_any<float>(x, M, N, sx_m, sx_n, (uint8_t*)y, sy_m, s, workspace, mode, st);
    else launch_tensor_quant_any<_Float16>(x, M, N, sx_m, sx_n, (uint8_t*)y, sy_m, s, workspace, mode, st);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_bucket_convert(const wq_fp8_quant_desc* items, int64_t n_items, void* out_base, int bm, int bn,
                                    int mode, void* stream)
{
    if (n_items < 0 || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (!known_mode(mode)) return WQ_ERR_MODE;
    if (n_items == 0) return WQ_OK;
    if (!items || !out_base) return WQ_ERR_NULL;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    Fp8QuantArgs a{};
    a.descs = items;
    a.bm = bm;
    a.bn = bn;
    a.out_base = (char*)out_base;
    launch_block_quant<2>(a, n_items, mode, (hipStream_t)stream);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_block_quant_tiles(const wq_fp8_quant_desc* tiles, int64_t n_tiles, int bm, int bn, int mode,
                                       void* stream)
{
    if (n_tiles < 0 || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (!known_mode(mode)) return WQ_ERR_MODE;
    if (n_tiles == 0) return WQ_OK;
    if (!tiles) return WQ_ERR_NULL;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    Fp8QuantArgs a{};
    a.descs = tiles;
    a.bm = bm;
    a.bn = bn;
    launch_block_quant<2>(a, n_tiles, mode, (hipStream_t)stream);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_block_quant_few(const wq_fp8_quant_desc* descs, int n_desc, void* out_base, int bm, int bn, int mode,
                                     void* stream)
{
    if (n_desc < 0 || n_desc > kFewMax || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (!known_mode(mode)) return WQ_ERR_MODE;
    if (n_desc == 0) return WQ_OK;
    if (!descs) return WQ_ERR_NULL;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    Fp8FewArgs a{};
    int64_t tiles = 0;
    int n = 0;
    for (int i = 0; i < n_desc; ++i) {          // `descs` is host memory: checked and copied into the kernel arguments
        const wq_fp8_quant_desc& d = descs[i];
        if (d.M < 0 || d.N < 0) return WQ_ERR_SHAPE;
        if (d.M == 0 || d.N == 0) continue;
        if (!d.x || (!out_base && (!d.y || !d.s))) return WQ_ERR_NULL;
        a.d[n] = d;
        a.tile_start[n] = tiles;
        tiles += cdiv64(d.M, bm) * cdiv64(d.N, bn);
        ++n;
    }
    if (n == 0) return WQ_OK;
    for (int i = n; i <= kFewMax; ++i) a.tile_start[i] = tiles;
    a.n_desc = n;
    a.bm = bm;
    a.bn = bn;
    a.out_base = (char*)out_base;
    hipStream_t st = (hipStream_t)stream;
    if (mode == WQ_FP8_MODE_TORCH) launch_block_quant_few_mode<WQ_FP8_MODE_TORCH>(a, tiles, st);
    else if (mode == WQ_FP8_MODE_TORCH_DEVICE) launch_block_quant_few_mode<WQ_FP8_MODE_TORCH_DEVICE>(a, tiles, st);
    else if (mode == WQ_FP8_MODE_UE8M0) launch_block_quant_few_mode<WQ_FP8_MODE_UE8M0>(a, tiles, st);
    else launch_block_quant_few_mode<WQ_FP8_MODE_TRITON>(a, tiles, st);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_bucket_convert_rows_off_lines(const wq_fp8_quant_desc* items, int64_t n_items, void* out_base, int bm,
                                                   int bn, int mode, void* stream)
{
    if (n_items < 0 || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (!known_mode(mode)) return WQ_ERR_MODE;
    if (n_items == 0) return WQ_OK;
    if (!items || !out_base) return WQ_ERR_NULL;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    Fp8QuantArgs a{};
    a.descs = items;
    a.bm = bm;
    a.bn = bn;
    a.out_base = (char*)out_base;
    const dim3 g = grid_for_items(n_items);
    hipStream_t st = (hipStream_t)stream;
    if (mode == WQ_FP8_MODE_TORCH) fp8_block_quant_plain_kernel<WQ_FP8_MODE_TORCH><<<g, kTileThreads, kOccupancyPadBytes, st>>>(a, n_items);
    else if (mode == WQ_FP8_MODE_TORCH_DEVICE) fp8_block_quant_plain_kernel<WQ_FP8_MODE_TORCH_DEVICE><<<g, kTileThreads, kOccupancyPadBytes, st>>>(a, n_items);
    else if (mode == WQ_FP8_MODE_UE8M0) fp8_block_quant_plain_kernel<WQ_FP8_MODE_UE8M0><<<g, kTileThreads, kOccupancyPadBytes, st>>>(a, n_items);
    else fp8_block_quant_plain_kernel<WQ_FP8_MODE_TRITON><<<g, kTileThreads, kOccupancyPadBytes, st>>>(a, n_items);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}
