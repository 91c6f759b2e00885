// block-FP8 (e4m3fn) -> bf16 dequantisation for gfx950.
//
// The tensor is cut into row segments of WQ_DEQ_SEG codes; a work item is WQ_DEQ_SEGS_PER_WG consecutive
// segments (rows are contiguous, so for N a multiple of the segment this is one contiguous 8 KiB run of
// input and 16 KiB of output) handled by a 256-thread workgroup.  A wavefront takes one segment per step:
// every lane loads 8 codes (8 bytes, the wave reads 512 contiguous bytes) and stores the 8 bf16 they
// become as ONE 16-byte store, so the wave writes 1 KiB contiguous per store instruction - split
// 16-byte halves per lane measured ~20 % slower.  All loads of a lane (codes and their block scales) are issued
// before the first use.  Codes are expanded with v_cvt_pk_f32_fp8, multiplied by the block's fp32 scale and rounded once
// to bf16 (v_cvt_pk_bf16_f32, RNE): the single rounding of the reference's y = x.to(f32) * s stored to bf16.

#include "wq_common.h"

namespace wq {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kSeg = WQ_DEQ_SEG;                 // codes per segment: 64 lanes x 8
constexpr int kSegsPerWg = WQ_DEQ_SEGS_PER_WG;   // 4 waves x kSteps
constexpr int kSteps = kSegsPerWg / 4;           // loads in flight per lane
// Measured on the DeepSeek-V3-shaped layer (768 tensors, one grouped launch; % of the 8 TB/s HBM peak):
// segments per workgroup x resident workgroups per CU: 32x8 74.0, 32x4 79.3, 16x8 76.5, 16x5 79.4 (used),
// 16x4 78.2, 8x8 79.7, 8x5 73.1.  A compute-free kernel with the same 1:2 read:write mix tops out at 83 %.
constexpr int kDeqItemsPerXcdRun = 32;
constexpr int kDeqWindow = 4;                          // steps whose loads are in flight (kSteps = all)
constexpr unsigned kDeqOccupancyPadBytes = 27 * 1024;  // unused dynamic LDS: at most 5 workgroups per CU
// A launch of at most this many work items ([4096, 4096] is 2048) fits the chip at full occupancy in one wave of
// workgroups; capped at 5 per CU it would run as one full wave and a partial one.  Such launches run uncapped
// ([4096, 4096], launches back to back: 12.3 -> 11.0 us; larger launches do not change).
constexpr int64_t kDeqSmallLaunchItems = 2048;
static_assert(kSeg == 512 && kSegsPerWg % 4 == 0, "a segment is 64 lanes x 8 codes; four waves per workgroup");

struct DeqArgs {
    wq_fp8_dequant_desc d;
    const wq_fp8_dequant_desc* descs;
    const int64_t* work_start;
    int32_t n_desc;
    int32_t block;
    const wq_fp8_dequant_item* items;     // per-item form
};

// RNE fp32 -> bf16 for two values packed in a dword (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b)
{
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

template <int MODE>
__device__ __forceinline__ float load_scale(const float* __restrict__ s, int64_t idx)
{
    float v = ldg<float>(s + idx);      // never a flat access: see the note at the element-wise path below
    if (MODE == WQ_DEQ_MODE_BF16SCALE) v = u2f(f32_to_bf16_bits(v) << 16);
    return v;
}

// four codes (one dword) -> four bf16 (two dwords)
__device__ __forceinline__ u32x2 dequant4(uint32_t codes, float sc)
{
    f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, false);
    f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, true);
    u32x2 o;
    o.x = pack_bf16x2(lo.x * sc, lo.y * sc);
    o.y = pack_bf16x2(hi.x * sc, hi.y * sc);
    return o;
}

// RNE fp32 -> fp16 for two values packed in a dword (two v_cvt_f16_f32; the packed conversion rounds toward zero).
// The empty asm keeps the fp32 product a value of its own: left alone, the compiler folds "convert(a * b)" into
// v_fma_mixlo_f16 a, b, 0, which rounds the exact product once (the reference rounds it to fp32 first) and turns a
// product of -0 into +0.
__device__ __forceinline__ uint32_t pack_f16x2(float a, float b)
{
    asm volatile("" : "+v"(a), "+v"(b));
    const _Float16 ha = (_Float16)a, hb = (_Float16)b;
    return (uint32_t)__builtin_bit_cast(uint16_t, ha) | ((uint32_t)__builtin_bit_cast(uint16_t, hb) << 16);
}

__device__ __forceinline__ u32x2 dequant4_f16(uint32_t codes, float sc)
{
    f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, false);
    f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, true);
    u32x2 o;
    o.x = pack_f16x2(lo.x * sc, lo.y * sc);
    o.y = pack_f16x2(hi.x * sc, hi.y * sc);
    return o;
}

__device__ __forceinline__ f32x4 dequant4_f32(uint32_t codes, float sc)
{
    f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, false);
    f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, true);
    return (f32x4){lo.x * sc, lo.y * sc, hi.x * sc, hi.y * sc};
}

// OUT: WQ_DTYPE_BF16 (the reference tool's default dtype), WQ_DTYPE_F16 (product rounded once to fp16) or WQ_DTYPE_F32
// (the un-rounded product).
// GROUPED: 0 = one tensor in the kernel arguments, 1 = descriptor array + prefix sums (the owner of a work item is
// searched), 2 = one pre-resolved descriptor per work item (a single scalar load, no search)
template <int MODE, int GROUPED, int OUT>
__global__ __launch_bounds__(256) void fp8_block_dequant_kernel(const DeqArgs a, const int64_t total_work)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_work) return;
    const int64_t item = xcd_chunked_item(slot, total_work, kDeqItemsPerXcdRun);
    wq_fp8_dequant_desc d;
    int64_t local = item;
    if (GROUPED == 1) {
        const int di = find_owner(a.work_start, a.n_desc, item, total_work);
        d = a.descs[di];
        local = item - a.work_start[di];
    } else if (GROUPED == 2) {
        const wq_fp8_dequant_item it = a.items[item];
        d = wq_fp8_dequant_desc{it.x, it.s, it.y, it.M, it.N};
        local = it.item;
    } else {
        d = a.d;
    }
    // 32-bit index arithmetic: N and the tensor's segment count are below 2^31 (checked on the host)
    const uint32_t block = (uint32_t)a.block;
    const int bshift = (block & (block - 1)) == 0 ? __builtin_ctz(block) : -1;   // power-of-two blocks shift
    const uint32_t N = (uint32_t)d.N;
    const uint32_t spr = (N + kSeg - 1) / kSeg;          // segments per row
    const uint32_t n_segs = (uint32_t)d.M * spr;
    const uint32_t kt = (N + block - 1) / block;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const uint8_t* x = (const uint8_t*)d.x;
    const bool vec = (N & 7) == 0 && ((uintptr_t)d.x & 7) == 0 && ((uintptr_t)d.y & 15) == 0 && (block & 7) == 0;
    // segment of step i is seg0 + 4i: consecutive segments go to consecutive waves, so one step of the
    // workgroup covers four consecutive segments.  (row, segment-in-row) advance incrementally.
    const uint32_t seg0 = (uint32_t)local * kSegsPerWg + wave;
    uint32_t r = seg0 / spr, c = seg0 - r * spr;

    if (vec) {
        u32x2 v[kSteps];
        float sc[kSteps];
        uint32_t row[kSteps], col[kSteps];
        bool ok[kSteps];
        // The loads of the workgroup's strip - codes and their block scales - run kDeqWindow steps ahead of their
        // use.  Lanes with nothing to do read the tensor's first codes / scale instead of branching
        // around the load: a predicated load makes the compiler wait for earlier loads first.
        auto issue = [&](int i) {
            row[i] = r;
            col[i] = c * kSeg + lane * 8;
            ok[i] = seg0 + 4 * i < n_segs && col[i] < N;
            v[i] = ldg_nt<u32x2>(x + (ok[i] ? (uint64_t)row[i] * N + col[i] : 0));
            const uint32_t sr = bshift >= 0 ? row[i] >> bshift : row[i] / block;
            const uint32_t sc_col = bshift >= 0 ? col[i] >> bshift : col[i] / block;
            sc[i] = ldg<float>(d.s + (ok[i] ? sr * kt + sc_col : 0));
            c += 4;
            while (c >= spr) { c -= spr; ++r; }
        };
#pragma unroll
        for (int i = 0; i < kDeqWindow && i < kSteps; ++i) issue(i);
#pragma unroll
        for (int i = 0; i < kSteps; ++i) {
            if (kDeqWindow < kSteps) {
                asm volatile("" :: "v"(v[i].x), "v"(sc[i]));
                if (i + kDeqWindow < kSteps) issue(i + kDeqWindow);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (!ok[i]) continue;
            if (MODE == WQ_DEQ_MODE_BF16SCALE) sc[i] = u2f(f32_to_bf16_bits(sc[i]) << 16);
            const uint64_t off = (uint64_t)row[i] * N + col[i];
            if (OUT == WQ_DTYPE_BF16 || OUT == WQ_DTYPE_F16) {
                const u32x2 a0 = OUT == WQ_DTYPE_BF16 ? dequant4(v[i].x, sc[i]) : dequant4_f16(v[i].x, sc[i]);
                const u32x2 a1 = OUT == WQ_DTYPE_BF16 ? dequant4(v[i].y, sc[i]) : dequant4_f16(v[i].y, sc[i]);
                const u32x4 o = {a0.x, a0.y, a1.x, a1.y};
                stg_nt<u32x4>((uint16_t*)d.y + off, o);
            } else {
                f32x4* yp = (f32x4*)((float*)d.y + off);
                stg_nt<f32x4>(yp, dequant4_f32(v[i].x, sc[i]));
                stg_nt<f32x4>(yp + 1, dequant4_f32(v[i].y, sc[i]));
            }
        }
    } else {
        // element-wise path: any N, alignment and block size.  Global-address-space accesses like everywhere else: a flat
        // (generic-pointer) access anywhere in the kernel makes the compiler drain every outstanding memory operation
        // (vmcnt(0)) at each wait of the vector path above, which then sends its four stores one round trip at a time.
#pragma nounroll
        for (int i = 0; i < kSteps; ++i) {
            if (seg0 + 4 * i >= n_segs) break;
#pragma nounroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t cc = c * kSeg + k * 64 + lane;
                if (cc >= N) break;
                const float sc = load_scale<MODE>(d.s, (r / block) * kt + cc / block);
                const uint64_t off = (uint64_t)r * N + cc;
                const uint32_t code = ldg<uint8_t>(x + off);
                const f32x2 f = __builtin_amdgcn_cvt_pk_f32_fp8((int)code, false);
                if (OUT == WQ_DTYPE_BF16) stg<uint16_t>((uint16_t*)d.y + off, (uint16_t)(pack_bf16x2(f.x * sc, 0.0f) & 0xFFFFu));
                else if (OUT == WQ_DTYPE_F16) stg<uint16_t>((uint16_t*)d.y + off, (uint16_t)(pack_f16x2(f.x * sc, 0.0f) & 0xFFFFu));
                else stg<float>((float*)d.y + off, f.x * sc);
            }
            c += 4;
            while (c >= spr) { c -= spr; ++r; }
        }
    }
}

static inline int64_t deq_work_items(int64_t M, int64_t N)
{
    return cdiv64(M * cdiv64(N, kSeg), kSegsPerWg);
}

}  // namespace wq

using namespace wq;

template <int GROUPED>
static int launch_deq(const DeqArgs& a, int64_t work, int mode, int out_dtype, hipStream_t st)
{
    const dim3 g = grid_for_items(work);
    const unsigned kDeqOccupancyPadBytes = work <= kDeqSmallLaunchItems ? 0u : wq::kDeqOccupancyPadBytes;
    if (mode == WQ_DEQ_MODE_F32SCALE) {
        if (out_dtype == WQ_DTYPE_BF16) fp8_block_dequant_kernel<WQ_DEQ_MODE_F32SCALE, GROUPED, WQ_DTYPE_BF16><<<g, 256, kDeqOccupancyPadBytes, st>>>(a, work);
        else if (out_dtype == WQ_DTYPE_F16) fp8_block_dequant_kernel<WQ_DEQ_MODE_F32SCALE, GROUPED, WQ_DTYPE_F16><<<g, 256, kDeqOccupancyPadBytes, st>>>(a, work);
        else fp8_block_dequant_kernel<WQ_DEQ_MODE_F32SCALE, GROUPED, WQ_DTYPE_F32><<<g, 256, kDeqOccupancyPadBytes, st>>>(a, work);
    } else {
        if (out_dtype == WQ_DTYPE_BF16) fp8_block_dequant_kernel<WQ_DEQ_MODE_BF16SCALE, GROUPED, WQ_DTYPE_BF16><<<g, 256, kDeqOccupancyPadBytes, st>>>(a, work);
        else fp8_block_dequant_kernel<WQ_DEQ_MODE_BF16SCALE, GROUPED, WQ_DTYPE_F32><<<g, 256, kDeqOccupancyPadBytes, st>>>(a, work);
    }
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

static int check_deq(int64_t block, int mode, int out_dtype)
{
    if (block <= 0) return WQ_ERR_SHAPE;
    if (mode != WQ_DEQ_MODE_F32SCALE && mode != WQ_DEQ_MODE_BF16SCALE) return WQ_ERR_MODE;
    if (out_dtype != WQ_DTYPE_BF16 && out_dtype != WQ_DTYPE_F32 && out_dtype != WQ_DTYPE_F16) return WQ_ERR_MODE;
    if (out_dtype == WQ_DTYPE_F16 && mode != WQ_DEQ_MODE_F32SCALE) return WQ_ERR_UNSUPPORTED;   // the loader's variant is bf16
    return WQ_OK;
}

WQ_EXPORT int wq_fp8_block_dequant(const void* x, const float* s, void* y, int out_dtype, int64_t M, int64_t N,
                                   int block, int mode, void* stream)
{
    if (M < 0 || N < 0) return WQ_ERR_SHAPE;
    int rc = check_deq(block, mode, out_dtype);
    if (rc) return rc;
    if (M == 0 || N == 0) return WQ_OK;
    if (!x || !s || !y) return WQ_ERR_NULL;
    // the kernel indexes rows, columns and segments with 32-bit integers
    if (N >= (1ll << 31) || M >= (1ll << 31) || M * cdiv64(N, kSeg) >= (1ll << 31)) return WQ_ERR_TOO_LARGE;
    DeqArgs a{};
    a.d = wq_fp8_dequant_desc{x, s, y, M, N};
    a.block = block;
    return launch_deq<0>(a, deq_work_items(M, N), mode, out_dtype, (hipStream_t)stream);
}

WQ_EXPORT int wq_fp8_block_dequant_grouped(const wq_fp8_dequant_desc* descs, const int64_t* work_start, int n_desc,
                                           int64_t total_work, int out_dtype, int block, int mode, void* stream)
{
    if (n_desc < 0 || total_work < 0) return WQ_ERR_SHAPE;
    int rc = check_deq(block, mode, out_dtype);
    if (rc) return rc;
    if (n_desc == 0 || total_work == 0) return WQ_OK;
    if (!descs || !work_start) return WQ_ERR_NULL;
    DeqArgs a{};
    a.descs = descs;
    a.work_start = work_start;
    a.n_desc = n_desc;
    a.block = block;
    return launch_deq<1>(a, total_work, mode, out_dtype, (hipStream_t)stream);
}

WQ_EXPORT int wq_fp8_block_dequant_items(const wq_fp8_dequant_item* items, int64_t n_items, int out_dtype, int block,
                                         int mode, void* stream)
{
    if (n_items < 0) return WQ_ERR_SHAPE;
    int rc = check_deq(block, mode, out_dtype);
    if (rc) return rc;
    if (n_items == 0) return WQ_OK;
    if (!items) return WQ_ERR_NULL;
    DeqArgs a{};
    a.items = items;
    a.block = block;
    return launch_deq<2>(a, n_items, mode, out_dtype, (hipStream_t)stream);
}
