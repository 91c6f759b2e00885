// bf16 -> block-FP8 -> bf16 in one pass ("FP8-aligned" weights) for gfx950.
//
// A trainer that wants its bf16 weight to carry exactly the values the rollout engine sees after FP8 quantisation
// calls the block quantiser and then the block dequantiser (slime_plugins/models/glm5/glm5.py:105-165:
// blockwise_cast_to_fp8_triton or quant_weight_ue8m0, then block_quant_dequant to bf16).  The two passes move
// 3 + 3 bytes per element and materialise the codes; this kernel moves 2 + 2: the 128x128 block is loaded into
// registers exactly as in the quantiser (eight 16-byte loads per lane, all in flight), amax / scale / codes are
// computed by the quantiser's own element functions, and each group of four codes is expanded again
// (v_cvt_pk_f32_fp8), multiplied by the block scale and rounded once to bf16 (v_cvt_pk_bf16_f32) - the
// dequantiser's arithmetic - before a single 16-byte store per piece.  Results are bit-identical to running the
// two kernels one after the other; the scale tensor is written only when the caller asks for it.

#include "wq_common.h"

namespace wq {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kFakeThreads = 256;
constexpr int kFakeRowSlots = kFakeThreads / 16;
constexpr int kFakeLoads = 128 / kFakeRowSlots;
// Measured on one [151936, 2560] tensor (% of the 8 TB/s HBM peak at 4 bytes per element; the plain copy kernel reaches
// 73-78 % on the same box): resident workgroups per CU 8: 72.7, 7: 73.5, 5: 74.7, 4: 74.4, 3: 75.5 (used); runs of
// 8 / 16 / 32 / 64 tiles per XCD: 73.5 / 74.2 / 74.4 / 74.1.  The quantiser followed by the dequantiser: 78.8 % of their
// 6 bytes per element, i.e. 1.42x the time.
constexpr int kFakeTilesPerXcdRun = 32;
constexpr int kFakeWindow = 8;                          // 16-byte loads in flight per lane (8 = the whole tile)
constexpr unsigned kFakeOccupancyPadBytes = 50 * 1024;  // unused dynamic LDS: at most 3 workgroups per CU

struct FakeArgs {
    const uint16_t* x;
    uint16_t* y;
    float* s;  // may be null
    int64_t M, N, sx_m, sx_n, sy_m;
    int32_t bm, bn;
};

__device__ __forceinline__ uint32_t pack_bf16x2_rne(float a, float b)
{
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// four codes (one dword) -> four bf16 (two dwords): f32(code) * scale, one rounding
__device__ __forceinline__ u32x2 expand4(uint32_t codes, float sc)
{
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, true);
    u32x2 o;
    o.x = pack_bf16x2_rne(lo.x * sc, lo.y * sc);
    o.y = pack_bf16x2_rne(hi.x * sc, hi.y * sc);
    return o;
}

template <int MODE>
__device__ __forceinline__ void fake_tile_vec128(const FakeArgs& a, int64_t tm, int64_t tn, int kt, uint32_t* lds)
{
    const int t = threadIdx.x;
    const int cc = t & 15, rb = t >> 4;
    const char* xt = (const char*)a.x + (tm * 128 * a.sx_m + tn * 128) * 2;
    char* yt = (char*)a.y + (tm * 128 * a.sy_m + tn * 128) * 2;
    const uint32_t xrow = (uint32_t)a.sx_m * 2u, yrow = (uint32_t)a.sy_m * 2u;
    const int rows = (int)min((int64_t)128, a.M - tm * 128);
    const int pieces = (int)min((int64_t)16, (a.N - tn * 128) >> 3);
    const bool col_ok = cc < pieces;
    const bool full = rows == 128 && pieces == 16;
    const uint32_t coff = (uint32_t)min(cc, pieces - 1) * 16u;

    // every lane loads from a valid address (row and piece clamped into the tile); lanes outside the tensor are zeroed.
    // Full tiles keep kFakeWindow loads in flight per lane while the block maximum is folded (see the quantiser).
    u32x4 v[kFakeLoads];
    uint32_t m = 0;
    if (full) {
#pragma unroll
        for (int i = 0; i < kFakeWindow && i < kFakeLoads; ++i)
            v[i] = ldg_nt<u32x4>(xt + ((uint32_t)(rb + kFakeRowSlots * i) * xrow + coff));
#pragma unroll
        for (int i = 0; i < kFakeLoads; ++i) {
            m = pk_absmax(m, v[i].x);
            m = pk_absmax(m, v[i].y);
            m = pk_absmax(m, v[i].z);
            m = pk_absmax(m, v[i].w);
            __builtin_amdgcn_sched_barrier(0);
            if (i + kFakeWindow < kFakeLoads)
                v[i + kFakeWindow] = ldg_nt<u32x4>(xt + ((uint32_t)(rb + kFakeRowSlots * (i + kFakeWindow)) * xrow + coff));
        }
    } else {
#pragma unroll
        for (int i = 0; i < kFakeLoads; ++i) {
            const uint32_t r = (uint32_t)min(rb + kFakeRowSlots * i, rows - 1);
            v[i] = ldg_nt<u32x4>(xt + (r * xrow + coff));
        }
#pragma unroll
        for (int i = 0; i < kFakeLoads; ++i)
            if (!(col_ok && rb + kFakeRowSlots * i < rows)) v[i] = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < kFakeLoads; ++i) {
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
    for (int i = 0; i < kFakeRowSlots / 4; ++i) {
        const u32x4 q = ((const u32x4*)lds)[i];
        m = max(m, max(max(q.x, q.y), max(q.z, q.w)));
    }

    const Fp8BlockParams p = fp8_block_params<MODE>(m);
    if (t == 0 && a.s) stg<float>(a.s + (tm * kt + tn), p.scale);

    if (p.fast) {
#pragma unroll
        for (int i = 0; i < kFakeLoads; ++i) {
            const u32x2 lo = expand4(fp8_quant4_fast<MODE>(v[i].x, v[i].y, p), p.scale);
            const u32x2 hi = expand4(fp8_quant4_fast<MODE>(v[i].z, v[i].w, p), p.scale);
            const u32x4 o = {lo.x, lo.y, hi.x, hi.y};
            if (full || (col_ok && rb + kFakeRowSlots * i < rows))
                stg_nt_sc1<u32x4>(yt + ((uint32_t)(rb + kFakeRowSlots * i) * yrow + (uint32_t)cc * 16u), o);
        }
    } else {
        // NaN / Inf block (rare): the literal element functions; rows are re-read so that the register copy of the
        // block is never indexed dynamically
#pragma nounroll
        for (int i = 0; i < kFakeLoads; ++i) {
            if (!(col_ok && rb + kFakeRowSlots * i < rows)) continue;
            const u32x4 w = ldg<u32x4>(xt + ((uint32_t)(rb + kFakeRowSlots * i) * xrow + (uint32_t)cc * 16u));
            const u32x2 lo = expand4(fp8_quant4_exact<MODE>(w.x, w.y, p), p.scale);
            const u32x2 hi = expand4(fp8_quant4_exact<MODE>(w.z, w.w, p), p.scale);
            const u32x4 o = {lo.x, lo.y, hi.x, hi.y};
            stg<u32x4>(yt + ((uint32_t)(rb + kFakeRowSlots * i) * yrow + (uint32_t)cc * 16u), o);
        }
    }
}

// any block shape, strides and alignment: one workgroup per block, two passes (the second one hits L2)
template <int MODE>
__device__ __forceinline__ void fake_tile_generic(const FakeArgs& a, int64_t tm, int64_t tn, int kt, uint32_t* lds)
{
    const int64_t r0 = tm * a.bm, c0 = tn * a.bn;
    const int rows = (int)min((int64_t)a.bm, a.M - r0), cols = (int)min((int64_t)a.bn, a.N - c0);
    const int n = rows * cols;
    uint32_t m = 0;
    for (int e = threadIdx.x; e < n; e += blockDim.x) {
        const int i = e / cols, j = e - i * cols;
        m = max(m, (uint32_t)a.x[(r0 + i) * a.sx_m + (c0 + j) * a.sx_n] & 0x7FFFu);
    }
    m = wave64_max_u32(m);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    m = 0;
    for (int w = 0; w < kFakeThreads / 64; ++w) m = max(m, lds[w]);
    const Fp8BlockParams p = fp8_block_params<MODE>(m);
    if (threadIdx.x == 0 && a.s) a.s[tm * kt + tn] = p.scale;
    for (int e = threadIdx.x; e < n; e += blockDim.x) {
        const int i = e / cols, j = e - i * cols;
        const float xv = u2f((uint32_t)a.x[(r0 + i) * a.sx_m + (c0 + j) * a.sx_n] << 16);
        const uint32_t code = fp8_quant1_exact<MODE>(xv, p);
        const f32x2 f = __builtin_amdgcn_cvt_pk_f32_fp8((int)code, false);
        a.y[(r0 + i) * a.sy_m + (c0 + j)] = (uint16_t)pack_bf16x2_rne(f.x * p.scale, 0.0f);
    }
}

template <int MODE, bool VEC>
__global__ __launch_bounds__(kFakeThreads) void fp8_block_fake_quant_kernel(const FakeArgs a, const int64_t total_tiles)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds[kFakeRowSlots];
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_tiles) return;  // uniform per workgroup
    const int64_t tile = xcd_chunked_item(slot, total_tiles, kFakeTilesPerXcdRun);
    const int kt = (int)((a.N + a.bn - 1) / a.bn);
    const int64_t tm = tile / kt, tn = tile - tm * kt;
    if (VEC) fake_tile_vec128<MODE>(a, tm, tn, kt, lds);
    else fake_tile_generic<MODE>(a, tm, tn, kt, lds);
}

template <int MODE>
static void launch_fake(const FakeArgs& a, int64_t tiles, hipStream_t st)
{
    const dim3 g = grid_for_items(tiles);
    // the decision reads host-visible arguments only
    const bool vec = a.bm == 128 && a.bn == 128 && a.sx_n == 1 && (a.sx_m & 7) == 0 && (a.N & 7) == 0 && (a.sy_m & 7) == 0 &&
                     ((uintptr_t)a.x & 15) == 0 && ((uintptr_t)a.y & 15) == 0 && a.sx_m >= 0 && a.sx_m < (1 << 22) &&
                     a.sy_m >= 0 && a.sy_m < (1 << 22);
    if (vec) fp8_block_fake_quant_kernel<MODE, true><<<g, kFakeThreads, kFakeOccupancyPadBytes, st>>>(a, tiles);
    else fp8_block_fake_quant_kernel<MODE, false><<<g, kFakeThreads, 0, st>>>(a, tiles);
}

}  // namespace wq

using namespace wq;

WQ_EXPORT int wq_fp8_block_quant_dequant(const void* x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, void* y,
                                         int64_t sy_m, float* s, int bm, int bn, int mode, void* stream)
{
    if (M < 0 || N < 0 || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (mode != WQ_FP8_MODE_TORCH && mode != WQ_FP8_MODE_TRITON && mode != WQ_FP8_MODE_TORCH_DEVICE &&
        mode != WQ_FP8_MODE_UE8M0)
        return WQ_ERR_MODE;
    if (M == 0 || N == 0) return WQ_OK;
    if (!x || !y) return WQ_ERR_NULL;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    FakeArgs a{(const uint16_t*)x, (uint16_t*)y, s, M, N, sx_m, sx_n, sy_m, bm, bn};
    const int64_t tiles = cdiv64(M, bm) * cdiv64(N, bn);
    hipStream_t st = (hipStream_t)stream;
    switch (mode) {
    case WQ_FP8_MODE_TORCH: launch_fake<WQ_FP8_MODE_TORCH>(a, tiles, st); break;
    case WQ_FP8_MODE_TORCH_DEVICE: launch_fake<WQ_FP8_MODE_TORCH_DEVICE>(a, tiles, st); break;
    case WQ_FP8_MODE_UE8M0: launch_fake<WQ_FP8_MODE_UE8M0>(a, tiles, st); break;
    default: launch_fake<WQ_FP8_MODE_TRITON>(a, tiles, st); break;
    }
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}
