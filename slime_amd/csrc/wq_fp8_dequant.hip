// block-FP8 (e4m3fn) -> bf16 dequantisation for gfx950.
//
// A work item is a strip of WQ_DEQ_ROWS rows x WQ_DEQ_COLS columns handled by one 256-thread
// workgroup: each wavefront reads one 1 KiB row segment per step (16 bytes = 16 codes per lane)
// and writes the 2 KiB of bf16 it becomes as two 16-byte stores per lane.  Codes are expanded with
// v_cvt_pk_f32_fp8, multiplied by the block's fp32 scale (one rounding, to bf16, RNE) - the same
// single rounding as the reference's y = (x.to(f32) * s) stored to bf16.

#include "wq_common.h"

namespace wq {

typedef float f32x2 __attribute__((ext_vector_type(2)));

struct DeqArgs {
    wq_fp8_dequant_desc d;
    const wq_fp8_dequant_desc* descs;
    const int64_t* work_start;
    int32_t n_desc;
    int32_t block;
};

__device__ __forceinline__ int find_desc_deq(const int64_t* __restrict__ start, int n, int64_t t)
{
    int lo = 0, hi = n;
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (start[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// RNE fp32 -> bf16 for two values packed in a dword (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b)
{
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

template <int MODE>
__device__ __forceinline__ float load_scale(const float* __restrict__ s, int64_t idx)
{
    float v = s[idx];
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

// OUT: WQ_DTYPE_BF16 (the reference tool's default dtype) or WQ_DTYPE_F32 (the un-rounded product).
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 dequant4_f32(uint32_t codes, float sc)
{
    f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, false);
    f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, true);
    return (f32x4){lo.x * sc, lo.y * sc, hi.x * sc, hi.y * sc};
}

template <int MODE, bool GROUPED, int OUT>
__global__ __launch_bounds__(256) void fp8_block_dequant_kernel(const DeqArgs a, const int64_t total_work)
{
    const int64_t item = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (item >= total_work) return;
    wq_fp8_dequant_desc d;
    int64_t local = item;
    if (GROUPED) {
        const int di = find_desc_deq(a.work_start, a.n_desc, item);
        d = a.descs[di];
        local = item - a.work_start[di];
    } else {
        d = a.d;
    }
    const int block = a.block;
    const int64_t strips = (d.N + WQ_DEQ_COLS - 1) / WQ_DEQ_COLS;
    const int64_t sm = local / strips, sn = local - sm * strips;
    const int64_t kt = (d.N + block - 1) / block;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t col = sn * WQ_DEQ_COLS + lane * 16;
    const uint8_t* x = (const uint8_t*)d.x;
    uint16_t* y = (uint16_t*)d.y;
    float* yf = (float*)d.y;
    const bool vec = (d.N & 15) == 0 && ((uintptr_t)d.x & 15) == 0 && ((uintptr_t)d.y & 15) == 0 && (block & 15) == 0;

    if (vec) {
        if (col >= d.N) return;
        const int64_t sidx_col = col / block;
        u32x4 v[4];
        int64_t rows[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            rows[i] = sm * WQ_DEQ_ROWS + wave + 4 * i;
            v[i] = (u32x4){0u, 0u, 0u, 0u};
            if (rows[i] < d.M) v[i] = __builtin_nontemporal_load((const u32x4*)(x + rows[i] * d.N + col));
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (rows[i] >= d.M) continue;
            const float sc = load_scale<MODE>(d.s, (rows[i] / block) * kt + sidx_col);
            if (OUT == WQ_DTYPE_BF16) {
                const u32x2 a0 = dequant4(v[i].x, sc), a1 = dequant4(v[i].y, sc);
                const u32x2 a2 = dequant4(v[i].z, sc), a3 = dequant4(v[i].w, sc);
                const u32x4 o0 = {a0.x, a0.y, a1.x, a1.y}, o1 = {a2.x, a2.y, a3.x, a3.y};
                u32x4* yp = (u32x4*)(y + rows[i] * d.N + col);
                __builtin_nontemporal_store(o0, yp);
                __builtin_nontemporal_store(o1, yp + 1);
            } else {
                f32x4* yp = (f32x4*)(yf + rows[i] * d.N + col);
                __builtin_nontemporal_store(dequant4_f32(v[i].x, sc), yp);
                __builtin_nontemporal_store(dequant4_f32(v[i].y, sc), yp + 1);
                __builtin_nontemporal_store(dequant4_f32(v[i].z, sc), yp + 2);
                __builtin_nontemporal_store(dequant4_f32(v[i].w, sc), yp + 3);
            }
        }
    } else {
        // element-wise tail path: any N / alignment / block size
        for (int r = wave; r < WQ_DEQ_ROWS; r += 4) {
            const int64_t row = sm * WQ_DEQ_ROWS + r;
            if (row >= d.M) break;
            for (int k = 0; k < 16; ++k) {
                const int64_t c = sn * WQ_DEQ_COLS + k * 64 + lane;
                if (c >= d.N) break;
                const float sc = load_scale<MODE>(d.s, (row / block) * kt + c / block);
                uint32_t code = x[row * d.N + c];
                f32x2 f = __builtin_amdgcn_cvt_pk_f32_fp8((int)code, false);
                if (OUT == WQ_DTYPE_BF16) y[row * d.N + c] = (uint16_t)(pack_bf16x2(f.x * sc, 0.0f) & 0xFFFFu);
                else yf[row * d.N + c] = f.x * sc;
            }
        }
    }
}

}  // namespace wq

using namespace wq;

template <bool GROUPED>
static int launch_deq(const DeqArgs& a, int64_t work, int mode, int out_dtype, hipStream_t st)
{
    const dim3 g = grid_for_items(work);
    if (mode == WQ_DEQ_MODE_F32SCALE) {
        if (out_dtype == WQ_DTYPE_BF16) fp8_block_dequant_kernel<WQ_DEQ_MODE_F32SCALE, GROUPED, WQ_DTYPE_BF16><<<g, 256, 0, st>>>(a, work);
        else fp8_block_dequant_kernel<WQ_DEQ_MODE_F32SCALE, GROUPED, WQ_DTYPE_F32><<<g, 256, 0, st>>>(a, work);
    } else {
        if (out_dtype == WQ_DTYPE_BF16) fp8_block_dequant_kernel<WQ_DEQ_MODE_BF16SCALE, GROUPED, WQ_DTYPE_BF16><<<g, 256, 0, st>>>(a, work);
        else fp8_block_dequant_kernel<WQ_DEQ_MODE_BF16SCALE, GROUPED, WQ_DTYPE_F32><<<g, 256, 0, st>>>(a, work);
    }
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

static int check_deq(int64_t block, int mode, int out_dtype)
{
    if (block <= 0) return WQ_ERR_SHAPE;
    if (mode != WQ_DEQ_MODE_F32SCALE && mode != WQ_DEQ_MODE_BF16SCALE) return WQ_ERR_MODE;
    if (out_dtype != WQ_DTYPE_BF16 && out_dtype != WQ_DTYPE_F32) return WQ_ERR_MODE;
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
    DeqArgs a{};
    a.d = wq_fp8_dequant_desc{x, s, y, M, N};
    a.block = block;
    return launch_deq<false>(a, cdiv64(M, WQ_DEQ_ROWS) * cdiv64(N, WQ_DEQ_COLS), mode, out_dtype, (hipStream_t)stream);
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
    return launch_deq<true>(a, total_work, mode, out_dtype, (hipStream_t)stream);
}
