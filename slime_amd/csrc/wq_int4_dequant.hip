// INT4 pack-quantized -> bf16, and the quantise-dequantise forward of the INT4 QAT straight-through
// estimator, for gfx950.
//
// int4_dequant_kernel: every lane turns one packed int32 (8 nibbles) into 8 bf16 and writes them with ONE
// 16-byte store, so a wavefront reads 256 contiguous bytes and writes 1 KiB contiguous per step; the two steps
// of a lane are both in flight before first use.  f32(nibble - 8) * f32(scale) has at most 12 significant bits,
// so the fp32 product is exact and the only rounding is the final one to bf16, as in the reference's
// (int8.to(f32) * scale.to(f32)).to(bf16).
//
// int4_fake_ste_kernel: a 128-element group is owned by 16 adjacent lanes (32 / 64: 4 / 8 lanes), one 16-byte
// load and one 16-byte store per lane; x / s is an IEEE division, amax / 7 a division or a multiplication by RN(1/7)
// (torch evaluates `tensor / 7` the first way on CPU tensors and the second way on GPU tensors).

#include "wq_common.h"

namespace wq {

typedef float f32x2d __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2d __attribute__((ext_vector_type(2)));

// Work item size and residency by measurement (Qwen3-30B-A3B experts, 8 layers, % of the HBM peak; a compute-free 1:4 stream of
// the same shapes peaks at 82 % with two or four steps): 8 words per lane at 3 workgroups per CU 77.4-77.8; 4 words at 2 / 3 / 4 / 6
// per CU 54.4 / 70.5 / 77.2 / 76.9; 3 words 73-76; 2 words at 6 per CU 72.8, at full occupancy 79.0-80.1 (used; runs of 16 / 64 / 128
// items per XCD instead of 32: 77.4 / 79.5 / 79.4); 1 word 64-65.
constexpr int kDqSteps = 2;                       // packed words per lane
constexpr int kDqWordsPerWg = 256 * kDqSteps;     // 2 KiB of packed input, 16 KiB of bf16 output
static_assert(kDqWordsPerWg == WQ_INT4_DEQ_WORDS_PER_ITEM, "work item size is part of the C ABI");
constexpr int kDqItemsPerXcdRun = 32;
constexpr int kDqOccupancyPadBytes = 0;           // unused dynamic LDS that would cap workgroups per CU: no cap

__device__ __forceinline__ uint32_t pack2_bf16(float a, float b)
{
    f32x2d v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2d));
}

// ITEMS: one pre-resolved descriptor per work item (a bucket of tensors in one launch) instead of one tensor in the
// kernel arguments; the descriptor points at the item's first word, its first scale and its first output element.
template <bool ITEMS>
__global__ __launch_bounds__(256) void int4_dequant_kernel(const uint32_t* __restrict__ packed,
                                                          const uint16_t* __restrict__ scale,
                                                          uint16_t* __restrict__ y, int64_t n_words, int group,
                                                          const wq_int4_dequant_item* __restrict__ items,
                                                          int64_t total_items)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_items) return;
    const int64_t item = xcd_chunked_item(slot, total_items, kDqItemsPerXcdRun);
    int64_t w0 = item * kDqWordsPerWg + threadIdx.x;
    if (ITEMS) {
        const wq_int4_dequant_item it = items[item];
        packed = (const uint32_t*)it.packed;
        scale = (const uint16_t*)it.scale;
        y = (uint16_t*)it.y;
        n_words = it.n_words;
        w0 = threadIdx.x;
    }
    const int gshift = (group & (group - 1)) == 0 ? __builtin_ctz((unsigned)group) : -1;
    uint32_t w[kDqSteps];
    uint32_t sb[kDqSteps];
#pragma unroll
    for (int i = 0; i < kDqSteps; ++i) {
        // lanes past the end re-read the last word instead of branching around the load
        const int64_t k = min(w0 + i * 256, n_words - 1);
        w[i] = ldg_nt<uint32_t>(packed + k);
        const int64_t g = gshift >= 0 ? (k * 8) >> gshift : (k * 8) / group;   // rows are whole groups: flat group index
        sb[i] = ldg<uint16_t>(scale + g);
    }
#pragma unroll
    for (int i = 0; i < kDqSteps; ++i) {
        const int64_t k = w0 + i * 256;
        if (k >= n_words) continue;
        const float s = u2f(sb[i] << 16);
        float f[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = (float)((int)((w[i] >> (4 * j)) & 0xFu) - 8) * s;
        const u32x4 o = {pack2_bf16(f[0], f[1]), pack2_bf16(f[2], f[3]), pack2_bf16(f[4], f[5]), pack2_bf16(f[6], f[7])};
        stg_nt<u32x4>(y + k * 8, o);
    }
}

// Plain form for everything the kernel above does not take: scales in fp16 or fp32 (the reference converts whatever
// dtype it finds with .to(float32)), groups of any size >= 1 that divide the row (group 1 = one scale per element, the
// reference's group_size <= 0 case), rows that are not a multiple of 8 long (the last word of a row is cut).  One
// lane per packed word; with an fp32 scale the product is rounded in fp32 and again to bf16, as in the reference.
template <typename S> __device__ __forceinline__ float scale_as_f32(const void* p, int64_t i);
template <> __device__ __forceinline__ float scale_as_f32<uint16_t>(const void* p, int64_t i) { return u2f((uint32_t)((const uint16_t*)p)[i] << 16); }
template <> __device__ __forceinline__ float scale_as_f32<_Float16>(const void* p, int64_t i) { return (float)((const _Float16*)p)[i]; }
template <> __device__ __forceinline__ float scale_as_f32<float>(const void* p, int64_t i) { return ((const float*)p)[i]; }

template <typename S>
__global__ __launch_bounds__(256) void int4_dequant_any_kernel(const uint32_t* __restrict__ packed, const void* __restrict__ scale,
                                                              uint16_t* __restrict__ y, int64_t M, int64_t N, int64_t group)
{
    const int64_t words_per_row = (N + 7) / 8;
    const int64_t k = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * 256 + threadIdx.x;
    if (k >= M * words_per_row) return;
    const int64_t row = k / words_per_row, c0 = (k - row * words_per_row) * 8;
    const uint32_t w = packed[k];
    const int64_t groups_per_row = N / group;
    for (int j = 0; j < 8 && c0 + j < N; ++j) {
        const float s = scale_as_f32<S>(scale, row * groups_per_row + (c0 + j) / group);
        const float f = (float)((int)((w >> (4 * j)) & 0xFu) - 8) * s;
        y[row * N + c0 + j] = (uint16_t)f32_to_bf16_bits(f);
    }
}

// ---- QAT straight-through forward ------------------------------------------------------------------

constexpr int kSteGroupsPerWg = 64;
constexpr int kSteItemsPerXcdRun = 32;
constexpr int kSteOccupancyPadBytes = 36 * 1024;
constexpr int kSteWindow = 4;                     // 16-byte loads in flight per lane (4 = all of a work item with 128-element groups)

// ITEMS: one pre-resolved descriptor per work item (many tensors in one launch), pointing at the item's first group.
template <int L, bool ITEMS>
__global__ __launch_bounds__(256) void int4_fake_ste_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                           int64_t n_groups, int64_t total_items, int div7,
                                                           const wq_int4_ste_item* __restrict__ items, char* y_base)
{
    constexpr int CL = 256 / L;
    constexpr int STEPS = kSteGroupsPerWg / CL;
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_items) return;
    const int64_t item = xcd_chunked_item(slot, total_items, kSteItemsPerXcdRun);
    const int cl = threadIdx.x / L, ll = threadIdx.x % L;
    int64_t g0 = item * kSteGroupsPerWg + cl;
    if (ITEMS) {
        const wq_int4_ste_item it = items[item];
        x = (const uint16_t*)it.x;
        y = (uint16_t*)(y_base + (uintptr_t)it.y);       // y_base is null when the items hold addresses
        n_groups = it.n_groups;
        g0 = cl;
    }
    u32x4 v[STEPS];
    auto issue = [&](int i) {
        const int64_t g = min(g0 + i * CL, n_groups - 1);
        v[i] = ldg_nt<u32x4>(x + g * (8 * L) + ll * 8);
    };
#pragma unroll
    for (int i = 0; i < kSteWindow && i < STEPS; ++i) issue(i);
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        if (kSteWindow < STEPS) {
            asm volatile("" :: "v"(v[i].x));
            if (i + kSteWindow < STEPS) issue(i + kSteWindow);
            __builtin_amdgcn_sched_barrier(0);
        }
        const int64_t g = g0 + i * CL;
        const uint32_t wd[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
        float xs[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { xs[2 * j] = bf16lo(wd[j]); xs[2 * j + 1] = bf16hi(wd[j]); }
        // amax in bf16 (exact), converted to fp32: x_view.abs().float().amax(); torch.amax propagates NaN, and so
        // does the integer max on magnitude bits
        uint32_t mb = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) mb = pk_absmax(mb, wd[j]);
        mb = pk_fold(mb);
        mb = max(mb, dpp_u32<0xB1>(mb));
        mb = max(mb, dpp_u32<0x4E>(mb));
        if (L >= 8) mb = max(mb, dpp_u32<0x141>(mb));
        if (L >= 16) mb = max(mb, dpp_u32<0x140>(mb));
        float s = div7 == WQ_DIV7_DEVICE ? u2f(mb << 16) * (1.0f / 7.0f) : u2f(mb << 16) / 7.0f;
        s = (s != s) ? s : fmaxf(s, 1e-5f);           // clamp(min=1e-5) keeps NaN
        float o[8];
        // Finite amax.  Under the reciprocal-multiply rule s is the scale of the pack kernel, for which
        // q0 = x*r, q = fma(fma(-q0, s, x), r, q0) rounds to the same integer as the IEEE quotient for every bf16 x
        // of the group (the exhaustive check of the pack function covers exactly these pairs).  |q| <= 7 there, so
        // the clamp is a no-op; adding and subtracting 1.5 * 2^23 rounds half to even.  The result carries the
        // sign of x, zero included (round and clamp keep it, s is positive); it is restored on the bf16 pairs.
        const bool fast = mb < kBf16Inf;
        if (fast) {
            // under the division rule s is an arbitrary fp32 number: the correctly rounded reciprocal (one division
            // per lane) keeps the two-FMA quotient exact for any divisor
            const float r = div7 == WQ_DIV7_DEVICE ? rcp_refined(s) : 1.0f / s;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = ((div_by_scale(xs[j], s, r) + 12582912.0f) - 12582912.0f) * s;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float q = __builtin_rintf(xs[j] / s);
                if (q == q) q = fminf(fmaxf(q, -7.0f), 7.0f);
                o[j] = q * s;
            }
        }
        if (g < n_groups) {
            u32x4 r = {pack2_bf16(o[0], o[1]), pack2_bf16(o[2], o[3]), pack2_bf16(o[4], o[5]), pack2_bf16(o[6], o[7])};
            if (fast) r = (r & 0x7FFF7FFFu) | (v[i] & 0x80008000u);
            stg_nt_sc1<u32x4>(y + g * (8 * L) + ll * 8, r);
        }
    }
}

}  // namespace wq

using namespace wq;

WQ_EXPORT int wq_int4_dequant(const int32_t* packed, const void* scale, void* y, int64_t M, int64_t N, int group,
                              void* stream)
{
    if (M < 0 || N < 0 || group <= 0 || group % 8 != 0 || N % group != 0) return WQ_ERR_SHAPE;
    if (M == 0 || N == 0) return WQ_OK;
    if (!packed || !scale || !y) return WQ_ERR_NULL;
    if (((uintptr_t)y & 15) || ((uintptr_t)packed & 3) || ((uintptr_t)scale & 1)) return WQ_ERR_ALIGN;
    const int64_t n_words = M * (N / 8);
    const int64_t items = cdiv64(n_words, kDqWordsPerWg);
    int4_dequant_kernel<false><<<grid_for_items(items), 256, kDqOccupancyPadBytes, (hipStream_t)stream>>>(
        (const uint32_t*)packed, (const uint16_t*)scale, (uint16_t*)y, n_words, group, nullptr, items);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_dequant_any(const int32_t* packed, const void* scale, int scale_dtype, void* y, int64_t M, int64_t N,
                                  int group, void* stream)
{
    if (M < 0 || N < 0 || group <= 0 || N % group != 0) return WQ_ERR_SHAPE;
    if (scale_dtype != WQ_DTYPE_BF16 && scale_dtype != WQ_DTYPE_F16 && scale_dtype != WQ_DTYPE_F32) return WQ_ERR_MODE;
    if (M == 0 || N == 0) return WQ_OK;
    if (!packed || !scale || !y) return WQ_ERR_NULL;
    const int salign = scale_dtype == WQ_DTYPE_F32 ? 3 : 1;
    if (((uintptr_t)y & 1) || ((uintptr_t)packed & 3) || ((uintptr_t)scale & salign)) return WQ_ERR_ALIGN;
    const int64_t words = M * cdiv64(N, 8);
    const dim3 g = grid_for_items(cdiv64(words, 256));
    hipStream_t st = (hipStream_t)stream;
    if (scale_dtype == WQ_DTYPE_F32)
        int4_dequant_any_kernel<float><<<g, 256, 0, st>>>((const uint32_t*)packed, scale, (uint16_t*)y, M, N, group);
    else if (scale_dtype == WQ_DTYPE_F16)
        int4_dequant_any_kernel<_Float16><<<g, 256, 0, st>>>((const uint32_t*)packed, scale, (uint16_t*)y, M, N, group);
    else
        int4_dequant_any_kernel<uint16_t><<<g, 256, 0, st>>>((const uint32_t*)packed, scale, (uint16_t*)y, M, N, group);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_dequant_items(const wq_int4_dequant_item* items, int64_t n_items, int group, void* stream)
{
    if (n_items < 0 || group < 8 || (group & (group - 1)) != 0 || group > WQ_INT4_DEQ_WORDS_PER_ITEM * 8) return WQ_ERR_SHAPE;
    if (n_items == 0) return WQ_OK;
    if (!items) return WQ_ERR_NULL;
    int4_dequant_kernel<true><<<grid_for_items(n_items), 256, kDqOccupancyPadBytes, (hipStream_t)stream>>>(
        nullptr, nullptr, nullptr, 0, group, items, n_items);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_fake_quant_ste(const void* x, void* y, int64_t M, int64_t N, int group, int div7, void* stream)
{
    if (M < 0 || N < 0 || group <= 0 || N % group != 0) return WQ_ERR_SHAPE;
    if (div7 != WQ_DIV7_IEEE && div7 != WQ_DIV7_DEVICE) return WQ_ERR_MODE;
    if (group != 32 && group != 64 && group != 128) return WQ_ERR_UNSUPPORTED;
    if (M == 0 || N == 0) return WQ_OK;
    if (!x || !y) return WQ_ERR_NULL;
    if (((uintptr_t)x & 15) || ((uintptr_t)y & 15)) return WQ_ERR_ALIGN;
    const int64_t n_groups = M * (N / group);
    const int64_t items = cdiv64(n_groups, kSteGroupsPerWg);
    hipStream_t st = (hipStream_t)stream;
    const dim3 g = grid_for_items(items);
    if (group == 32) int4_fake_ste_kernel<4, false><<<g, 256, kSteOccupancyPadBytes, st>>>((const uint16_t*)x, (uint16_t*)y, n_groups, items, div7, nullptr, nullptr);
    else if (group == 64) int4_fake_ste_kernel<8, false><<<g, 256, kSteOccupancyPadBytes, st>>>((const uint16_t*)x, (uint16_t*)y, n_groups, items, div7, nullptr, nullptr);
    else int4_fake_ste_kernel<16, false><<<g, 256, kSteOccupancyPadBytes, st>>>((const uint16_t*)x, (uint16_t*)y, n_groups, items, div7, nullptr, nullptr);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_fake_quant_ste_items(const wq_int4_ste_item* items, int64_t n_items, void* y_base, int group, int div7,
                                           void* stream)
{
    if (n_items < 0) return WQ_ERR_SHAPE;
    if (div7 != WQ_DIV7_IEEE && div7 != WQ_DIV7_DEVICE) return WQ_ERR_MODE;
    if (group != 32 && group != 64 && group != 128) return WQ_ERR_UNSUPPORTED;
    if (n_items == 0) return WQ_OK;
    if (!items) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    const dim3 g = grid_for_items(n_items);
    if (group == 32) int4_fake_ste_kernel<4, true><<<g, 256, kSteOccupancyPadBytes, st>>>(nullptr, nullptr, 0, n_items, div7, items, (char*)y_base);
    else if (group == 64) int4_fake_ste_kernel<8, true><<<g, 256, kSteOccupancyPadBytes, st>>>(nullptr, nullptr, 0, n_items, div7, items, (char*)y_base);
    else int4_fake_ste_kernel<16, true><<<g, 256, kSteOccupancyPadBytes, st>>>(nullptr, nullptr, 0, n_items, div7, items, (char*)y_base);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}
