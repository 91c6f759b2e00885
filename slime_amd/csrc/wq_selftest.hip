// libslime_amd_wq_test.so: on-device self-checks of the element functions and of the hardware number-format
// conversions the production kernels rely on, plus the compute-free kernels (copy, 2:1 / 4:1 streams, an empty launch)
// that hardware counters and achieved bandwidths are scaled against.  Instruments of the tests and the benchmark; the
// product library holds none of this.
//
// The production element functions replace the reference's per-element IEEE division by a
// reciprocal-and-refine sequence and its software casts by gfx950 conversion instructions.  These
// kernels compare them, over the complete input domain, with the literal arithmetic (IEEE "/",
// software round-to-nearest-even), so that the shortcut is licensed by exhaustion, not by argument.

#include "wq_common.h"
#include "../../include/slime_amd_wq_test.h"

namespace wq {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__global__ void selftest_init_kernel(uint64_t* out)
{
    out[0] = 0;
    out[1] = ~0ull;
}

__device__ __forceinline__ void report(uint64_t* out, uint64_t key)
{
    atomicAdd((unsigned long long*)&out[0], 1ull);
    atomicMin((unsigned long long*)&out[1], (unsigned long long)key);
}

// grid.x = 16384 threads' worth of x quadruples per amax, grid.y = amax index
template <int MODE>
__global__ __launch_bounds__(256) void selftest_fp8_elem_kernel(uint32_t amax_lo, uint32_t amax_hi, uint64_t* out)
{
    const uint32_t a = amax_lo + blockIdx.y;
    if (a >= amax_hi || a >= kBf16Inf) return;
    const uint32_t x0 = (blockIdx.x * 256u + threadIdx.x) * 4u;
    if (x0 >= 65536u) return;
    const Fp8BlockParams p = fp8_block_params<MODE>(a);
    const uint32_t w0 = x0 | ((x0 + 1u) << 16), w1 = (x0 + 2u) | ((x0 + 3u) << 16);
    const uint32_t fast = fp8_quant4_fast<MODE>(w0, w1, p);
    const uint32_t exact = fp8_quant4_exact<MODE>(w0, w1, p);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t xb = x0 + k;
        if ((xb & 0x7FFFu) > a) continue;  // not reachable: |x| <= block amax
        if (((fast >> (8 * k)) & 0xFFu) != ((exact >> (8 * k)) & 0xFFu)) report(out, ((uint64_t)a << 16) | xb);
    }
}

__global__ __launch_bounds__(256) void selftest_int4_elem_kernel(uint32_t amax_lo, uint32_t amax_hi, uint64_t* out)
{
    const uint32_t a = amax_lo + blockIdx.y;
    if (a >= amax_hi || a >= kBf16Inf) return;
    // each thread packs eight consecutive bf16 patterns with the production function; patterns beyond
    // the group's amax (unreachable) are replaced by zero on both sides
    const uint32_t x0 = (blockIdx.x * 256u + threadIdx.x) * 8u;
    if (x0 >= 65536u) return;
    const float scale = int4_scale_sym(u2f(a << 16));
    const float rcp = rcp_refined(scale);
    if (f2u(rcp) != f2u(1.0f / scale)) report(out, ((uint64_t)a << 16) | 0xFFFFu);
    float x[8];
    uint32_t want = 0;
    bool range_ok = true;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t xb = x0 + j;
        x[j] = ((xb & 0x7FFFu) > a) ? 0.0f : u2f(xb << 16);
        const int qi = (int)__builtin_rintf(x[j] / scale);
        range_ok = range_ok && qi >= -7 && qi <= 7;
        want |= ((uint32_t)(qi + 8) & 0xFu) << (4 * j);
    }
    // both packers: the byte-gathering one the pack kernel uses and the shift-add one
    const uint32_t got = pack8_sym_bytes(x, scale, rcp);
    if (got != want || pack8_sym(x, scale, rcp) != want || !range_ok) report(out, ((uint64_t)a << 16) | x0);
}

// hardware fp32 -> e4m3fn vs software, both word positions of the packed conversion
__global__ __launch_bounds__(256) void selftest_cvt_fp8_kernel(uint64_t lo, uint64_t hi, uint64_t* out)
{
    for (uint64_t b = lo + (uint64_t)blockIdx.x * 256u + threadIdx.x; b < hi; b += (uint64_t)gridDim.x * 256u) {
        const uint32_t u = (uint32_t)b;
        const uint32_t mag = u & 0x7FFFFFFFu;
        const bool is_nan = mag > 0x7F800000u;
        if (!is_nan && mag > 0x43E80000u) continue;  // |v| > 464: overflow behaviour is never relied on
        const float f = u2f(u);
        const uint32_t sw = f32_to_e4m3fn_sw(f);
        const uint32_t h0 = cvt_pk_fp8_lo(f, 0.0f, 0u);
        const uint32_t h1 = cvt_pk_fp8_hi(0.0f, f, 0u);
        uint32_t g0 = h0 & 0xFFu, g1 = (h1 >> 24) & 0xFFu;
        bool bad;
        if (is_nan) bad = ((g0 & 0x7Fu) != 0x7Fu) || ((g1 & 0x7Fu) != 0x7Fu);
        else bad = (g0 != sw) || (g1 != sw);
        if (bad) report(out, b);
    }
}

// hardware fp32 -> bf16 (v_cvt_pk_bf16_f32) vs software RNE, non-NaN inputs
__global__ __launch_bounds__(256) void selftest_cvt_bf16_kernel(uint64_t lo, uint64_t hi, uint64_t* out)
{
    for (uint64_t b = lo + (uint64_t)blockIdx.x * 256u + threadIdx.x; b < hi; b += (uint64_t)gridDim.x * 256u) {
        const uint32_t u = (uint32_t)b;
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) continue;
        f32x2 v = {u2f(u), u2f(u ^ 0x80000000u)};
        const uint32_t hw = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
        const uint32_t sw = f32_to_bf16_bits(v.x) | (f32_to_bf16_bits(v.y) << 16);
        if (hw != sw) report(out, b);
    }
}

// hardware e4m3fn -> fp32 (v_cvt_pk_f32_fp8) vs the definition, all 256 codes in all 4 byte lanes
__global__ void selftest_decode_fp8_kernel(uint64_t* out)
{
    const uint32_t c = threadIdx.x;  // 256 threads
    const uint32_t e = (c >> 3) & 0xFu, m = c & 7u;
    uint32_t want;
    if (e == 0xFu && m == 7u) want = 0x7FC00000u;
    else if (e == 0) want = f2u((float)m * 0.001953125f);
    else want = ((e - 7u + 127u) << 23) | (m << 20);
    want |= (c & 0x80u) << 24;
    const uint32_t packed = c | ((c ^ 0xFFu) << 8) | (c << 16) | ((c ^ 0xFFu) << 24);
    f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)packed, false);
    f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)packed, true);
    const bool nan = (e == 0xFu && m == 7u);
    bool bad = nan ? !(lo.x != lo.x && hi.x != hi.x) : (f2u(lo.x) != want || f2u(hi.x) != want);
    if (bad) report(out, c);
}

// A plain copy, launched the way that streams fastest on this part (measured with a compute-free sweep over work order,
// residency and loads per lane): runs of 64 consecutive 16 KiB items per XCD, two workgroups per CU, four 16-byte loads
// per lane in flight.  In dispatch order at full occupancy the same copy is 10 points slower.
constexpr int kCopyItemsPerXcdRun = 64;
constexpr unsigned kCopyOccupancyPadBytes = 77 * 1024;

__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16,
                                                   int64_t items)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= items) return;
    const int64_t base = xcd_chunked_item(slot, items, kCopyItemsPerXcdRun) * 1024 + threadIdx.x;
    u32x4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_nontemporal_load(src + min(base + i * 256, n16 - 1));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t k = base + i * 256;
        if (k < n16) __builtin_nontemporal_store(v[i], dst + k);
    }
}

// A compute-free stream with R bytes read per byte written (R = 2: the block-FP8 quantiser's mix, R = 4: the INT4 packer's):
// an item is STEPS x 4 KiB of output, the xor of R consecutive pieces of the input of that size.  It shows what the memory
// system gives this read:write mix on the box at hand, the way the plain copy does for 1:1.
constexpr int kFoldItemsPerXcdRun = 64;
// Launch shape by measurement (% of the 8 TB/s HBM peak, 4 GiB read): both mixes stream best with eight 16-byte loads per lane
// and two workgroups per CU - 2:1 83.3 (4 / 3 workgroups per CU: 78-80), 4:1 83.7 (four loads per lane 80.8, sixteen 78; at full
// occupancy 74-77).
constexpr unsigned kFoldPadBytes2 = 77 * 1024, kFoldPadBytes4 = 77 * 1024;      // two workgroups per CU
constexpr int kFoldSteps2 = 4, kFoldSteps4 = 2;                                 // output pieces per lane

template <int R, int STEPS>
__global__ __launch_bounds__(256) void fold_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t items)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= items) return;
    const int64_t item = xcd_chunked_item(slot, items, kFoldItemsPerXcdRun);
    const u32x4* in = src + item * (R * STEPS * 256) + threadIdx.x;
    u32x4 v[R][STEPS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < STEPS; ++i) v[r][i] = __builtin_nontemporal_load(in + (r * STEPS + i) * 256);
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        u32x4 acc = v[0][i];
#pragma unroll
        for (int r = 1; r < R; ++r) acc ^= v[r][i];
        __builtin_nontemporal_store(acc, dst + item * (STEPS * 256) + i * 256 + threadIdx.x);
    }
}

// The mirror image for the dequantisers: a compute-free stream with W bytes written per byte read (W = 2: FP8 -> bf16,
// W = 4: INT4 -> bf16).  An item is STEPS x 4 KiB of input; output piece w of input piece i is the input with w added to
// every dword, so every output byte depends on the data.
template <int W, int STEPS>
__global__ __launch_bounds__(256) void expand_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t items)
{
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= items) return;
    const int64_t item = xcd_chunked_item(slot, items, kFoldItemsPerXcdRun);
    const u32x4* in = src + item * (STEPS * 256) + threadIdx.x;
    u32x4 v[STEPS];
#pragma unroll
    for (int i = 0; i < STEPS; ++i) v[i] = __builtin_nontemporal_load(in + i * 256);
    u32x4* out = dst + item * (W * STEPS * 256) + threadIdx.x;
#pragma unroll
    for (int i = 0; i < STEPS; ++i)
#pragma unroll
        for (int w = 0; w < W; ++w) __builtin_nontemporal_store(v[i] + (uint32_t)w, out + (i * W + w) * 256);
}

__global__ void empty_kernel() {}

}  // namespace wq

using namespace wq;

WQ_EXPORT int wq_test_abi_version(void) { return WQ_ABI_VERSION; }

WQ_EXPORT int wq_selftest_fp8_elem(uint32_t amax_lo, uint32_t amax_hi, int mode, uint64_t* out, void* stream)
{
    if (!out) return WQ_ERR_NULL;
    if (amax_hi < amax_lo || amax_hi > 0x8000u) return WQ_ERR_SHAPE;
    if (mode != WQ_FP8_MODE_TORCH && mode != WQ_FP8_MODE_TRITON && mode != WQ_FP8_MODE_TORCH_DEVICE) return WQ_ERR_MODE;
    hipStream_t st = (hipStream_t)stream;
    selftest_init_kernel<<<1, 1, 0, st>>>(out);
    WQ_LAUNCH_CHECK();
    if (amax_hi == amax_lo) return WQ_OK;
    dim3 grid(64, amax_hi - amax_lo, 1);
    if (mode == WQ_FP8_MODE_TORCH) selftest_fp8_elem_kernel<WQ_FP8_MODE_TORCH><<<grid, 256, 0, st>>>(amax_lo, amax_hi, out);
    else if (mode == WQ_FP8_MODE_TORCH_DEVICE) selftest_fp8_elem_kernel<WQ_FP8_MODE_TORCH_DEVICE><<<grid, 256, 0, st>>>(amax_lo, amax_hi, out);
    else selftest_fp8_elem_kernel<WQ_FP8_MODE_TRITON><<<grid, 256, 0, st>>>(amax_lo, amax_hi, out);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_selftest_int4_elem(uint32_t amax_lo, uint32_t amax_hi, uint64_t* out, void* stream)
{
    if (!out) return WQ_ERR_NULL;
    if (amax_hi < amax_lo || amax_hi > 0x8000u) return WQ_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    selftest_init_kernel<<<1, 1, 0, st>>>(out);
    WQ_LAUNCH_CHECK();
    if (amax_hi == amax_lo) return WQ_OK;
    dim3 grid(32, amax_hi - amax_lo, 1);  // 32 x 256 threads x 8 patterns = 65536 per amax
    selftest_int4_elem_kernel<<<grid, 256, 0, st>>>(amax_lo, amax_hi, out);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

static int launch_range(void (*k)(uint64_t, uint64_t, uint64_t*), uint64_t lo, uint64_t hi, uint64_t* out, void* stream)
{
    if (!out) return WQ_ERR_NULL;
    if (hi < lo || hi > (1ull << 32)) return WQ_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    selftest_init_kernel<<<1, 1, 0, st>>>(out);
    WQ_LAUNCH_CHECK();
    if (hi == lo) return WQ_OK;
    uint64_t blocks = (hi - lo + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    k<<<(unsigned)blocks, 256, 0, st>>>(lo, hi, out);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_selftest_cvt_fp8(uint64_t lo, uint64_t hi, uint64_t* out, void* stream)
{
    return launch_range(selftest_cvt_fp8_kernel, lo, hi, out, stream);
}

WQ_EXPORT int wq_selftest_cvt_bf16(uint64_t lo, uint64_t hi, uint64_t* out, void* stream)
{
    return launch_range(selftest_cvt_bf16_kernel, lo, hi, out, stream);
}

WQ_EXPORT int wq_selftest_decode_fp8(uint64_t* out, void* stream)
{
    if (!out) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    selftest_init_kernel<<<1, 1, 0, st>>>(out);
    WQ_LAUNCH_CHECK();
    selftest_decode_fp8_kernel<<<1, 256, 0, st>>>(out);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_copy_bytes(const void* src, void* dst, int64_t n_bytes, void* stream)
{
    if (n_bytes < 0 || (n_bytes & 15)) return WQ_ERR_SHAPE;
    if (n_bytes == 0) return WQ_OK;
    if (!src || !dst) return WQ_ERR_NULL;
    if (((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return WQ_ERR_ALIGN;
    const int64_t n16 = n_bytes / 16;
    if (n16 == 0) return WQ_OK;
    const int64_t items = cdiv64(n16, 1024);
    copy_kernel<<<grid_for_items(items), 256, kCopyOccupancyPadBytes, (hipStream_t)stream>>>((const u32x4*)src, (u32x4*)dst,
                                                                                           n16, items);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_stream_fold_bytes(const void* src, void* dst, int64_t n_out_bytes, int reads_per_write, void* stream)
{
    if (n_out_bytes < 0 || (n_out_bytes % 16384)) return WQ_ERR_SHAPE;
    if (reads_per_write != 2 && reads_per_write != 4) return WQ_ERR_MODE;
    if (n_out_bytes == 0) return WQ_OK;
    if (!src || !dst) return WQ_ERR_NULL;
    if (((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return WQ_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    if (reads_per_write == 2) {
        const int64_t items = n_out_bytes / (kFoldSteps2 * 4096);
        fold_kernel<2, kFoldSteps2><<<grid_for_items(items), 256, kFoldPadBytes2, st>>>((const u32x4*)src, (u32x4*)dst, items);
    } else {
        const int64_t items = n_out_bytes / (kFoldSteps4 * 4096);
        fold_kernel<4, kFoldSteps4><<<grid_for_items(items), 256, kFoldPadBytes4, st>>>((const u32x4*)src, (u32x4*)dst, items);
    }
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_empty_launch(int64_t workgroups, int threads, void* stream)
{
    if (workgroups <= 0 || workgroups > (1ll << 30) || threads <= 0 || threads > 1024) return WQ_ERR_SHAPE;
    empty_kernel<<<grid_for_items(workgroups), threads, 0, (hipStream_t)stream>>>();
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

// Launch shapes by measurement (% of the 8 TB/s HBM peak, 2 GiB read; input pieces per lane x workgroups per CU):
// 1:2 - 2x2 83.6 (used), 1x4 83.1, 2x3 80.5, 1x8 78.9, 1x2 61, 4x2 78.2;  1:4 - 1x3 79.5 (used), 2x2 75.9, 1x4 75.5, 4x3 73.0,
// 1x8 71.8.  With the dequantiser's own access pattern (8-byte loads, one 16-byte store per load) the 1:2 stream gives the
// same 82.4-82.6 at two workgroups per CU and 76-78 at five.
constexpr int kExpandSteps2 = 2, kExpandSteps4 = 1;
constexpr unsigned kExpandPadBytes2 = 77 * 1024, kExpandPadBytes4 = 50 * 1024;
WQ_EXPORT int wq_stream_expand_bytes(const void* src, void* dst, int64_t n_in_bytes, int writes_per_read, void* stream)
{
    if (n_in_bytes < 0 || (n_in_bytes % 16384)) return WQ_ERR_SHAPE;
    if (writes_per_read != 2 && writes_per_read != 4) return WQ_ERR_MODE;
    if (n_in_bytes == 0) return WQ_OK;
    if (!src || !dst) return WQ_ERR_NULL;
    if (((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return WQ_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    if (writes_per_read == 2) {
        const int64_t items = n_in_bytes / (kExpandSteps2 * 4096);
        expand_kernel<2, kExpandSteps2><<<grid_for_items(items), 256, kExpandPadBytes2, st>>>((const u32x4*)src, (u32x4*)dst, items);
    } else {
        const int64_t items = n_in_bytes / (kExpandSteps4 * 4096);
        expand_kernel<4, kExpandSteps4><<<grid_for_items(items), 256, kExpandPadBytes4, st>>>((const u32x4*)src, (u32x4*)dst, items);
    }
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}
