// Device-side helpers shared by the gfx950 weight-conversion kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/slime_amd_wq.h"

#define WQ_EXPORT extern "C" __attribute__((visibility("default")))

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

namespace wq {

constexpr float kFp8Max = 448.0f;
constexpr uint32_t kBf16Floor1em12 = 0x2B8Du;  // bf16(1e-12): the clamp bound after torch rounds it to bf16
constexpr uint32_t kBf16Inf = 0x7F80u;

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// Global-memory accessors.  Tensor pointers reach the kernels through descriptors (plain void*), for
// which the compiler cannot prove the global address space and would emit FLAT instructions; the casts
// make every access a GLOBAL one.  *_nt variants carry the non-temporal hint (streamed once).
#define WQ_GLOBAL __attribute__((address_space(1)))
template <typename T> __device__ __forceinline__ T ldg_nt(const void* p) { return __builtin_nontemporal_load((const WQ_GLOBAL T*)p); }
template <typename T> __device__ __forceinline__ T ldg(const void* p) { return *(const WQ_GLOBAL T*)p; }
template <typename T> __device__ __forceinline__ void stg_nt(void* p, T v) { __builtin_nontemporal_store(v, (WQ_GLOBAL T*)p); }
// The same with `sc1` next to `nt` (the compiler's non-temporal store emits `nt` only, hence the assembly; 4-, 8- and
// 16-byte forms).  Which of the two streams faster depends on the kernel's read:write mix - measured per kernel, two
// alternating pairs of builds in one session, % of HBM peak `nt` -> `nt sc1`: delta pass (1:1) 77.8 -> 82.1, QAT forward
// (1:1) 79.8 -> 82.1, fake INT4 (1:1) 75.9-77.1 -> 77.4-78.5, FP8-aligned weight (1:1) 73.9 -> 75.0, block-FP8 quantiser (2:1)
// 79.9-80.0 -> 80.6-81.4 and 76.2 -> 76.9 on the Qwen3-4B shapes; but INT4 packer (4:1) 81.5-82.3 -> 81.2-81.4, FP8 -> bf16
// (1:2) 80.1 -> 79.6, INT4 -> bf16 (1:4) 79.0 -> 76.6, per-row FP8 77.3 -> 75.8.  Each kernel uses the one that won.
template <typename T> __device__ __forceinline__ void stg_nt_sc1(void* p, T v)
{
    WQ_GLOBAL T* gp = (WQ_GLOBAL T*)p;
    static_assert(sizeof(T) == 4 || sizeof(T) == 8 || sizeof(T) == 16, "dword, dwordx2 and dwordx4 stores");
    if constexpr (sizeof(T) == 4) asm volatile("global_store_dword %0, %1, off nt sc1" :: "v"(gp), "v"(v) : "memory");
    else if constexpr (sizeof(T) == 8) asm volatile("global_store_dwordx2 %0, %1, off nt sc1" :: "v"(gp), "v"(v) : "memory");
    // A store of more than 8 bytes still reads its data registers after it has issued: a VALU instruction that overwrites
    // them needs two wait states behind it on this family.  The compiler's hazard recogniser adds them for its own stores
    // but does not look inside assembly (without them the FP8-aligned weight of a ragged matrix came out wrong).
    else asm volatile("global_store_dwordx4 %0, %1, off nt sc1\n\ts_nop 1" :: "v"(gp), "v"(v) : "memory");
}
template <typename T> __device__ __forceinline__ void stg(void* p, T v) { *(WQ_GLOBAL T*)p = v; }

// A dword holds two bf16: element 2k in the low half, 2k+1 in the high half.
__device__ __forceinline__ float bf16lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return u2f(w & 0xFFFF0000u); }

// Magnitude bits of a bf16 order exactly like the values, so the block amax is an integer max;
// a NaN (> 0x7F80) wins the max and so propagates like torch.max does.
__device__ __forceinline__ uint32_t pk_absmax(uint32_t acc, uint32_t w)
{
    u16x2 a = __builtin_bit_cast(u16x2, acc);
    u16x2 b = __builtin_bit_cast(u16x2, w & 0x7FFF7FFFu);
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}
__device__ __forceinline__ uint32_t pk_fold(uint32_t acc) { return max(acc & 0xFFFFu, acc >> 16); }

// fp32 -> bf16, round to nearest even, NaN -> 0x7FC0 (sign dropped).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// Software fp32 -> e4m3fn, RNE, non-saturating (|f| > 464, Inf, NaN -> NaN code, sign kept).
// Used on the slow paths (NaN/Inf blocks, generic layouts) and as the checker of the hardware
// conversion in the self-tests.
__device__ __forceinline__ uint32_t f32_to_e4m3fn_sw(float f)
{
    uint32_t u = f2u(f);
    uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7FFFFFFFu;
    uint32_t code;
    if (a >= 0x43F00000u) {
        code = 0x7Fu;
    } else if (a < 0x3C800000u) {
        // k * 2^-9, k = RNE(|f| * 512) in 0..8; adding 2^23 leaves k in the low mantissa bits
        float t = u2f(a) * 512.0f + 8388608.0f;
        code = f2u(t) & 0xFu;
    } else {
        uint32_t c = ((a >> 20) & 0x7FFu) - ((127u - 7u) << 3);
        uint32_t rem = a & 0xFFFFFu;
        if (rem > 0x80000u || (rem == 0x80000u && (c & 1u))) c += 1u;
        code = c;
    }
    return sign | code;
}

// Hardware conversion of two fp32 to two e4m3fn bytes in the low 16 bits (v_cvt_pk_fp8_f32;
// OCP encoding on gfx950).  Inputs must already be within +-448*(1+2^-20): the production
// paths guarantee it, so saturation behaviour is never relied on.
__device__ __forceinline__ uint32_t cvt_pk_fp8_lo(float a, float b, uint32_t old)
{
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
}
__device__ __forceinline__ uint32_t cvt_pk_fp8_hi(float a, float b, uint32_t old)
{
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true);
}

// ---- work-item order ------------------------------------------------------------------------
// Workgroups are dealt to the eight XCDs round-robin in dispatch order, and every XCD has its own L2
// and address-translation cache.  A streaming kernel is measurably faster (about +10 points of HBM
// utilisation on the block quantiser) when each XCD walks a contiguous run of work items instead of
// every eighth one.  Within each span of 8*C dispatch slots, XCD k therefore takes items
// [k*C, (k+1)*C) of the span; slots past the last full span keep the identity order.  The map is a
// bijection on [0, total).
constexpr int kXcds = 8;
__device__ __forceinline__ int64_t xcd_chunked_item(int64_t slot, int64_t total, int C)
{
    if (C <= 0) return slot;
    const int64_t span = (int64_t)kXcds * C;
    const int64_t blk = slot / span;
    if ((blk + 1) * span > total) return slot;
    const int r = (int)(slot - blk * span);
    return blk * span + (int64_t)(r % kXcds) * C + r / kXcds;
}

// Owner of flat work item t in a grouped launch: the largest i with start[i] <= t, where start[] is the
// exclusive prefix sum of per-tensor item counts (n + 1 entries, start[n] = total > t).  The first probe
// is the proportional guess - exact when all tensors have equally many items (the experts of a layer) -
// and the binary search only runs on the side of the guess that holds t.  All values are
// workgroup-uniform, so this is scalar code.
__device__ __forceinline__ int find_owner(const int64_t* __restrict__ start, int n, int64_t t, int64_t total)
{
    int g = (int)((float)t * ((float)n / (float)total));
    g = g < 0 ? 0 : (g > n - 1 ? n - 1 : g);
    int lo = 0, hi = n;
    if (start[g] <= t) {
        if (t < start[g + 1]) return g;
        lo = g + 1;
    } else {
        hi = g;
    }
    while (hi - lo > 1) {  // invariant: start[lo] <= t < start[hi]
        const int mid = (lo + hi) >> 1;
        if (start[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

// ---- pass-through work item of a bucket launch ------------------------------------------------------
// Copies n bytes (n <= WQ_BUCKET_COPY_BYTES) with the 256 lanes of the workgroup.  The widest access that the
// alignment of both pointers allows is used; all loads of the 16-byte form are issued before the first store.
constexpr int kCopyItemBytes = WQ_BUCKET_COPY_BYTES;
template <typename V>
__device__ __forceinline__ void copy_units(const char* src, char* dst, int n)
{
    const int units = n / (int)sizeof(V);
    for (int u = threadIdx.x; u < units; u += 256) stg_nt<V>(dst + (size_t)u * sizeof(V), ldg_nt<V>(src + (size_t)u * sizeof(V)));
    for (int b = units * (int)sizeof(V) + threadIdx.x; b < n; b += 256) stg<uint8_t>(dst + b, ldg<uint8_t>(src + b));
}
__device__ __forceinline__ void copy_item(const void* src_, void* dst_, int n)
{
    const char* src = (const char*)src_;
    char* dst = (char*)dst_;
    const uintptr_t a = (uintptr_t)src | (uintptr_t)dst;
    if ((a & 15) == 0) {
        constexpr int kSteps = kCopyItemBytes / (256 * 16);
        const int pieces = n >> 4;
        u32x4 v[kSteps];
#pragma unroll
        for (int i = 0; i < kSteps; ++i) {
            const int p = i * 256 + threadIdx.x;
            v[i] = ldg_nt<u32x4>(src + (size_t)(p < pieces ? p : 0) * 16);      // lanes past the end re-read piece 0
        }
#pragma unroll
        for (int i = 0; i < kSteps; ++i) {
            const int p = i * 256 + threadIdx.x;
            if (p < pieces) stg_nt<u32x4>(dst + (size_t)p * 16, v[i]);
        }
        for (int b = (pieces << 4) + threadIdx.x; b < n; b += 256) stg<uint8_t>(dst + b, ldg<uint8_t>(src + b));
    } else if ((a & 7) == 0) {
        copy_units<u32x2>(src, dst, n);
    } else if ((a & 3) == 0) {
        copy_units<uint32_t>(src, dst, n);
    } else if ((a & 1) == 0) {
        copy_units<uint16_t>(src, dst, n);
    } else {
        copy_units<uint8_t>(src, dst, n);
    }
}

// ---- 16-lane (DPP row) all-reduce max.  After it every lane of the row holds the row max.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}
__device__ __forceinline__ uint32_t row16_max_u32(uint32_t v)
{
    v = max(v, dpp_u32<0xB1>(v));   // quad_perm [1,0,3,2]
    v = max(v, dpp_u32<0x4E>(v));   // quad_perm [2,3,0,1]
    v = max(v, dpp_u32<0x141>(v));  // row_half_mirror
    v = max(v, dpp_u32<0x140>(v));  // row_mirror
    return v;
}
// fp32 max / min with the DPP-permuted copy of the same register in ONE instruction (v_max_f32_dpp).  Written as
// inline assembly because the compiler, from fmaxf(v, dpp(v)), emits four (copy, DPP move, canonicalise, max) - and the
// group-wise INT4 kernels, which run these reductions once per 8 elements, are bound by VALU issue.  A quiet NaN operand
// is dropped, as fmaxf / fminf do; a signalling NaN (which no torch operation produces) becomes a quiet NaN result.
// `s_nop 1`: a DPP read needs two wait states after the VALU write of its source.
#define WQ_DPP_F32_OP(NAME, OP, CTRL)                                                                        \
    __device__ __forceinline__ float NAME(float v)                                                           \
    {                                                                                                        \
        float r;                                                                                             \
        asm("s_nop 1\n\t" OP " %0, %1, %1 " CTRL " row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v));          \
        return r;                                                                                            \
    }
WQ_DPP_F32_OP(max_f32_quad_1032, "v_max_f32_dpp", "quad_perm:[1,0,3,2]")
WQ_DPP_F32_OP(max_f32_quad_2301, "v_max_f32_dpp", "quad_perm:[2,3,0,1]")
WQ_DPP_F32_OP(max_f32_half_mirror, "v_max_f32_dpp", "row_half_mirror")
WQ_DPP_F32_OP(max_f32_mirror, "v_max_f32_dpp", "row_mirror")
WQ_DPP_F32_OP(min_f32_quad_1032, "v_min_f32_dpp", "quad_perm:[1,0,3,2]")
WQ_DPP_F32_OP(min_f32_quad_2301, "v_min_f32_dpp", "quad_perm:[2,3,0,1]")
WQ_DPP_F32_OP(min_f32_half_mirror, "v_min_f32_dpp", "row_half_mirror")
WQ_DPP_F32_OP(min_f32_mirror, "v_min_f32_dpp", "row_mirror")
#undef WQ_DPP_F32_OP

// all-reduce over L = 4, 8 or 16 adjacent lanes (L = 16: a DPP row)
template <int L>
__device__ __forceinline__ float lanes_max_f32(float v)
{
    v = max_f32_quad_1032(v);
    v = max_f32_quad_2301(v);
    if (L >= 8) v = max_f32_half_mirror(v);
    if (L >= 16) v = max_f32_mirror(v);
    return v;
}
template <int L>
__device__ __forceinline__ float lanes_min_f32(float v)
{
    v = min_f32_quad_1032(v);
    v = min_f32_quad_2301(v);
    if (L >= 8) v = min_f32_half_mirror(v);
    if (L >= 16) v = min_f32_mirror(v);
    return v;
}
__device__ __forceinline__ float row16_max_f32(float v) { return lanes_max_f32<16>(v); }
__device__ __forceinline__ float row16_min_f32(float v) { return lanes_min_f32<16>(v); }
// NaN-propagating fp32 maximum over the wavefront
__device__ __forceinline__ float wave64_max_nanprop_f32(float v)
{
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const float o = u2f((uint32_t)__shfl_xor((int)f2u(v), m));
        v = (v != v || o != o) ? __builtin_nanf("") : fmaxf(v, o);
    }
    return v;
}
__device__ __forceinline__ uint32_t wave64_max_u32(uint32_t v)
{
    v = row16_max_u32(v);
    v = max(v, (uint32_t)__shfl_xor((int)v, 16));
    v = max(v, (uint32_t)__shfl_xor((int)v, 32));
    return v;
}

// ---- scale rules -------------------------------------------------------------------------

// mode TORCH: amax is a bf16 magnitude bit pattern (possibly NaN/Inf).
__device__ __forceinline__ float fp8_scale_torch(uint32_t amax_bf16_bits)
{
    uint32_t a = amax_bf16_bits < kBf16Floor1em12 ? kBf16Floor1em12 : amax_bf16_bits;
    return u2f(a << 16) / kFp8Max;
}
// mode TORCH_DEVICE: the same expression as torch's GPU kernels evaluate it.  There `tensor / python_scalar` is
// computed as tensor * (1.0f / scalar), so the scale is f32(amax) * RN(1/448) - up to one ulp away from the
// quotient above.
__device__ __forceinline__ float fp8_scale_torch_device(uint32_t amax_bf16_bits)
{
    uint32_t a = amax_bf16_bits < kBf16Floor1em12 ? kBf16Floor1em12 : amax_bf16_bits;
    return u2f(a << 16) * (1.0f / kFp8Max);
}
// mode TRITON: fp32 amax floored at 1e-10f.
__device__ __forceinline__ float fp8_scale_triton(uint32_t amax_bf16_bits)
{
    float a = u2f(amax_bf16_bits << 16);
    a = (a != a) ? a : fmaxf(a, 1e-10f);
    return a / kFp8Max;
}

// mode UE8M0: fp32 amax floored at 1e-4f, scale = the smallest power of two >= amax / 448 (a power of two maps to
// itself, as 2^ceil(log2(.)) does).  amax / 448 is a normal number here (>= 2.2e-7); NaN and Inf pass through.
__device__ __forceinline__ float fp8_scale_ue8m0(uint32_t amax_bf16_bits)
{
    float a = u2f(amax_bf16_bits << 16);
    a = (a != a) ? a : fmaxf(a, 1e-4f);
    const uint32_t u = f2u(a / kFp8Max);
    if ((u & 0x7F800000u) == 0x7F800000u || (u & 0x007FFFFFu) == 0u) return u2f(u);
    return u2f((u & 0x7F800000u) + 0x00800000u);
}

// The two torch modes divide every element by the scale; the Triton and UE8M0 modes multiply by its reciprocal.
constexpr bool fp8_mode_divides(int mode) { return mode != WQ_FP8_MODE_TRITON && mode != WQ_FP8_MODE_UE8M0; }

// Per-block constants of the element function.
struct Fp8BlockParams {
    float scale;  // value stored to the scale tensor
    float rcp;    // correctly rounded 1/scale
    bool fast;    // amax finite: the refinement below reproduces IEEE x/scale exactly
};

template <int MODE>
__device__ __forceinline__ Fp8BlockParams fp8_block_params(uint32_t amax_bf16_bits)
{
    Fp8BlockParams p;
    p.scale = MODE == WQ_FP8_MODE_TORCH          ? fp8_scale_torch(amax_bf16_bits)
              : MODE == WQ_FP8_MODE_TORCH_DEVICE ? fp8_scale_torch_device(amax_bf16_bits)
              : MODE == WQ_FP8_MODE_UE8M0        ? fp8_scale_ue8m0(amax_bf16_bits)
                                                 : fp8_scale_triton(amax_bf16_bits);
    p.rcp = 1.0f / p.scale;
    p.fast = amax_bf16_bits < kBf16Inf;
    return p;
}

// q = RN(x / scale) without a per-element division: q0 = RN(x*r), rem = x - q0*scale (exact in an
// FMA), q = RN(q0 + rem*r).  With r the correctly rounded reciprocal this is the correctly rounded
// quotient for every (x, scale) pair the block quantiser can produce; wq_selftest_fp8_elem checks the
// whole domain against the IEEE division.  An exact zero loses its sign here (+0 + -0 = +0); callers
// restore the sign bit on the fp8 code.
__device__ __forceinline__ float div_by_scale(float x, float scale, float rcp)
{
    float q0 = x * rcp;
    float rem = __builtin_fmaf(-q0, scale, x);
    return __builtin_fmaf(rem, rcp, q0);
}

// mode TORCH slow/reference element function: IEEE division, NaN-propagating clamp, software RNE.
__device__ __forceinline__ uint32_t fp8_elem_exact_torch(float x, float scale)
{
    float q = x / scale;
    if (q == q) q = fminf(fmaxf(q, -kFp8Max), kFp8Max);
    return f32_to_e4m3fn_sw(q);
}
__device__ __forceinline__ uint32_t fp8_elem_exact_triton(float x, float s_inv)
{
    float q = x * s_inv;
    if (q == q) q = fminf(fmaxf(q, -kFp8Max), kFp8Max);
    return f32_to_e4m3fn_sw(q);
}

// Sign bits of the four bf16 in (w0, w1) moved to bits 7, 15, 23, 31.
__device__ __forceinline__ uint32_t bf16x4_signs_to_bytes(uint32_t w0, uint32_t w1)
{
    // bytes picked: w0.b1, w0.b3, w1.b1, w1.b3  (v_perm_b32: selector bytes 0-3 = second operand)
    return __builtin_amdgcn_perm(w1, w0, 0x07050301u) & 0x80808080u;
}

// Four bf16 (two dwords) -> four e4m3fn bytes, production path (block amax finite).
template <int MODE>
__device__ __forceinline__ uint32_t fp8_quant4_fast(uint32_t w0, uint32_t w1, const Fp8BlockParams& p)
{
    float q0, q1, q2, q3;
    if (fp8_mode_divides(MODE)) {
        q0 = div_by_scale(bf16lo(w0), p.scale, p.rcp);
        q1 = div_by_scale(bf16hi(w0), p.scale, p.rcp);
        q2 = div_by_scale(bf16lo(w1), p.scale, p.rcp);
        q3 = div_by_scale(bf16hi(w1), p.scale, p.rcp);
    } else {
        q0 = bf16lo(w0) * p.rcp;
        q1 = bf16hi(w0) * p.rcp;
        q2 = bf16lo(w1) * p.rcp;
        q3 = bf16hi(w1) * p.rcp;
    }
    // |q| <= 448*(1+2^-22): clamping to +-448 cannot change the RNE result (next boundary is 464),
    // so the clamp of the reference is a no-op here and is skipped.
    uint32_t r = cvt_pk_fp8_lo(q0, q1, 0u);
    r = cvt_pk_fp8_hi(q2, q3, r);
    if (fp8_mode_divides(MODE)) r |= bf16x4_signs_to_bytes(w0, w1);
    return r;
}

template <int MODE>
__device__ __forceinline__ uint32_t fp8_quant1_exact(float x, const Fp8BlockParams& p)
{
    return fp8_mode_divides(MODE) ? fp8_elem_exact_torch(x, p.scale) : fp8_elem_exact_triton(x, p.rcp);
}

template <int MODE>
__device__ __forceinline__ uint32_t fp8_quant4_exact(uint32_t w0, uint32_t w1, const Fp8BlockParams& p)
{
    return fp8_quant1_exact<MODE>(bf16lo(w0), p) | (fp8_quant1_exact<MODE>(bf16hi(w0), p) << 8) |
           (fp8_quant1_exact<MODE>(bf16lo(w1), p) << 16) | (fp8_quant1_exact<MODE>(bf16hi(w1), p) << 24);
}

// ---- INT4 ---------------------------------------------------------------------------------

__device__ __forceinline__ float int4_scale_sym(float amax) { return fmaxf(amax * (1.0f / 7.0f), 1e-5f); }

// rintf(q) + 8 in the low four bits: 12582912 = 1.5 * 2^23 makes the add round q to an integer
// (half to even) and leaves it, offset by 8, in the low mantissa bits.
constexpr float kRoundMagic = 12582920.0f;        // 1.5 * 2^23 + 8
constexpr uint32_t kRoundMagicBits = 0x4B400000u;  // bits of (kRoundMagic + n) are kRoundMagicBits + n for n in 0..15
__device__ __forceinline__ uint32_t nibble_of(float q) { return f2u(q + kRoundMagic) & 0xFu; }

// Sum over j of (kRoundMagicBits << 4j) modulo 2^32: what the un-masked accumulation of pack8_sym
// carries on top of the packed nibbles.
constexpr uint32_t magic_carry()
{
    uint32_t s = 0;
    for (int j = 0; j < 8; ++j) s += (uint32_t)((uint64_t)kRoundMagicBits << (4 * j));
    return s;
}

// Correctly rounded 1/scale from the hardware approximation and one Newton step; equal to the IEEE
// reciprocal for every scale the symmetric rule can produce from a bf16 amax (wq_selftest_int4_elem
// checks it together with the quotients).
__device__ __forceinline__ float rcp_refined(float s)
{
    const float r0 = __builtin_amdgcn_rcpf(s);
    return __builtin_fmaf(__builtin_fmaf(-s, r0, 1.0f), r0, r0);
}

// acc's byte BYTE <- low byte of (q + magic): v_add_f32_sdwa with the other bytes of the destination preserved.
// `s_nop 0`: on this family a VALU instruction that writes part of a register (dst_sel other than DWORD) needs one wait
// state before a VALU instruction that reads the register - the next add into the same word (UNUSED_PRESERVE reads the
// destination) or the final shift-or.  The compiler's hazard recogniser does not look inside inline assembly, so the
// helper carries the wait state itself, like the DPP helpers above.
#define WQ_ADD_TO_BYTE(BYTE)                                                                                        \
    __device__ __forceinline__ void add_magic_to_byte##BYTE(uint32_t& acc, float q, float magic)                    \
    {                                                                                                               \
        asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_" #BYTE " dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\ts_nop 0" \
            : "+v"(acc) : "v"(q), "v"(magic));                                                                      \
    }
WQ_ADD_TO_BYTE(1)
WQ_ADD_TO_BYTE(2)
WQ_ADD_TO_BYTE(3)
#undef WQ_ADD_TO_BYTE

// Eight exact quotients -> one packed word, 9 instructions after the divisions: for |rintf(q)| <= 7 the low BYTE of
// bits(q + kRoundMagic) is rintf(q) + 8 (its upper nibble is zero), so the even elements are gathered as the four
// bytes of one register and the odd ones of another - each add writing its byte straight into place - and
// even | odd << 4 is the word sum_j (q_j + 8) << 4j.
__device__ __forceinline__ uint32_t pack8_sym_bytes(const float (&x)[8], float scale, float rcp)
{
    const float magic = kRoundMagic;
    uint32_t even = f2u(div_by_scale(x[0], scale, rcp) + magic);      // byte 0; bytes 1-3 are overwritten below
    uint32_t odd = f2u(div_by_scale(x[1], scale, rcp) + magic);
    add_magic_to_byte1(even, div_by_scale(x[2], scale, rcp), magic);
    add_magic_to_byte1(odd, div_by_scale(x[3], scale, rcp), magic);
    add_magic_to_byte2(even, div_by_scale(x[4], scale, rcp), magic);
    add_magic_to_byte2(odd, div_by_scale(x[5], scale, rcp), magic);
    add_magic_to_byte3(even, div_by_scale(x[6], scale, rcp), magic);
    add_magic_to_byte3(odd, div_by_scale(x[7], scale, rcp), magic);
    return (odd << 4) | even;
}

// Eight exact quotients -> one packed word.  For |rintf(q)| <= 7 the float q + kRoundMagic has the bit
// pattern kRoundMagicBits + (rintf(q) + 8), so the words can be shifted and added without masking and the
// constant part removed once at the end: one add and one shift-add per element.
__device__ __forceinline__ uint32_t pack8_sym(const float (&x)[8], float scale, float rcp)
{
    uint32_t acc = f2u(div_by_scale(x[0], scale, rcp) + kRoundMagic);
#pragma unroll
    for (int j = 1; j < 8; ++j) acc += f2u(div_by_scale(x[j], scale, rcp) + kRoundMagic) << (4 * j);
    return acc - magic_carry();
}

// Host-side launch helpers.
inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Grid for n workgroups of 256 threads, addressed in the kernels as blockIdx.x + blockIdx.y * gridDim.x.
// x stays at or below 2^22 workgroups so that gridDim.x * blockDim.x fits 32 bits.
inline dim3 grid_for_items(int64_t n)
{
    const int64_t lim = 1 << 22;
    if (n <= lim) return dim3((unsigned)(n > 0 ? n : 1), 1, 1);
    return dim3((unsigned)lim, (unsigned)cdiv64(n, lim), 1);
}

}  // namespace wq

#define WQ_LAUNCH_CHECK()                              \
    do {                                               \
        hipError_t e_ = hipGetLastError();             \
        if (e_ != hipSuccess) return (int)e_;          \
    } while (0)
