/*
 * CPU oracle for the low-precision weight-conversion path.  TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped package links, loads or calls this file; only tests/, the
 * smoke check and the cpu_baseline leg of the benchmark do, and only as the checker.
 *
 * Every function is a scalar restatement of the arithmetic of one reference function
 * (paths relative to the reference checkout):
 *
 *   wqo_fp8_block_quant   mode 0: tools/convert_hf_to_fp8.py:41-75 (block_fp8) as torch evaluates it on CPU tensors
 *                         mode 2: the same, as torch evaluates it on GPU tensors (scalar division = reciprocal multiply)
 *                         mode 1: slime/backends/megatron_utils/kernels/fp8_kernel.py:24-58
 *                         mode 3: power-of-two (UE8M0) scales, the branch of _quantize_param at
 *                                 megatron_to_hf/processors/quantizer_fp8.py:103-106 - its arithmetic is sglang's
 *                                 quant_weight_ue8m0 (sglang v0.5.15.post1, NOT vendored in the reference; it wraps
 *                                 DeepGEMM's per_block_cast_to_fp8 with use_ue8m0): fp32 amax floored at 1e-4,
 *                                 sf = 2^ceil(log2(amax / 448)), y = e4m3(x * (1 / sf)), no clamp
 *   wqo_fp8_channel_quant tools/convert_hf_to_fp8.py:78-83 (channel_fp8)
 *   wqo_fp8_tensor_quant  tools/convert_hf_to_fp8.py:86-91 (tensor_fp8), same arithmetic as
 *                         megatron_to_hf/processors/quantizer_fp8.py:114-116
 *   wqo_fp8_tensor_quant_any  the same function on fp16 / fp32 weights (channel_fp8 on those dtypes is
 *                         wqo_fp8_block_quant_any with blocks of one row)
 *   wqo_fp8_block_dequant mode 0: tools/fp8_cast_bf16.py:16-41 (weight_dequant)
 *                         mode 1: slime/backends/megatron_utils/hf_to_megatron/common.py:42-56
 *   wqo_int4_fake_quant   slime/backends/megatron_utils/kernels/int4_qat/fake_int4_quant_cuda.cu:37-267
 *   wqo_int4_pack_layer   tools/convert_hf_to_int4_direct.py:32-153 (pack_layer, quantize,
 *                         round_to_quantized_type_dtype, pack_to_int32), literal chain
 *   wqo_int4_dequant      tools/convert_k2_thinking_int4_to_bf16.py:55-84 (_dequantize_tensor)
 *   wqo_int4_fake_ste     docker/patch/latest/megatron.patch:212-246 (_FakeInt4QuantizationSTE.forward)
 *
 * Number formats are handled with integer bit manipulation written for this file
 * (no library conversion is used), so that the torch restatement in torch_ref.py and
 * this file are two independent witnesses.  Pinning status:
 *   - conversions (fp32->e4m3fn RNE, e4m3fn->fp32, fp32->bf16 RNE): checked against
 *     torch's casts over dense sweeps of the input domain (tests/test_oracle_formats.py).
 *   - block/channel/tensor FP8 quant and both dequant modes: checked against the
 *     op-for-op torch restatement, against hand-derived known answers (zero-block scale
 *     bits 0x27212492, -0.0 -> 0x80, amax element -> 0x7E/0xFE), against the invariants
 *     of the reference's tests/test_block_fp8_zero_block.py:38-75 and the known-answer
 *     test tests/test_hf_to_megatron.py:345-358.
 *   - fp8 mode 1 (Triton kernel): the restatement assumes IEEE round-to-nearest for both
 *     divisions and the multiply.  No reference test or vector exists, and on NVIDIA hardware
 *     Triton's "/" is not guaranteed IEEE-exact (PARITY UNPINNED there).  On MI355X it is
 *     pinned: oracle/triton_ref.py restates the kernel in Triton and the GPU tests find it
 *     bit-identical to this file's reading for every bf16 amax and every bf16 value.
 *   - fp8 mode 3: PARITY UNPINNED.  The algorithm lives in a third-party dependency that is absent from the
 *     reference checkout; it is restated from that library's published source as remembered, and pinned only by
 *     what the mathematics fixes: the scale is the smallest power of two >= max(amax, 1e-4) / 448, the codes are one
 *     RNE of an exactly scaled value and never exceed 448, and the literal log2 / ceil / pow chain in torch_ref.py
 *     agrees with the exponent arithmetic used here for every bf16 amax.
 *   - fp8 mode 2 and the bf16 divisor of the per-tensor form: pinned by torch's own GPU
 *     kernels run on the same inputs (tests/test_gpu_fp8.py).
 *   - wqo_int4_fake_quant: the reference kernel is CUDA-only, has no test and cannot be
 *     built here without generated (hipified) code: PARITY UNPINNED against reference
 *     output.  Pinned to the source text by exact rational arithmetic on small inputs,
 *     closed-form cases and invariants (tests/test_oracle_int4.py).
 *   - wqo_int4_pack_layer: torch-primitive chain; checked op-for-op against torch_ref.py
 *     and against the closed form sum((q_j+8) << 4j).
 *
 * Build: make -C oracle   (gcc -O2 -fno-fast-math -ffp-contract=off; SSE2 fp32 = IEEE).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define WQO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ formats */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

WQO_API float wqo_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; NaN -> 0x7FC0 (what torch's cast produces). */
WQO_API uint16_t wqo_f32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* fp32 -> OCP e4m3fn (bias 7, no infinities, 0x7F/0xFF = NaN), round to nearest even,
 * non-saturating: anything that rounds above 448 (|f| > 464) and Inf/NaN become NaN with
 * the sign kept.  Subnormal results are multiples of 2^-9. */
WQO_API uint8_t wqo_f32_to_e4m3fn(float f)
{
    uint32_t u = f2u(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7FFFFFFFu;
    uint8_t code;
    if (a >= 0x43F00000u) {                 /* >= 480, Inf, NaN */
        code = 0x7F;
    } else if (a < 0x3C800000u) {           /* < 2^-6: result is k * 2^-9, k in 0..8 */
        float t = u2f(a) * 512.0f;          /* exact: power-of-two scaling upward */
        /* round half to even on an exactly representable t in [0, 8) */
        float fl = floorf(t);
        float r = t - fl;
        uint32_t k = (uint32_t)fl;
        if (r > 0.5f || (r == 0.5f && (k & 1u))) k += 1;
        code = (uint8_t)k;                  /* k == 8 is 0x08 = 2^-6, the smallest normal */
    } else {
        uint32_t e = (a >> 23) - 127u + 7u; /* biased e4m3 exponent, 1..15 */
        uint32_t m = (a >> 20) & 7u;
        uint32_t rem = a & 0xFFFFFu;
        uint32_t c = (e << 3) | m;
        if (rem > 0x80000u || (rem == 0x80000u && (m & 1u))) c += 1; /* carry may bump exponent */
        code = (uint8_t)c;                  /* c <= 0x7F because a < 480 */
    }
    return (uint8_t)(sign | code);
}

WQO_API float wqo_e4m3fn_to_f32(uint8_t b)
{
    uint32_t sign = ((uint32_t)b & 0x80u) << 24;
    uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
    uint32_t u;
    if (e == 0xFu && m == 7u) u = 0x7FC00000u;
    else if (e == 0) {
        /* m * 2^-9 */
        float v = (float)m * 0.001953125f;
        u = f2u(v);
    } else u = ((e - 7u + 127u) << 23) | (m << 20);
    return u2f(u | sign);
}

WQO_API void wqo_f32_to_e4m3fn_n(const float *x, uint8_t *y, int64_t n)
{ for (int64_t i = 0; i < n; ++i) y[i] = wqo_f32_to_e4m3fn(x[i]); }
WQO_API void wqo_e4m3fn_to_f32_n(const uint8_t *x, float *y, int64_t n)
{ for (int64_t i = 0; i < n; ++i) y[i] = wqo_e4m3fn_to_f32(x[i]); }
WQO_API void wqo_f32_to_bf16_n(const float *x, uint16_t *y, int64_t n)
{ for (int64_t i = 0; i < n; ++i) y[i] = wqo_f32_to_bf16(x[i]); }

/* ------------------------------------------------------------------ helpers */

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

/* torch.max / torch.clamp propagate NaN; fmaxf does not. */
static inline float max_nanprop(float a, float b)
{ if (a != a) return a; if (b != b) return b; return a > b ? a : b; }

static inline float clamp_nanprop(float v, float lo, float hi)
{ if (v != v) return v; if (v < lo) return lo; if (v > hi) return hi; return v; }

#define FP8_MAX 448.0f

/* bf16 value of the Python scalar 1e-12 after torch rounds it into a bf16 clamp bound. */
#define BF16_1EM12_BITS 0x2B8Du

/* amax in the weight dtype (bf16: |x| and max are exact), then clamp(min=1e-12) in bf16,
 * then fp32 / 448.   tools/convert_hf_to_fp8.py:59-65,79-80,87 */
static inline float scale_from_amax_mode0(float amax_bf16_exact)
{
    float floor_v = wqo_bf16_to_f32(BF16_1EM12_BITS);
    float a = amax_bf16_exact;
    if (a == a && a < floor_v) a = floor_v;
    return a / FP8_MAX;
}

/* The same expression as torch's GPU kernels evaluate it (mode 2): `tensor / python_scalar` is computed there
 * as tensor * (1.0f / scalar) (aten/src/ATen/native/cuda/BinaryDivTrueKernel.cu, the is_cpu_scalar branch), so the
 * scale is amax * RN(1/448).  The reference tool loads its tensors onto the accelerator
 * (tools/convert_hf_to_fp8.py:127), so this is what it writes when a GPU is present; mode 0 is what its CPU test
 * (tests/test_block_fp8_zero_block.py) exercises. */
static inline float scale_from_amax_mode2(float amax_bf16_exact)
{
    float floor_v = wqo_bf16_to_f32(BF16_1EM12_BITS);
    float a = amax_bf16_exact;
    if (a == a && a < floor_v) a = floor_v;
    volatile float inv = 1.0f / FP8_MAX;
    return a * inv;
}
static inline float scale_torch(float amax, int mode)
{ return mode == 2 ? scale_from_amax_mode2(amax) : scale_from_amax_mode0(amax); }

static inline uint8_t quant_elem_mode0(float x, float scale)
{
    float q = x / scale;                               /* true fp32 division, :67 */
    q = clamp_nanprop(q, -FP8_MAX, FP8_MAX);           /* :68 */
    return wqo_f32_to_e4m3fn(q);                       /* :70 */
}

/* fp8_kernel.py:51-55 : fp32 amax floored at eps, scale = amax/448, multiply by 1/scale. */
static inline float scale_from_amax_mode1(float amax)
{
    /* tl.maximum(a, eps): NaN handling of the reference kernel is not pinned; finite only */
    float a = amax > 1e-10f ? amax : 1e-10f;
    if (amax != amax) a = amax;
    return a / FP8_MAX;
}

/* Smallest power of two >= v for a positive finite v (a power of two maps to itself); NaN and Inf pass through. */
static inline float pow2_ceil(float v)
{
    uint32_t u = f2u(v);
    if ((u & 0x7F800000u) == 0x7F800000u) return v;
    if ((u & 0x7F800000u) == 0) {                       /* subnormal: scale up, recurse, scale down */
        return pow2_ceil(v * 0x1p64f) * 0x1p-64f;
    }
    if ((u & 0x007FFFFFu) == 0) return v;
    return u2f((u & 0x7F800000u) + 0x00800000u);
}
static inline float scale_from_amax_mode3(float amax)
{
    float a = amax < 1e-4f ? 1e-4f : amax;              /* .clamp(1e-4); NaN stays NaN */
    return pow2_ceil(a / FP8_MAX);
}
static inline uint8_t quant_elem_mode3(float x, float s_inv) { return wqo_f32_to_e4m3fn(x * s_inv); }

static inline uint8_t quant_elem_mode1(float x, float s_inv)
{
    float q = x * s_inv;
    q = clamp_nanprop(q, -FP8_MAX, FP8_MAX);
    return wqo_f32_to_e4m3fn(q);
}

/* ------------------------------------------------------------------ FP8 quant */

/* x: bf16 bits, element (i,j) at x[i*sx_m + j*sx_n].  y: [M,N] contiguous bytes.
 * s: [cdiv(M,bm), cdiv(N,bn)] contiguous fp32.  Out-of-range elements of an edge block
 * count as +0.0 (F.pad value=0.0 / masked load other=0.0). */
/* fp16 bits -> fp32 (exact) */
WQO_API float wqo_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0x1F) return u2f(sign | 0x7F800000u | (m << 13));
    if (e == 0) {
        float v = (float)m * 0x1p-24f;          /* subnormal: m * 2^-24, exact */
        return sign ? -v : v;
    }
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* element (any of the dtypes the reference functions take) -> fp32, exact.  dtype: 0 bf16, 1 fp32, 2 fp16 */
static inline float load_any(const void *x, int dtype, int64_t off)
{
    if (dtype == 1) return ((const float *)x)[off];
    if (dtype == 2) return wqo_f16_to_f32(((const uint16_t *)x)[off]);
    return wqo_bf16_to_f32(((const uint16_t *)x)[off]);
}

/* clamp(min=1e-12) happens in the weight dtype: the bound is 1e-12 rounded to that dtype - 0x2B8D in bf16,
 * 0 in fp16 (1e-12 is below half the smallest fp16 subnormal), 1e-12f in fp32. */
static inline float torch_floor(int dtype)
{ return dtype == 1 ? 1e-12f : dtype == 2 ? 0.0f : wqo_bf16_to_f32(BF16_1EM12_BITS); }

WQO_API int wqo_fp8_block_quant_any(const void *x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                                    int64_t bm, int64_t bn, int mode, uint8_t *y, float *s)
{
    if (M < 0 || N < 0 || bm <= 0 || bn <= 0 || mode < 0 || mode > 2 || dtype < 0 || dtype > 2) return 1;
    int64_t nt = cdiv(M, bm), kt = cdiv(N, bn);
    volatile float inv448 = 1.0f / FP8_MAX;
#pragma omp parallel for schedule(static)
    for (int64_t bi = 0; bi < nt; ++bi) {
        for (int64_t bj = 0; bj < kt; ++bj) {
            int64_t r0 = bi * bm, r1 = r0 + bm < M ? r0 + bm : M;
            int64_t c0 = bj * bn, c1 = c0 + bn < N ? c0 + bn : N;
            float amax = 0.0f;
            for (int64_t i = r0; i < r1; ++i)
                for (int64_t j = c0; j < c1; ++j)
                    amax = max_nanprop(amax, fabsf(load_any(x, dtype, i * sx_m + j * sx_n)));
            float scale, s_inv = 0.0f;
            if (mode == 1) { scale = scale_from_amax_mode1(amax); s_inv = 1.0f / scale; }
            else {
                float a = amax;
                if (a == a && a < torch_floor(dtype)) a = torch_floor(dtype);
                scale = mode == 2 ? a * inv448 : a / FP8_MAX;
            }
            s[bi * kt + bj] = scale;
            for (int64_t i = r0; i < r1; ++i)
                for (int64_t j = c0; j < c1; ++j) {
                    float v = load_any(x, dtype, i * sx_m + j * sx_n);
                    y[i * N + j] = mode != 1 ? quant_elem_mode0(v, scale) : quant_elem_mode1(v, s_inv);
                }
        }
    }
    return 0;
}

WQO_API int wqo_fp8_block_quant(const uint16_t *x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                                int64_t bm, int64_t bn, int mode, uint8_t *y, float *s)
{
    if (M < 0 || N < 0 || bm <= 0 || bn <= 0 || mode < 0 || mode > 3) return 1;
    int64_t nt = cdiv(M, bm), kt = cdiv(N, bn);
#pragma omp parallel for schedule(static)
    for (int64_t bi = 0; bi < nt; ++bi) {
        for (int64_t bj = 0; bj < kt; ++bj) {
            int64_t r0 = bi * bm, r1 = r0 + bm < M ? r0 + bm : M;
            int64_t c0 = bj * bn, c1 = c0 + bn < N ? c0 + bn : N;
            float amax = 0.0f;                 /* padding contributes |+0| */
            for (int64_t i = r0; i < r1; ++i)
                for (int64_t j = c0; j < c1; ++j)
                    amax = max_nanprop(amax, fabsf(wqo_bf16_to_f32(x[i * sx_m + j * sx_n])));
            float scale, s_inv = 0.0f;
            if (mode == 3) { scale = scale_from_amax_mode3(amax); s_inv = 1.0f / scale; }
            else if (mode != 1) scale = scale_torch(amax, mode);
            else { scale = scale_from_amax_mode1(amax); s_inv = 1.0f / scale; }
            s[bi * kt + bj] = scale;
            for (int64_t i = r0; i < r1; ++i)
                for (int64_t j = c0; j < c1; ++j) {
                    float v = wqo_bf16_to_f32(x[i * sx_m + j * sx_n]);
                    y[i * N + j] = mode == 3 ? quant_elem_mode3(v, s_inv)
                                   : mode != 1 ? quant_elem_mode0(v, scale) : quant_elem_mode1(v, s_inv);
                }
        }
    }
    return 0;
}

WQO_API int wqo_fp8_channel_quant(const uint16_t *x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                                  int mode, uint8_t *y, float *s)
{
    if (M < 0 || N < 0 || (mode != 0 && mode != 2)) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i) {
        float amax = 0.0f;
        for (int64_t j = 0; j < N; ++j)
            amax = max_nanprop(amax, fabsf(wqo_bf16_to_f32(x[i * sx_m + j * sx_n])));
        float scale = scale_torch(amax, mode);
        s[i] = scale;
        for (int64_t j = 0; j < N; ++j)
            y[i * N + j] = quant_elem_mode0(wqo_bf16_to_f32(x[i * sx_m + j * sx_n]), scale);
    }
    return 0;
}

/* tensor_fp8 (convert_hf_to_fp8.py:86-91) and the per-tensor branch of _quantize_param
 * (quantizer_fp8.py:114-116): the scale is a 0-dim fp32 tensor, which does not take part in torch's
 * type promotion, so `weight / scale` is a bf16 tensor: the fp32 quotient is rounded to bf16 BEFORE the
 * clamp and the e4m3 cast (two roundings).  block_fp8 and channel_fp8 divide by a dimensioned fp32
 * tensor and keep the fp32 quotient.  On GPU tensors (mode 2) torch additionally converts the 0-dim divisor to
 * the result dtype before dividing: the division is by bf16(scale), the scale returned stays fp32 (observed on
 * torch 2.10 / ROCm: every element agrees with this reading, 1.7 % disagree with the fp32 divisor). */
static inline uint8_t quant_elem_tensor(float x, float scale)
{
    float q = wqo_bf16_to_f32(wqo_f32_to_bf16(x / scale));
    q = clamp_nanprop(q, -FP8_MAX, FP8_MAX);
    return wqo_f32_to_e4m3fn(q);
}

WQO_API int wqo_fp8_tensor_quant(const uint16_t *x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                                 int mode, uint8_t *y, float *s)
{
    if (M < 0 || N < 0 || (mode != 0 && mode != 2)) return 1;
    float amax = 0.0f;
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j)
            amax = max_nanprop(amax, fabsf(wqo_bf16_to_f32(x[i * sx_m + j * sx_n])));
    float scale = scale_torch(amax, mode);
    float divisor = mode == 2 ? wqo_bf16_to_f32(wqo_f32_to_bf16(scale)) : scale;
    s[0] = scale;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j)
            y[i * N + j] = quant_elem_tensor(wqo_bf16_to_f32(x[i * sx_m + j * sx_n]), divisor);
    return 0;
}

/* fp32 -> fp16 bits, round-to-nearest-even, subnormals kept, overflow to infinity, NaN stays NaN (quiet). */
WQO_API uint16_t wqo_f32_to_f16(float f)
{
    uint32_t u = f2u(f), sign = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));      /* NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);                               /* >= 2^16 (and inf): inf */
    if (a < 0x33000000u) return (uint16_t)sign;                                            /* < 2^-25: zero */
    if (a < 0x38800000u) {
        /* below 2^-14: subnormal result = RNE(|f| * 2^24), an integer of at most 11 bits (1024 = the smallest normal) */
        int e = (int)(a >> 23);                                /* biased exponent, 102..112 */
        uint32_t m = (a & 0x7FFFFFu) | 0x800000u;              /* 24-bit significand: |f| = m * 2^(e-150) */
        int shift = 126 - e;                                   /* |f| * 2^24 = m >> shift, shift in 14..24 */
        uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
    /* normal: drop 13 bits of the significand with RNE; the carry walks into the exponent (up to infinity) */
    uint32_t r = a - 0x38000000u;                              /* rebias 127 -> 15 */
    uint32_t q = r >> 13, rem = r & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
}

WQO_API void wqo_f32_to_f16_n(const float *x, uint16_t *y, int64_t n)
{ for (int64_t i = 0; i < n; ++i) y[i] = wqo_f32_to_f16(x[i]); }

/* value rounded to the weight dtype and widened again: what a torch op with that result dtype leaves behind */
static inline float round_to_dtype(float v, int dtype)
{
    if (dtype == 1) return v;
    if (dtype == 2) return wqo_f16_to_f32(wqo_f32_to_f16(v));
    return wqo_bf16_to_f32(wqo_f32_to_bf16(v));
}

/* tensor_fp8 for the other floating dtypes the reference function takes (convert_hf_to_fp8.py:86-91; dtype as in
 * load_any).  `weight / scale` has the weight's dtype (the 0-dim fp32 scale does not take part in type promotion): the
 * fp32 quotient is rounded to it - no second rounding for fp32 weights - and on GPU tensors (mode 2) the divisor is
 * converted to it first. */
WQO_API int wqo_fp8_tensor_quant_any(const void *x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                                     int mode, uint8_t *y, float *s)
{
    if (M < 0 || N < 0 || (mode != 0 && mode != 2) || dtype < 0 || dtype > 2) return 1;
    volatile float inv448 = 1.0f / FP8_MAX;
    float amax = 0.0f;
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j)
            amax = max_nanprop(amax, fabsf(load_any(x, dtype, i * sx_m + j * sx_n)));
    float a = amax;
    if (a == a && a < torch_floor(dtype)) a = torch_floor(dtype);
    float scale = mode == 2 ? a * inv448 : a / FP8_MAX;
    float divisor = mode == 2 ? round_to_dtype(scale, dtype) : scale;
    s[0] = scale;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float q = round_to_dtype(load_any(x, dtype, i * sx_m + j * sx_n) / divisor, dtype);
            y[i * N + j] = wqo_f32_to_e4m3fn(clamp_nanprop(q, -FP8_MAX, FP8_MAX));
        }
    return 0;
}

/* ------------------------------------------------------------------ FP8 dequant */

/* mode 0: y = bf16( f32(x) * s )                      tools/fp8_cast_bf16.py:25-28
 * mode 1: y = bf16( f32(bf16(x)) * f32(bf16(s)) )     hf_to_megatron/common.py:47-54
 *         (e4m3 -> bf16 is exact; the bf16*bf16 product is formed in fp32 and rounded once) */
WQO_API int wqo_fp8_block_dequant(const uint8_t *x, const float *s, int64_t M, int64_t N,
                                  int64_t block, int mode, uint16_t *y)
{
    if (M < 0 || N < 0 || block <= 0 || (mode != 0 && mode != 1)) return 1;
    int64_t kt = cdiv(N, block);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float sc = s[(i / block) * kt + (j / block)];
            if (mode == 1) sc = wqo_bf16_to_f32(wqo_f32_to_bf16(sc));
            y[i * N + j] = wqo_f32_to_bf16(wqo_e4m3fn_to_f32(x[i * N + j]) * sc);
        }
    return 0;
}

/* ------------------------------------------------------------------ INT4 fake quant */

static inline float ld_elem(const void *x, int dtype, int64_t off)
{
    if (dtype == 0) return wqo_bf16_to_f32(((const uint16_t *)x)[off]);
    if (dtype == 3) return (float)((const double *)x)[off];      /* static_cast<float>(x[...]), .cu:70 */
    return ((const float *)x)[off];
}
static inline void st_elem(void *p, int dtype, int64_t off, float v)
{
    if (dtype == 0) ((uint16_t *)p)[off] = wqo_f32_to_bf16(v);
    else if (dtype == 3) ((double *)p)[off] = (double)v;         /* static_cast<scalar_t>(val), .cu:92 */
    else ((float *)p)[off] = v;
}

/* Group = (bm x bn) block of the matrix; elements outside [M,N] read as 0.0f
 * (.cu:218-222).  sym: scale = fmaxf(amax * (1.0f/7.0f), 1e-5f); q = rintf(x/scale)
 * (.cu:233-234,254).  asym: scale = fmaxf((max-min) * (1.0f/15.0f), 1e-5f);
 * zero = clamp(-rintf(min/scale), 0, 15); q = rintf(x/scale) + zero (.cu:235-240,255-257).
 * fmaxf/fminf drop NaN operands exactly as the device functions do.  Outputs q [M,N],
 * scale/zero [cdiv(M,bm), cdiv(N,bn)], all contiguous, in the input dtype (0 = bf16, 1 = fp32, 3 = fp64: the
 * three types of AT_DISPATCH_FLOATING_TYPES_AND(BFloat16), .cu:352; every type is converted to fp32 on load).
 * Supported group shapes are the ones for which the reference kernels are well defined:
 * (1, 32k) and (bm, bn) with bn dividing 32 and bm*bn a multiple of 32. */
WQO_API int wqo_int4_fake_quant(const void *x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                                int64_t bm, int64_t bn, int sym, void *q, void *scale, void *zero)
{
    if (M < 0 || N < 0 || bm <= 0 || bn <= 0 || (dtype != 0 && dtype != 1 && dtype != 3)) return 1;
    if ((bm * bn) % 32 != 0) return 2;
    if (!((bm == 1 && bn % 32 == 0) || (32 % bn == 0))) return 3;
    const float SYM_CONS = 1.0f / 7.0f, ASYM_CONS = 1.0f / 15.0f;
    int64_t gm = cdiv(M, bm), gn = cdiv(N, bn);
#pragma omp parallel for schedule(static)
    for (int64_t bi = 0; bi < gm; ++bi)
        for (int64_t bj = 0; bj < gn; ++bj) {
            float vmax = -INFINITY, vmin = INFINITY;
            for (int64_t di = 0; di < bm; ++di)
                for (int64_t dj = 0; dj < bn; ++dj) {
                    int64_t i = bi * bm + di, j = bj * bn + dj;
                    float v = (i < M && j < N) ? ld_elem(x, dtype, i * sx_m + j * sx_n) : 0.0f;
                    if (sym) vmax = fmaxf(vmax, fabsf(v));
                    else { vmax = fmaxf(vmax, v); vmin = fminf(vmin, v); }
                }
            float sc, zp = 0.0f;
            if (sym) sc = fmaxf(vmax * SYM_CONS, 1e-5f);
            else {
                sc = fmaxf((vmax - vmin) * ASYM_CONS, 1e-5f);
                /* the device fmaxf orders -0 < +0, so a zero result is +0: "+ 0.0f" spells that out */
                zp = fminf(fmaxf(-rintf(vmin / sc), 0.0f), 15.0f) + 0.0f;
            }
            st_elem(scale, dtype, bi * gn + bj, sc);
            st_elem(zero, dtype, bi * gn + bj, zp);
            for (int64_t di = 0; di < bm; ++di)
                for (int64_t dj = 0; dj < bn; ++dj) {
                    int64_t i = bi * bm + di, j = bj * bn + dj;
                    if (i >= M || j >= N) continue;
                    float v = ld_elem(x, dtype, i * sx_m + j * sx_n);
                    v = sym ? rintf(v / sc) : rintf(v / sc) + zp;
                    st_elem(q, dtype, i * N + j, v);
                }
        }
    return 0;
}

/* ------------------------------------------------------------------ INT4 pack_layer */

static inline float round_half_even(float v) { return rintf(v); } /* default rounding mode */

/* Literal pack_layer chain on bf16 weights [M,N] contiguous, N % gs == 0, N % 8 == 0.
 *   (q, scale_b[, zero_b]) = fake_int4_quant(w, (1,gs), sym)        convert_hf_to_int4_direct.py:124
 *   sym:  d = bf16(q * scale_b)                                      :128-129
 *         r = bf16(d / scale_b) ; clamp to int8 range ; round ; int8 :108,85,146-151
 *         nib = uint8(q2 + 8)                                        :49-50
 *   asym: d = bf16(bf16(q - zero_b) * scale_b)                       :130-131
 *         r = bf16(d / scale_b) ; r = bf16(r + zero_b) ; clamp to uint8 range ; round ; uint8
 *         packed_zp[c, g] (zero points transposed, 8 row-consecutive zero points per int32,
 *         nibble order 0,4,1,5,2,6,3,7)                              :134-141
 *   packed[i, c] = sum_j int32(nib[i, 8c+j]) << 4j  (int32 wrap-around)  :68-70
 * packed: int32 [M, N/8]; scale_out: bf16 [M, N/gs]; packed_zp: int32 [N/gs, M/8] or NULL. */
WQO_API int wqo_int4_pack_layer(const uint16_t *w, int64_t M, int64_t N, int64_t gs, int sym,
                                int32_t *packed, uint16_t *scale_out, int32_t *packed_zp)
{
    if (M < 0 || N < 0 || gs <= 0 || N % gs != 0 || N % 8 != 0 || gs % 32 != 0) return 1;
    if (!sym && (M % 8 != 0 || !packed_zp)) return 1;
    int64_t G = N / gs;
    size_t ne = (size_t)(M * N), ng = (size_t)(M * G);
    uint16_t *q = (uint16_t *)malloc((ne ? ne : 1) * 2);
    uint16_t *zb = (uint16_t *)malloc((ng ? ng : 1) * 2);
    uint8_t *nib = (uint8_t *)malloc(ne ? ne : 1);
    if (!q || !zb || !nib) { free(q); free(zb); free(nib); return 4; }
    int rc = wqo_int4_fake_quant(w, 0, M, N, N, 1, 1, gs, sym, q, scale_out, zb);
    if (rc) { free(q); free(zb); free(nib); return rc; }
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float sb = wqo_bf16_to_f32(scale_out[i * G + j / gs]);
            float qv = wqo_bf16_to_f32(q[i * N + j]);
            if (sym) {
                float d = wqo_bf16_to_f32(wqo_f32_to_bf16(qv * sb));
                float r = wqo_bf16_to_f32(wqo_f32_to_bf16(d / sb));
                r = clamp_nanprop(r, -128.0f, 127.0f);
                int q2 = (int)round_half_even(r);
                nib[i * N + j] = (uint8_t)(q2 + 8);
            } else {
                float z = wqo_bf16_to_f32(zb[i * G + j / gs]);
                float t = wqo_bf16_to_f32(wqo_f32_to_bf16(qv - z));
                float d = wqo_bf16_to_f32(wqo_f32_to_bf16(t * sb));
                float r = wqo_bf16_to_f32(wqo_f32_to_bf16(d / sb));
                r = wqo_bf16_to_f32(wqo_f32_to_bf16(r + z));
                r = clamp_nanprop(r, 0.0f, 255.0f);
                nib[i * N + j] = (uint8_t)(int)round_half_even(r);
            }
        }
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t c = 0; c < N / 8; ++c) {
            uint32_t acc = 0;
            for (int j = 0; j < 8; ++j) acc += (uint32_t)nib[i * N + 8 * c + j] << (4 * j);
            packed[i * (N / 8) + c] = (int32_t)acc;
        }
    if (!sym) {
        static const int order[8] = {0, 4, 1, 5, 2, 6, 3, 7};
        for (int64_t g = 0; g < G; ++g)
            for (int64_t c = 0; c < M / 8; ++c) {
                uint32_t acc = 0;
                for (int j = 0; j < 8; ++j) {
                    int32_t z = (int32_t)wqo_bf16_to_f32(zb[(8 * c + j) * G + g]);
                    acc += (uint32_t)z << (4 * order[j]);
                }
                packed_zp[g * (M / 8) + c] = (int32_t)acc;
            }
    }
    free(q); free(zb); free(nib);
    return 0;
}

/* ------------------------------------------------------------------ INT4 -> bf16, QAT forward */

/* y[i,j] = bf16( f32(nibble(i,j) - 8) * f32(scale[i, j/gs]) ); nibble j of word c at bits [4j,4j+4).
 * tools/convert_k2_thinking_int4_to_bf16.py:55-84 (_dequantize_tensor); the unpacking there is
 * compressed_tensors.unpack_from_int32 (third party, not vendored: PARITY UNPINNED against it; the bit layout is
 * the inverse of pack_to_int32, tools/convert_hf_to_int4_direct.py:32-75, which is pinned). */
WQO_API int wqo_int4_dequant(const int32_t *packed, const uint16_t *scale, int64_t M, int64_t N, int64_t gs,
                             uint16_t *y)
{
    if (M < 0 || N < 0 || gs <= 0 || N % gs != 0 || N % 8 != 0) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            uint32_t w = (uint32_t)packed[i * (N / 8) + j / 8];
            int q = (int)((w >> (4 * (j % 8))) & 0xFu) - 8;
            float s = wqo_bf16_to_f32(scale[i * (N / gs) + j / gs]);
            y[i * N + j] = wqo_f32_to_bf16((float)q * s);
        }
    return 0;
}

/* The same function for the other inputs the reference accepts: scale stored as bf16 (0), fp32 (1) or fp16 (2) and
 * converted with .to(float32) (:69); group_size <= 0 (pass gs = 1: one scale per element, :74-75); N not a multiple
 * of 8 (packed is [M, ceil(N/8)], the tail of a row's last word is cut).  (float)q * s is one fp32 rounding, the
 * conversion to bf16 a second one. */
WQO_API int wqo_int4_dequant_any(const int32_t *packed, const void *scale, int scale_dtype, int64_t M, int64_t N,
                                 int64_t gs, uint16_t *y)
{
    if (M < 0 || N < 0 || gs <= 0 || N % gs != 0 || scale_dtype < 0 || scale_dtype > 2) return 1;
    int64_t wpr = (N + 7) / 8;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            uint32_t w = (uint32_t)packed[i * wpr + j / 8];
            int q = (int)((w >> (4 * (j % 8))) & 0xFu) - 8;
            float s = load_any(scale, scale_dtype, i * (N / gs) + j / gs);
            y[i * N + j] = wqo_f32_to_bf16((float)q * s);
        }
    return 0;
}

/* Forward of the INT4 QAT straight-through estimator, docker/patch/latest/megatron.patch:212-246:
 * s = clamp(f32(amax_bf16) / 7, min=1e-5); y = bf16( clamp(round(f32(x) / s), -7, 7) * s ).  bf16 [M,N], N % gs == 0.
 * div7 = 0: `/ 7` is a division (torch on CPU tensors); 1: a multiplication by RN(1/7) (torch on GPU tensors, the
 * only place this function runs in the reference). */
WQO_API int wqo_int4_fake_ste(const uint16_t *x, int64_t M, int64_t N, int64_t gs, int div7, uint16_t *y)
{
    if (M < 0 || N < 0 || gs <= 0 || N % gs != 0 || (div7 != 0 && div7 != 1)) return 1;
    volatile float inv7 = 1.0f / 7.0f;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; ++i)
        for (int64_t g = 0; g < N / gs; ++g) {
            float amax = 0.0f;
            for (int64_t k = 0; k < gs; ++k) amax = max_nanprop(amax, fabsf(wqo_bf16_to_f32(x[i * N + g * gs + k])));
            float s = div7 ? amax * inv7 : amax / 7.0f;
            if (s == s && s < 1e-5f) s = 1e-5f;
            for (int64_t k = 0; k < gs; ++k) {
                float q = rintf(wqo_bf16_to_f32(x[i * N + g * gs + k]) / s);
                q = clamp_nanprop(q, -7.0f, 7.0f);
                y[i * N + g * gs + k] = wqo_f32_to_bf16(q * s);
            }
        }
    return 0;
}

/* Number of OpenMP threads the loops above will use (1 when built without OpenMP). */
#ifdef _OPENMP
#include <omp.h>
WQO_API int wqo_num_threads(void) { return omp_get_max_threads(); }
WQO_API void wqo_set_num_threads(int n) { omp_set_num_threads(n); }
#else
WQO_API int wqo_num_threads(void) { return 1; }
WQO_API void wqo_set_num_threads(int n) { (void)n; }
#endif
