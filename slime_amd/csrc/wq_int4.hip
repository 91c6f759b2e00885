// Group-wise INT4 quantisation for gfx950.
//
// int4_pack_kernel: fused symmetric quantise + nibble pack for bf16 rows.  A group of G = 8*L
// elements (L = 4, 8 or 16 lanes; G = 32, 64, 128) is owned by L adjacent lanes: one 16-byte load
// per lane brings the whole group into registers, the amax is an integer max over bf16 magnitude
// bits reduced with DPP inside the 16-lane row, the scale is max(amax * (1/7), 1e-5) in fp32, every
// element is divided exactly (reciprocal + two FMA), rounded half-to-even by a magic-constant add
// and the eight 4-bit codes of the lane are assembled into the one int32 the lane stores.  One HBM
// read of x, one write of the packed words, one bf16 scale per group.  The dequantise /
// re-quantise chain that the reference runs between its fake-quant kernel and the packing is the
// identity on the integer codes for every reachable (code, bf16 scale) pair, so it is not executed.
//
// int4_fake_quant_kernel: the general "fake quant" form (codes, scale and zero point written in the
// input dtype) for any supported group shape, strides, bf16 or fp32, symmetric or asymmetric.

#include "wq_common.h"

namespace wq {

constexpr int kGroupsPerWg = WQ_INT4_GROUPS_PER_WG;
constexpr int kPackItemsPerXcdRun = 32;  // 32 work items = 512 KiB of contiguous input per XCD run
constexpr unsigned kPackOccupancyPadBytes = 0;
// 16-byte loads in flight per lane (a work item of 128-element groups has four).  With the byte-gathering pack function:
// 1: 78.3, 2: 79.4, 3: 80.1, 4: 80.6 % of HBM peak on 16 layers of experts, 79.0 -> 79.3 on all 48; any residency cap
// below 7 workgroups per CU costs 6-15 points.
constexpr int kPackWindow = 4;

struct Int4PackArgs {
    wq_int4_pack_desc d;
    const wq_int4_pack_desc* descs;
    const int64_t* work_start;
    int32_t n_desc;
    char* out_base;       // per-item form only: when set, packed and scale of every descriptor are byte offsets from here
};

template <int L>
__device__ __forceinline__ uint32_t lanes_max_u32(uint32_t v)
{
    v = max(v, dpp_u32<0xB1>(v));
    v = max(v, dpp_u32<0x4E>(v));
    if (L >= 8) v = max(v, dpp_u32<0x141>(v));
    if (L >= 16) v = max(v, dpp_u32<0x140>(v));
    return v;
}

__device__ __forceinline__ void unpack8(const u32x4& v, float (&x)[8])
{
    x[0] = bf16lo(v.x); x[1] = bf16hi(v.x); x[2] = bf16lo(v.y); x[3] = bf16hi(v.y);
    x[4] = bf16lo(v.z); x[5] = bf16hi(v.z); x[6] = bf16lo(v.w); x[7] = bf16hi(v.w);
}

// max |x| over the lane's eight values; fmaxf drops NaN operands exactly as the reference kernel's does
__device__ __forceinline__ float absmax8(const float (&x)[8])
{
    float m = fmaxf(fabsf(x[0]), fabsf(x[1]));
    m = fmaxf(fmaxf(m, fabsf(x[2])), fabsf(x[3]));
    m = fmaxf(fmaxf(m, fabsf(x[4])), fabsf(x[5]));
    m = fmaxf(fmaxf(m, fabsf(x[6])), fabsf(x[7]));
    return m;
}

typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
// fp32 -> bf16 bits, RNE, by v_cvt_pk_bf16_f32 (identical to the software rounding for all non-NaN inputs)
__device__ __forceinline__ uint32_t bf16_bits_hw(float f)
{
    f32x2_t v = {f, 0.0f};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t)) & 0xFFFFu;
}

// Scales at or above 2^121 (bf16 bits 0x7C00): the reference's dequantise / re-quantise chain is no
// longer the identity there - bf16(7 * scale) can overflow to infinity, which its clamp turns into the
// code 127 and its packing sum then carries into the neighbouring nibbles.  Such groups (weights of
// magnitude ~1e37) take the literal chain so that even this corner packs the words the reference packs.
constexpr uint32_t kLiteralChainScaleBits = 0x7C00u;

__device__ __forceinline__ float bf16_round(float f) { return u2f(f32_to_bf16_bits(f) << 16); }

__device__ __forceinline__ uint32_t code_literal(float x, float scale, float sb)
{
    const float q = __builtin_rintf(x / scale);
    const float d = bf16_round(q * sb);
    float r = bf16_round(d / sb);
    if (r == r) r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (uint32_t)((int)__builtin_rintf(r) + 8) & 0xFFu;  // int8 + 8, reinterpreted as uint8
}

__device__ __forceinline__ uint32_t pack8_literal(const float (&x)[8], float scale, float sb)
{
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) w += code_literal(x[j], scale, sb) << (4 * j);
    return w;
}

// Writes n_words words collected in LDS to dst (4-byte aligned, not on a 128-byte line) as whole lines: single words up to
// the first line boundary and after the last 16-byte piece, 16-byte stores in between - a wavefront per KiB, starting on a
// line.  All threads of the workgroup call it after a barrier.
__device__ __forceinline__ void store_words_by_lines(char* dst, const uint32_t* stage, int n_words)
{
    const int head = min((int)(((128u - ((uintptr_t)dst & 127u)) & 127u) >> 2), n_words);   // words before the first line
    const int pieces = (n_words - head) >> 2;                                               // whole 16-byte pieces from there
    const int t = threadIdx.x;
    if (t < head) stg_nt<uint32_t>(dst + (uint32_t)(t * 4), stage[t]);
    for (int p = t; p < pieces; p += 256) {
        const int w0 = head + 4 * p;
        const u32x4 o = {stage[w0], stage[w0 + 1], stage[w0 + 2], stage[w0 + 3]};
        stg_nt<u32x4>(dst + (uint32_t)(w0 * 4), o);
    }
    const int tail = head + 4 * pieces + t;
    if (tail < n_words) stg_nt<uint32_t>(dst + (uint32_t)(tail * 4), stage[tail]);
}

// Contiguous tensors only: group g of the tensor starts at x + g*G, its packed words at
// packed + g*L, its scale at scale[g].
// GROUPED: 0 = one tensor in the kernel arguments, 1 = descriptor array + prefix sums (the owner of a work item is
// searched), 2 = one pre-resolved descriptor per work item (a single scalar load, no search)
template <int L, int GROUPED>
__global__ __launch_bounds__(256) void int4_pack_kernel(const Int4PackArgs a, const int64_t total_work)
{
    constexpr int CL = 256 / L;              // groups per step of the workgroup
    constexpr int STEPS = kGroupsPerWg / CL; // kGroupsPerWg = 64: 1 (L=4), 2 (L=8), 4 (L=16)
    static_assert(STEPS >= 1, "a work item must cover at least one step of the workgroup");
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_work) return;
    const int64_t item = xcd_chunked_item(slot, total_work, kPackItemsPerXcdRun);
    wq_int4_pack_desc d;
    int64_t local = item;
    if (GROUPED == 1) {
        const int di = find_owner(a.work_start, a.n_desc, item, total_work);
        d = a.descs[di];
        local = item - a.work_start[di];
    } else if (GROUPED == 2) {
        d = a.descs[item];
        local = 0;
        if (a.out_base) {
            d.packed = (int32_t*)(a.out_base + (uintptr_t)d.packed);
            d.scale = a.out_base + (uintptr_t)d.scale;
        }
        if (d.n_groups < 0) {                      // pass-through item: -n_groups bytes from x to packed
            copy_item(d.x, d.packed, (int)-d.n_groups);
            return;
        }
    } else {
        d = a.d;
    }
    const int cl = threadIdx.x / L, ll = threadIdx.x % L;
    // Workgroup-uniform base of the item (scalar registers) and 32-bit per-lane byte offsets from it: an item is at
    // most 64 groups = 16 KiB of input.
    const int64_t base = local * kGroupsPerWg;
    const int rem = (int)min((int64_t)kGroupsPerWg, d.n_groups - base);       // groups of the item, >= 1
    const char* xb = (const char*)d.x + base * (16 * L);
    char* pb = (char*)d.packed + base * (4 * L);
    char* sb = (char*)d.scale + base * 2;
    // Where the item's words do not start on a 128-byte line - a bucket packs its tensors back to back, and every INT4
    // weight is followed by its 8-byte weight_shape - each wavefront's 256-byte store would begin and end in the middle of
    // a line, and such streams lose 7 points of bandwidth on this part (81 -> 74 % of HBM peak on 16 layers of experts).
    // Those items collect their words in LDS and write them out as whole lines: 16-byte stores, a wavefront per KiB
    // starting on a line boundary, single words only before the first and after the last boundary (80 %).
    __shared__ uint32_t stage[kGroupsPerWg * L];
    const bool staged = GROUPED == 2 && ((uintptr_t)pb & 127u) != 0;          // uniform per workgroup

    // Rolling window: at most kPackWindow 16-byte loads per lane are in flight; the load of step i + window
    // is issued just before step i is processed (with the window as long as the item, all of them are issued up front).
    // Out-of-range groups re-read the item's last group instead of branching around the load (a
    // predicated load makes the compiler wait for earlier loads before issuing the next one).
    u32x4 v[STEPS];
    auto issue = [&](int i) {
        const int g = min(cl + i * CL, rem - 1);
        v[i] = ldg_nt<u32x4>(xb + (uint32_t)(g * (16 * L) + ll * 16));
    };
#pragma unroll
    for (int i = 0; i < kPackWindow && i < STEPS; ++i) issue(i);
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        if (i + kPackWindow < STEPS) issue(i + kPackWindow);
        __builtin_amdgcn_sched_barrier(0);
        const int g = cl + i * CL;
        float xs[8];
        unpack8(v[i], xs);
        const float scale = int4_scale_sym(lanes_max_f32<L>(absmax8(xs)));
        uint32_t w = pack8_sym_bytes(xs, scale, rcp_refined(scale));
        const uint32_t sb_bits = bf16_bits_hw(scale);
        if (sb_bits >= kLiteralChainScaleBits) w = pack8_literal(xs, scale, u2f(sb_bits << 16));
        if (g < rem) {
            if (staged) stage[g * L + ll] = w;
            else stg_nt<uint32_t>(pb + (uint32_t)((g * L + ll) * 4), w);
            if (ll == 0) stg<uint16_t>(sb + (uint32_t)(g * 2), (uint16_t)sb_bits);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (staged) {
        __syncthreads();
        store_words_by_lines(pb, stage, rem * L);
    }
}

// Any group size that is a multiple of 32, strided rows, unaligned pointers.  One 16-lane row per
// group, two passes over the group.
__global__ __launch_bounds__(256) void int4_pack_generic_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t N,
                                                               int64_t sx_m, int group, uint32_t* __restrict__ packed,
                                                               uint16_t* __restrict__ scale_out)
{
    const int64_t G = N / group;
    const int64_t total = M * G;
    const int64_t g = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * 16 + (threadIdx.x >> 4);
    const int ll = threadIdx.x & 15;
    const bool live = g < total;
    const int64_t row = live ? g / G : 0, gi = live ? g - row * G : 0;
    const uint16_t* xg = x + row * sx_m + gi * group;
    uint32_t m = 0;
    if (live)
        for (int e = ll; e < group; e += 16) m = max(m, (uint32_t)xg[e] & 0x7FFFu);
    m = lanes_max_u32<16>(m);
    const float scale = int4_scale_sym(u2f(m << 16));
    if (!live) return;
    const uint32_t sb_bits = f32_to_bf16_bits(scale);
    if (ll == 0) scale_out[g] = (uint16_t)sb_bits;
    const bool literal = sb_bits >= kLiteralChainScaleBits;
    const float sb = u2f(sb_bits << 16);
    uint32_t* pg = packed + row * (N / 8) + gi * (group / 8);
    for (int wi = ll; wi < group / 8; wi += 16) {
        uint32_t w = 0;
        for (int j = 0; j < 8; ++j) {
            const float xv = u2f((uint32_t)xg[wi * 8 + j] << 16);
            w += (literal ? code_literal(xv, scale, sb) : nibble_of(xv / scale)) << (4 * j);
        }
        pg[wi] = w;
    }
}

// ---- fake quant (codes in the input dtype) -------------------------------------------------------

template <typename T> __device__ __forceinline__ float ld_as_f32(const T* p, int64_t off);
template <> __device__ __forceinline__ float ld_as_f32<uint16_t>(const uint16_t* p, int64_t off)
{ return u2f((uint32_t)p[off] << 16); }
template <> __device__ __forceinline__ float ld_as_f32<float>(const float* p, int64_t off) { return p[off]; }
template <> __device__ __forceinline__ float ld_as_f32<double>(const double* p, int64_t off) { return (float)p[off]; }
template <typename T> __device__ __forceinline__ void st_from_f32(T* p, int64_t off, float v);
template <> __device__ __forceinline__ void st_from_f32<uint16_t>(uint16_t* p, int64_t off, float v)
{ p[off] = (uint16_t)f32_to_bf16_bits(v); }
template <> __device__ __forceinline__ void st_from_f32<float>(float* p, int64_t off, float v) { p[off] = v; }
template <> __device__ __forceinline__ void st_from_f32<double>(double* p, int64_t off, float v) { p[off] = (double)v; }

__device__ __forceinline__ float wave64_max_f32(float v)
{
    v = row16_max_f32(v);
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}
__device__ __forceinline__ float wave64_min_f32(float v)
{
    v = row16_min_f32(v);
    v = fminf(v, __shfl_xor(v, 16));
    v = fminf(v, __shfl_xor(v, 32));
    return v;
}

// One wavefront per (bm x bn) group.
template <typename T>
__global__ __launch_bounds__(256) void int4_fake_quant_kernel(const T* __restrict__ x, int64_t M, int64_t N,
                                                             int64_t sx_m, int64_t sx_n, int bm, int bn, int sym,
                                                             T* __restrict__ q, T* __restrict__ scale_out,
                                                             T* __restrict__ zero_out)
{
    const int64_t gn = (N + bn - 1) / bn, gm = (M + bm - 1) / bm;
    const int64_t grp = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * 4 + (threadIdx.x >> 6);
    if (grp >= gm * gn) return;  // uniform per wavefront
    const int lane = threadIdx.x & 63;
    const int64_t bi = grp / gn, bj = grp - bi * gn;
    const int64_t r0 = bi * bm, c0 = bj * bn;
    const int n = bm * bn;
    float vmax = -INFINITY, vmin = INFINITY;
    for (int e = lane; e < n; e += 64) {
        const int di = e / bn, dj = e - di * bn;
        const int64_t i = r0 + di, j = c0 + dj;
        const float v = (i < M && j < N) ? ld_as_f32<T>(x, i * sx_m + j * sx_n) : 0.0f;
        if (sym) vmax = fmaxf(vmax, fabsf(v));
        else { vmax = fmaxf(vmax, v); vmin = fminf(vmin, v); }
    }
    vmax = wave64_max_f32(vmax);
    float scale, zero = 0.0f;
    if (sym) {
        scale = fmaxf(vmax * (1.0f / 7.0f), 1e-5f);
    } else {
        vmin = wave64_min_f32(vmin);
        scale = fmaxf((vmax - vmin) * (1.0f / 15.0f), 1e-5f);
        // "+ 0.0f": a zero result is +0 whatever operand order the max instruction prefers for -0 vs +0
        zero = fminf(fmaxf(-__builtin_rintf(vmin / scale), 0.0f), 15.0f) + 0.0f;
    }
    if (lane == 0) {
        st_from_f32<T>(scale_out, grp, scale);
        st_from_f32<T>(zero_out, grp, zero);
    }
    for (int e = lane; e < n; e += 64) {
        const int di = e / bn, dj = e - di * bn;
        const int64_t i = r0 + di, j = c0 + dj;
        if (i < M && j < N) {
            float v = __builtin_rintf(ld_as_f32<T>(x, i * sx_m + j * sx_n) / scale);
            if (!sym) v += zero;  // the symmetric branch must not add: -0.0f + 0.0f would lose the sign
            st_from_f32<T>(q, i * N + j, v);
        }
    }
}

// Fast form of the kernel above for the layout the callers use: bf16, contiguous rows, (1 x 32 | 64 | 128) groups
// that tile the row.  A group is owned by L adjacent lanes (one 16-byte load, one 16-byte store per lane).  The
// symmetric branch with a finite amax uses the division-free element function of the pack kernel (same scale rule,
// same (amax, x) domain, same exhaustive check); codes carry the sign of x, zero included, as rintf(x / scale) does.
constexpr int kFakeGroupsPerWg = 64;
constexpr int kFakeItemsPerXcdRun = 32;
// resident workgroups per CU (fake quant of a [151936, 2560] tensor, sym / asym, % of HBM peak): 8: 77.7 / 76.1, 7: 78.0 / 76.2,
// 6: 77.6 / 76.2 (used), 5: 77.9 / 75.0, 4: 76.3-77.4 / 71.5-72.4, 3: 73.2 / 68.9; a rolling window of loads gains nothing
constexpr unsigned kFakeOccupancyPadBytes = 24 * 1024;
constexpr int kFakeQWindow = 4;           // 16-byte loads in flight per lane in the fake-quant kernel (4 = a whole item)

__device__ __forceinline__ uint32_t pack2_bf16_hw(float a, float b)
{
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// CONTIG: rows are back to back (row stride = row length), so a group's address is its flat index times the group
// size; otherwise (row, group-in-row) come from a 32-bit division - the host checks that the group count fits.
template <int L, bool SYM, bool CONTIG>
__global__ __launch_bounds__(256) void int4_fake_quant_vec_kernel(const uint16_t* __restrict__ x, int64_t sx_m,
                                                                 int groups_per_row, uint16_t* __restrict__ q,
                                                                 uint16_t* __restrict__ scale_out,
                                                                 uint16_t* __restrict__ zero_out, int64_t n_groups,
                                                                 int64_t total_items)
{
    constexpr int CL = 256 / L;
    constexpr int STEPS = kFakeGroupsPerWg / CL;
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_items) return;
    const int64_t item = xcd_chunked_item(slot, total_items, kFakeItemsPerXcdRun);
    const int cl = threadIdx.x / L, ll = threadIdx.x % L;
    const int64_t g0 = item * kFakeGroupsPerWg + cl;
    u32x4 v[STEPS];
    auto issue = [&](int i) {
        const int64_t g = min(g0 + i * CL, n_groups - 1);
        if (CONTIG) {
            v[i] = ldg_nt<u32x4>(x + g * (8 * L) + ll * 8);
        } else {
            const uint32_t row = (uint32_t)g / (uint32_t)groups_per_row, gc = (uint32_t)g - row * (uint32_t)groups_per_row;
            v[i] = ldg_nt<u32x4>(x + (int64_t)row * sx_m + gc * (8 * L) + ll * 8);
        }
    };
#pragma unroll
    for (int i = 0; i < kFakeQWindow && i < STEPS; ++i) issue(i);
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        if (kFakeQWindow < STEPS) {
            asm volatile("" :: "v"(v[i].x));
            if (i + kFakeQWindow < STEPS) issue(i + kFakeQWindow);
            __builtin_amdgcn_sched_barrier(0);
        }
        const int64_t g = g0 + i * CL;
        float xs[8];
        unpack8(v[i], xs);
        float o[8];
        float scale, zero = 0.0f;
        bool restore_sign = false;
        if (SYM) {
            const float amax = lanes_max_f32<L>(absmax8(xs));
            scale = int4_scale_sym(amax);
            if (amax < INFINITY) {
                const float r = rcp_refined(scale);
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = (div_by_scale(xs[j], scale, r) + 12582912.0f) - 12582912.0f;
                restore_sign = true;
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = __builtin_rintf(xs[j] / scale);
            }
        } else {
            float vmax = fmaxf(fmaxf(fmaxf(xs[0], xs[1]), fmaxf(xs[2], xs[3])), fmaxf(fmaxf(xs[4], xs[5]), fmaxf(xs[6], xs[7])));
            float vmin = fminf(fminf(fminf(xs[0], xs[1]), fminf(xs[2], xs[3])), fminf(fminf(xs[4], xs[5]), fminf(xs[6], xs[7])));
            vmax = lanes_max_f32<L>(vmax);
            vmin = lanes_min_f32<L>(vmin);
            scale = fmaxf((vmax - vmin) * (1.0f / 15.0f), 1e-5f);
            // x / scale by the correctly rounded reciprocal (one division per lane) and the two-FMA correction, which
            // yields the correctly rounded quotient for any fp32 divisor as long as the reciprocal is a normal number and
            // nothing overflows (Markstein's theorem); groups holding huge or non-finite values divide element by element.
            // The zero point's min / scale is one more such quotient.
            const float r = 1.0f / scale;
            const bool safe = scale < 0x1p100f && fmaxf(fabsf(vmax), fabsf(vmin)) * r < 0x1p60f;
            if (__builtin_amdgcn_ballot_w64(!safe) == 0) {
                zero = fminf(fmaxf(-__builtin_rintf(div_by_scale(vmin, scale, r)), 0.0f), 15.0f) + 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = __builtin_rintf(div_by_scale(xs[j], scale, r)) + zero;
            } else {
                zero = fminf(fmaxf(-__builtin_rintf(vmin / scale), 0.0f), 15.0f) + 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = __builtin_rintf(xs[j] / scale) + zero;
            }
        }
        if (g < n_groups) {
            u32x4 r = {pack2_bf16_hw(o[0], o[1]), pack2_bf16_hw(o[2], o[3]), pack2_bf16_hw(o[4], o[5]),
                       pack2_bf16_hw(o[6], o[7])};
            if (restore_sign) r = (r & 0x7FFF7FFFu) | (v[i] & 0x80008000u);
            stg_nt_sc1<u32x4>(q + g * (8 * L) + ll * 8, r);
            if (ll == 0) {
                stg<uint16_t>(scale_out + g, (uint16_t)f32_to_bf16_bits(scale));
                stg<uint16_t>(zero_out + g, (uint16_t)f32_to_bf16_bits(zero));
            }
        }
    }
}

// Asymmetric quantise + pack for the same layout: codes rintf(x / scale) + zero, then what the reference's
// pack_layer does to them before packing - dequantise to bf16, re-quantise, clamp to the uint8 range - and the
// un-masked shift-add of pack_to_int32 (a code above 15 spills into the neighbouring nibbles there, and so it
// does here).  That chain is the identity on every code in [0, 17] for every zero point and every bf16 scale below
// 2^121 (checked by exhaustion in the CPU tests); lanes whose eight codes are all in that range skip it, the others
// run it literally.
__device__ __forceinline__ uint32_t code_literal_asym(float q, float z, float sb)
{
    const float qb = bf16_round(q);            // the fake-quant kernel stores the code as bf16
    const float t = bf16_round(qb - z);
    const float d = bf16_round(t * sb);
    float r = bf16_round(d / sb);
    r = bf16_round(r + z);
    if (r == r) r = fminf(fmaxf(r, 0.0f), 255.0f);
    return (uint32_t)(int)__builtin_rintf(r);
}

// ITEMS: one pre-resolved descriptor per work item (many contiguous tensors in one launch), pointing at the item's
// first group; rows are then contiguous and groups are addressed flat.
template <int L, bool ITEMS>
__global__ __launch_bounds__(256) void int4_pack_asym_kernel(const uint16_t* __restrict__ x, int64_t sx_m,
                                                            int groups_per_row, uint32_t* __restrict__ packed,
                                                            uint16_t* __restrict__ scale_out,
                                                            uint16_t* __restrict__ zero_out, int64_t n_groups,
                                                            int64_t total_items,
                                                            const wq_int4_pack_asym_item* __restrict__ items,
                                                            char* out_base, char* zero_base)
{
    constexpr int CL = 256 / L;
    constexpr int STEPS = kFakeGroupsPerWg / CL;
    const int64_t slot = (int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
    if (slot >= total_items) return;
    const int64_t item = xcd_chunked_item(slot, total_items, kFakeItemsPerXcdRun);
    const int cl = threadIdx.x / L, ll = threadIdx.x % L;
    int64_t g0 = item * kFakeGroupsPerWg + cl;
    if (ITEMS) {
        const wq_int4_pack_asym_item it = items[item];
        x = (const uint16_t*)it.x;
        packed = (uint32_t*)(out_base + (uintptr_t)it.packed);        // bases are null for absolute addresses
        scale_out = (uint16_t*)(out_base + (uintptr_t)it.scale);
        zero_out = (uint16_t*)(zero_base + (uintptr_t)it.zero);
        n_groups = it.n_groups;
        g0 = cl;
        if (n_groups < 0) {                      // pass-through item: -n_groups bytes from x to packed
            copy_item(x, packed, (int)-n_groups);
            return;
        }
    }
    // items whose words do not start on a 128-byte line: collected in LDS, written as whole lines (see int4_pack_kernel)
    __shared__ uint32_t stage[ITEMS ? kFakeGroupsPerWg * L : 1];
    const bool staged = ITEMS && ((uintptr_t)packed & 127u) != 0;          // uniform per workgroup
    u32x4 v[STEPS];
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        const int64_t g = min(g0 + i * CL, n_groups - 1);
        if (ITEMS) {
            v[i] = ldg_nt<u32x4>(x + g * (8 * L) + ll * 8);
        } else if (sx_m == (int64_t)groups_per_row * (8 * L)) {     // contiguous rows (uniform branch)
            v[i] = ldg_nt<u32x4>(x + g * (8 * L) + ll * 8);
        } else {
            const uint32_t row = (uint32_t)g / (uint32_t)groups_per_row, gc = (uint32_t)g - row * (uint32_t)groups_per_row;
            v[i] = ldg_nt<u32x4>(x + (int64_t)row * sx_m + gc * (8 * L) + ll * 8);
        }
    }
#pragma unroll
    for (int i = 0; i < STEPS; ++i) {
        const int64_t g = g0 + i * CL;
        float xs[8];
        unpack8(v[i], xs);
        float vmax = fmaxf(fmaxf(fmaxf(xs[0], xs[1]), fmaxf(xs[2], xs[3])), fmaxf(fmaxf(xs[4], xs[5]), fmaxf(xs[6], xs[7])));
        float vmin = fminf(fminf(fminf(xs[0], xs[1]), fminf(xs[2], xs[3])), fminf(fminf(xs[4], xs[5]), fminf(xs[6], xs[7])));
        vmax = lanes_max_f32<L>(vmax);
        vmin = lanes_min_f32<L>(vmin);
        const float scale = fmaxf((vmax - vmin) * (1.0f / 15.0f), 1e-5f);
        const uint32_t sb_bits = f32_to_bf16_bits(scale);
        float q[8], zero;
        // x / scale (and min / scale of the zero point) by the correctly rounded reciprocal and the two-FMA correction
        // (see int4_fake_quant_vec_kernel)
        const float r = 1.0f / scale;
        const bool safe = scale < 0x1p100f && fmaxf(fabsf(vmax), fabsf(vmin)) * r < 0x1p60f;
        if (__builtin_amdgcn_ballot_w64(!safe) == 0) {
            zero = fminf(fmaxf(-__builtin_rintf(div_by_scale(vmin, scale, r)), 0.0f), 15.0f) + 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = __builtin_rintf(div_by_scale(xs[j], scale, r)) + zero;
        } else {
            zero = fminf(fmaxf(-__builtin_rintf(vmin / scale), 0.0f), 15.0f) + 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = __builtin_rintf(xs[j] / scale) + zero;
        }
        bool plain = sb_bits < kLiteralChainScaleBits;
#pragma unroll
        for (int j = 0; j < 8; ++j) plain = plain && q[j] >= 0.0f && q[j] <= 17.0f;
        uint32_t word = 0;
        if (plain) {
#pragma unroll
            for (int j = 0; j < 8; ++j) word += (uint32_t)q[j] << (4 * j);
        } else {
            const float sb = u2f(sb_bits << 16);
#pragma unroll
            for (int j = 0; j < 8; ++j) word += code_literal_asym(q[j], zero, sb) << (4 * j);
        }
        if (g < n_groups) {
            if (staged) stage[(int)g * L + ll] = word;
            else stg_nt<uint32_t>(packed + g * L + ll, word);
            if (ll == 0) {
                stg<uint16_t>(scale_out + g, (uint16_t)sb_bits);
                stg<uint16_t>(zero_out + g, (uint16_t)f32_to_bf16_bits(zero));
            }
        }
    }
    if (staged) {
        __syncthreads();
        store_words_by_lines((char*)packed, stage, (int)min(n_groups, (int64_t)kFakeGroupsPerWg) * L);
    }
}

template <bool SYM>
static bool launch_fake_vec(const uint16_t* x, int64_t M, int64_t N, int64_t sx_m, int bn, uint16_t* q, uint16_t* sc,
                            uint16_t* zp, hipStream_t st)
{
    const int64_t n_groups = M * (N / bn);
    const int64_t items = cdiv64(n_groups, kFakeGroupsPerWg);
    const dim3 g = grid_for_items(items);
    const int gpr = (int)(N / bn);
    if (sx_m == N) {
        if (bn == 32) int4_fake_quant_vec_kernel<4, SYM, true><<<g, 256, kFakeOccupancyPadBytes, st>>>(x, sx_m, gpr, q, sc, zp, n_groups, items);
        else if (bn == 64) int4_fake_quant_vec_kernel<8, SYM, true><<<g, 256, kFakeOccupancyPadBytes, st>>>(x, sx_m, gpr, q, sc, zp, n_groups, items);
        else int4_fake_quant_vec_kernel<16, SYM, true><<<g, 256, kFakeOccupancyPadBytes, st>>>(x, sx_m, gpr, q, sc, zp, n_groups, items);
    } else {
        if (bn == 32) int4_fake_quant_vec_kernel<4, SYM, false><<<g, 256, kFakeOccupancyPadBytes, st>>>(x, sx_m, gpr, q, sc, zp, n_groups, items);
        else if (bn == 64) int4_fake_quant_vec_kernel<8, SYM, false><<<g, 256, kFakeOccupancyPadBytes, st>>>(x, sx_m, gpr, q, sc, zp, n_groups, items);
        else int4_fake_quant_vec_kernel<16, SYM, false><<<g, 256, kFakeOccupancyPadBytes, st>>>(x, sx_m, gpr, q, sc, zp, n_groups, items);
    }
    return true;
}

// Per-item launches of more than kPackItemsPerLaunch items go out as several launches of about that size over
// consecutive parts of the table (the stream orders them; a launch gap is 1.6 us).  Measured on the 48 layers of experts
// (3.5 M items; same tensors, same buffers, same process, alternating builds): one launch 78.8-79.9 % of HBM peak, pieces
// of 2^16 / 2^18 / 2^20 items 79.7-81.3 %.  (The block-FP8 quantiser does not change with the same treatment.)
constexpr int64_t kPackItemsPerLaunch = 1 << 18;

template <int GROUPED>
static int launch_pack(const Int4PackArgs& a0, int64_t work, int group, hipStream_t st)
{
    Int4PackArgs a = a0;
    const int64_t pieces = GROUPED == 2 ? cdiv64(work, kPackItemsPerLaunch) : 1;
    const int64_t per = cdiv64(cdiv64(work, pieces), 256) * 256;     // whole XCD spans per piece
    for (int64_t done = 0; done < work; done += per) {
        const int64_t n = min(per, work - done);
        switch (group) {
        case 32: int4_pack_kernel<4, GROUPED><<<grid_for_items(n), 256, kPackOccupancyPadBytes, st>>>(a, n); break;
        case 64: int4_pack_kernel<8, GROUPED><<<grid_for_items(n), 256, kPackOccupancyPadBytes, st>>>(a, n); break;
        case 128: int4_pack_kernel<16, GROUPED><<<grid_for_items(n), 256, kPackOccupancyPadBytes, st>>>(a, n); break;
        default: return WQ_ERR_UNSUPPORTED;
        }
        WQ_LAUNCH_CHECK();
        if (GROUPED == 2) a.descs += n;
    }
    return WQ_OK;
}

}  // namespace wq

using namespace wq;

WQ_EXPORT int wq_int4_group_quant_pack(const void* x, int64_t M, int64_t N, int64_t sx_m, int group, int32_t* packed,
                                       void* scale, void* stream)
{
    if (M < 0 || N < 0 || group <= 0 || group % 32 != 0 || N % group != 0) return WQ_ERR_SHAPE;
    if (M == 0 || N == 0) return WQ_OK;
    if (!x || !packed || !scale) return WQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    const int64_t n_groups = M * (N / group);
    const bool fast = (group == 32 || group == 64 || group == 128) && sx_m == N && ((uintptr_t)x & 15) == 0;
    if (fast) {
        Int4PackArgs a{};
        a.d = wq_int4_pack_desc{x, packed, scale, n_groups};
        return launch_pack<0>(a, cdiv64(n_groups, kGroupsPerWg), group, st);
    }
    int4_pack_generic_kernel<<<grid_for_items(cdiv64(n_groups, 16)), 256, 0, st>>>(
        (const uint16_t*)x, M, N, sx_m, group, (uint32_t*)packed, (uint16_t*)scale);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_group_quant_pack_grouped(const wq_int4_pack_desc* descs, const int64_t* work_start, int n_desc,
                                               int64_t total_work, int group, void* stream)
{
    if (n_desc < 0 || total_work < 0) return WQ_ERR_SHAPE;
    if (group != 32 && group != 64 && group != 128) return WQ_ERR_UNSUPPORTED;
    if (n_desc == 0 || total_work == 0) return WQ_OK;
    if (!descs || !work_start) return WQ_ERR_NULL;
    Int4PackArgs a{};
    a.descs = descs;
    a.work_start = work_start;
    a.n_desc = n_desc;
    return launch_pack<1>(a, total_work, group, (hipStream_t)stream);
}

WQ_EXPORT int wq_int4_fake_quant(const void* x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, int bm,
                                 int bn, int sym, void* q, void* scale, void* zero, void* stream)
{
    if (M < 0 || N < 0 || bm <= 0 || bn <= 0) return WQ_ERR_SHAPE;
    if (dtype != WQ_DTYPE_BF16 && dtype != WQ_DTYPE_F32 && dtype != WQ_DTYPE_F64) return WQ_ERR_MODE;
    if (((int64_t)bm * bn) % 32 != 0) return WQ_ERR_SHAPE;
    if (!((bm == 1 && bn % 32 == 0) || (32 % bn == 0))) return WQ_ERR_UNSUPPORTED;
    if ((int64_t)bm * bn > (1 << 30)) return WQ_ERR_TOO_LARGE;
    if (M == 0 || N == 0) return WQ_OK;
    if (!x || !q || !scale || !zero) return WQ_ERR_NULL;
    const int64_t groups = cdiv64(M, bm) * cdiv64(N, bn);
    hipStream_t st = (hipStream_t)stream;
    const bool vec = dtype == WQ_DTYPE_BF16 && bm == 1 && (bn == 32 || bn == 64 || bn == 128) && sx_n == 1 && N % bn == 0 &&
                     (sx_m & 7) == 0 && N / bn < (1ll << 31) && ((uintptr_t)x & 15) == 0 && ((uintptr_t)q & 15) == 0 &&
                     (sx_m == N || groups < (1ll << 32));
    if (vec) {
        if (sym) launch_fake_vec<true>((const uint16_t*)x, M, N, sx_m, bn, (uint16_t*)q, (uint16_t*)scale, (uint16_t*)zero, st);
        else launch_fake_vec<false>((const uint16_t*)x, M, N, sx_m, bn, (uint16_t*)q, (uint16_t*)scale, (uint16_t*)zero, st);
    } else if (dtype == WQ_DTYPE_BF16)
        int4_fake_quant_kernel<uint16_t><<<grid_for_items(cdiv64(groups, 4)), 256, 0, st>>>(
            (const uint16_t*)x, M, N, sx_m, sx_n, bm, bn, sym, (uint16_t*)q, (uint16_t*)scale, (uint16_t*)zero);
    else if (dtype == WQ_DTYPE_F64)
        int4_fake_quant_kernel<double><<<grid_for_items(cdiv64(groups, 4)), 256, 0, st>>>(
            (const double*)x, M, N, sx_m, sx_n, bm, bn, sym, (double*)q, (double*)scale, (double*)zero);
    else
        int4_fake_quant_kernel<float><<<grid_for_items(cdiv64(groups, 4)), 256, 0, st>>>(
            (const float*)x, M, N, sx_m, sx_n, bm, bn, sym, (float*)q, (float*)scale, (float*)zero);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_group_quant_pack_asym(const void* x, int64_t M, int64_t N, int64_t sx_m, int group,
                                            int32_t* packed, void* scale, void* zero, void* stream)
{
    if (M < 0 || N < 0 || group <= 0 || N % group != 0) return WQ_ERR_SHAPE;
    if (group != 32 && group != 64 && group != 128) return WQ_ERR_UNSUPPORTED;
    if (M == 0 || N == 0) return WQ_OK;
    if (!x || !packed || !scale || !zero) return WQ_ERR_NULL;
    if (((uintptr_t)x & 15) || (sx_m & 7) || ((uintptr_t)packed & 3) || ((uintptr_t)scale & 1) || ((uintptr_t)zero & 1))
        return WQ_ERR_ALIGN;
    if (N / group >= (1ll << 31)) return WQ_ERR_TOO_LARGE;
    const int64_t n_groups = M * (N / group);
    if (sx_m != N && n_groups >= (1ll << 32)) return WQ_ERR_TOO_LARGE;      // strided rows: 32-bit group index
    const int64_t items = cdiv64(n_groups, kFakeGroupsPerWg);
    const dim3 g = grid_for_items(items);
    const int gpr = (int)(N / group);
    hipStream_t st = (hipStream_t)stream;
    const uint16_t* xp = (const uint16_t*)x;
    uint32_t* pp = (uint32_t*)packed;
    if (group == 32) int4_pack_asym_kernel<4, false><<<g, 256, kFakeOccupancyPadBytes, st>>>(xp, sx_m, gpr, pp, (uint16_t*)scale, (uint16_t*)zero, n_groups, items, nullptr, nullptr, nullptr);
    else if (group == 64) int4_pack_asym_kernel<8, false><<<g, 256, kFakeOccupancyPadBytes, st>>>(xp, sx_m, gpr, pp, (uint16_t*)scale, (uint16_t*)zero, n_groups, items, nullptr, nullptr, nullptr);
    else int4_pack_asym_kernel<16, false><<<g, 256, kFakeOccupancyPadBytes, st>>>(xp, sx_m, gpr, pp, (uint16_t*)scale, (uint16_t*)zero, n_groups, items, nullptr, nullptr, nullptr);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_group_quant_pack_asym_items(const wq_int4_pack_asym_item* items, int64_t n_items, void* out_base,
                                                  void* zero_base, int group, void* stream)
{
    if (n_items < 0) return WQ_ERR_SHAPE;
    if (group != 32 && group != 64 && group != 128) return WQ_ERR_UNSUPPORTED;
    if (n_items == 0) return WQ_OK;
    if (!items) return WQ_ERR_NULL;
    const dim3 g = grid_for_items(n_items);
    hipStream_t st = (hipStream_t)stream;
    char* ob = (char*)out_base;
    char* zb = (char*)zero_base;
    if (group == 32) int4_pack_asym_kernel<4, true><<<g, 256, kFakeOccupancyPadBytes, st>>>(nullptr, 0, 1, nullptr, nullptr, nullptr, 0, n_items, items, ob, zb);
    else if (group == 64) int4_pack_asym_kernel<8, true><<<g, 256, kFakeOccupancyPadBytes, st>>>(nullptr, 0, 1, nullptr, nullptr, nullptr, 0, n_items, items, ob, zb);
    else int4_pack_asym_kernel<16, true><<<g, 256, kFakeOccupancyPadBytes, st>>>(nullptr, 0, 1, nullptr, nullptr, nullptr, 0, n_items, items, ob, zb);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

// Zero points of many tensors into the AWQ layout in one launch: zp bf16 [M, G] (integers 0..15) -> int32 [G, M/8],
// word (g, r) = sum over k < 8 of zp[8r + k, g] << 4 * order[k], order = 0,4,1,5,2,6,3,7.  One lane per word.
__global__ __launch_bounds__(256) void int4_zero_point_pack_kernel(const wq_int4_zp_desc* __restrict__ descs,
                                                                  const int64_t* __restrict__ word_start, int n_desc,
                                                                  int64_t total_words, const char* zero_base, char* out_base)
{
    const int64_t w = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * 256 + threadIdx.x;
    if (w >= total_words) return;
    int lo = 0, hi = n_desc;                       // largest i with word_start[i] <= w
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (word_start[mid] <= w) lo = mid; else hi = mid;
    }
    const wq_int4_zp_desc d = descs[lo];
    const int64_t local = w - word_start[lo];
    const int64_t words_per_row = d.M / 8;
    const int64_t g = local / words_per_row, r = local - g * words_per_row;
    const uint16_t* zp = (const uint16_t*)(zero_base + (uintptr_t)d.zero);
    uint32_t acc = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int order = (k >> 1) + 4 * (k & 1);                       // 0,4,1,5,2,6,3,7
        const float z = u2f((uint32_t)zp[(r * 8 + k) * d.G + g] << 16);
        acc += (uint32_t)(int)z << (4 * order);
    }
    ((uint32_t*)(out_base + (uintptr_t)d.out))[local] = acc;
}

WQ_EXPORT int wq_int4_zero_point_pack_grouped(const wq_int4_zp_desc* descs, const int64_t* word_start, int n_desc,
                                              int64_t total_words, const void* zero_base, void* out_base, void* stream)
{
    if (n_desc < 0 || total_words < 0) return WQ_ERR_SHAPE;
    if (n_desc == 0 || total_words == 0) return WQ_OK;
    if (!descs || !word_start) return WQ_ERR_NULL;
    int4_zero_point_pack_kernel<<<grid_for_items(cdiv64(total_words, 256)), 256, 0, (hipStream_t)stream>>>(
        descs, word_start, n_desc, total_words, (const char*)zero_base, (char*)out_base);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}

WQ_EXPORT int wq_int4_bucket_convert(const wq_int4_pack_desc* items, int64_t n_items, void* out_base, int group,
                                     void* stream)
{
    if (n_items < 0) return WQ_ERR_SHAPE;
    if (group != 32 && group != 64 && group != 128) return WQ_ERR_UNSUPPORTED;
    if (n_items == 0) return WQ_OK;
    if (!items || !out_base) return WQ_ERR_NULL;
    Int4PackArgs a{};
    a.descs = items;
    a.out_base = (char*)out_base;
    return launch_pack<2>(a, n_items, group, (hipStream_t)stream);
}

WQ_EXPORT int wq_int4_group_quant_pack_items(const wq_int4_pack_desc* items, int64_t n_items, int group, void* stream)
{
    if (n_items < 0) return WQ_ERR_SHAPE;
    if (group != 32 && group != 64 && group != 128) return WQ_ERR_UNSUPPORTED;
    if (n_items == 0) return WQ_OK;
    if (!items) return WQ_ERR_NULL;
    Int4PackArgs a{};
    a.descs = items;
    return launch_pack<2>(a, n_items, group, (hipStream_t)stream);
}
