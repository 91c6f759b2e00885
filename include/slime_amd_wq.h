/*
 * slime_amd_wq.h - C ABI of libslime_amd_wq.so: MI355X (gfx950) kernels for slime's
 * low-precision weight-conversion path (bf16 -> block-FP8, bf16 -> group-INT4 pack,
 * block-FP8 -> bf16).
 *
 * Conventions
 *   - All data pointers are DEVICE pointers on the current HIP device unless a parameter is
 *     marked "host".  Sizes and strides are in ELEMENTS.  `stream` is a hipStream_t passed
 *     as void*; NULL selects the default stream.  Launches are asynchronous and are ordered
 *     on `stream` only; the library keeps no mutable global state and every entry point may
 *     be called concurrently from several host threads (one exception, documented there:
 *     wq_delta_xor_noalloc works in a device array owned by the library).  No entry point
 *     allocates, frees, clears memory with a memset node or synchronises, so every call may be
 *     recorded into a HIP graph (stream capture) and replayed on updated inputs.
 *   - Return value: 0 on success, a negative WQ_ERR_* for rejected arguments (nothing was
 *     launched), or a positive hipError_t reported by the launch.  wq_error_string() names any
 *     of them.
 *   - FP8 is OCP float8_e4m3fn (bias 7, max 448, 0x7F/0xFF NaN, no infinities).
 *   - Outputs are bit-identical to the reference torch path for finite inputs.  A NaN in a
 *     block makes the block's scale NaN and all its codes NaN (0x7F or 0xFF: the sign of a NaN
 *     code is unspecified, as it is host-dependent in the reference); +-Inf behaves as IEEE
 *     division does (finite/Inf = signed zero, Inf/Inf = NaN).
 *
 * Reference citations are paths inside the THUDM/slime checkout.
 */
#ifndef SLIME_AMD_WQ_H
#define SLIME_AMD_WQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WQ_ABI_VERSION 18

enum {
    WQ_OK = 0,
    WQ_ERR_NULL = -1,        /* a required pointer is NULL */
    WQ_ERR_SHAPE = -2,       /* negative size, zero block, N not a multiple of the group ... */
    WQ_ERR_MODE = -3,        /* unknown mode / dtype selector */
    WQ_ERR_UNSUPPORTED = -4, /* valid in the reference but not provided by this library */
    WQ_ERR_ALIGN = -5,       /* pointer or stride violates a documented alignment requirement */
    WQ_ERR_TOO_LARGE = -6    /* a count exceeds the launch limits of the entry point */
};

/* element type selectors */
enum { WQ_DTYPE_BF16 = 0, WQ_DTYPE_F32 = 1, WQ_DTYPE_F16 = 2, WQ_DTYPE_F64 = 3 };

/* FP8 block quant arithmetic.
 * WQ_FP8_MODE_TORCH  : amax clamped at bf16(1e-12) in bf16, scale = f32(amax)/448, q = f32(x)/scale
 *                      (IEEE division), clamp +-448, RNE to e4m3fn.
 *                      Replaces block_fp8, tools/convert_hf_to_fp8.py:41-75, as torch evaluates it on CPU
 *                      tensors (how the reference's own test runs it, tests/test_block_fp8_zero_block.py).
 * WQ_FP8_MODE_TORCH_DEVICE : the same function as torch evaluates it on GPU tensors (how the tool runs
 *                      it, tools/convert_hf_to_fp8.py:127): torch's GPU kernels compute
 *                      `tensor / python_scalar` as tensor * (1.0f/scalar), so
 *                      scale = f32(amax) * RN(1/448), up to one ulp from the quotient; everything else
 *                      (the IEEE x/scale, clamp, cast) is as in WQ_FP8_MODE_TORCH.
 * WQ_FP8_MODE_TRITON : fp32 amax floored at 1e-10f, scale = amax/448, q = f32(x)*(1.0f/scale).
 *                      Replaces _blockwise_cast_to_fp8_triton,
 *                      slime/backends/megatron_utils/kernels/fp8_kernel.py:24-58.
 * WQ_FP8_MODE_UE8M0  : power-of-two scales: fp32 amax floored at 1e-4, scale = 2^ceil(log2(amax/448)),
 *                      q = f32(x) * (1/scale) (exact), RNE to e4m3fn, no clamp (|q| <= 448 by construction).
 *                      Replaces quant_weight_ue8m0 as called at quantizer_fp8.py:103-106 - a function of sglang
 *                      (not vendored in the reference), so bit parity with it is unpinned; bf16 weights only
 *                      (wq_fp8_block_quant and the grouped / tile / bucket forms), 128x128 blocks in the reference. */
enum { WQ_FP8_MODE_TORCH = 0, WQ_FP8_MODE_TRITON = 1, WQ_FP8_MODE_TORCH_DEVICE = 2, WQ_FP8_MODE_UE8M0 = 3 };

/* FP8 block dequant arithmetic.
 * WQ_DEQ_MODE_F32SCALE  : y = bf16(f32(x) * s).  Replaces weight_dequant, tools/fp8_cast_bf16.py:16-41.
 * WQ_DEQ_MODE_BF16SCALE : y = bf16(f32(x) * f32(bf16(s))).  Replaces the dequant-on-read of
 *                         slime/backends/megatron_utils/hf_to_megatron/common.py:42-56. */
enum { WQ_DEQ_MODE_F32SCALE = 0, WQ_DEQ_MODE_BF16SCALE = 1 };

int wq_abi_version(void);
const char *wq_error_string(int code);

/* ---------------------------------------------------------------------------------------------
 * bf16 [M,N] -> e4m3fn [M,N] + fp32 scale [ceil(M/bm), ceil(N/bn)], one (bm x bn) block per scale.
 * x: bf16, element (i,j) at x[i*sx_m + j*sx_n] (any strides, as the reference kernel accepts,
 * fp8_kernel.py:51,72-75).  y: bytes, element (i,j) at y[i*sy_m + j].  s: contiguous.
 * Elements of an edge block outside [M,N] count as +0.0 (F.pad, convert_hf_to_fp8.py:51-56).
 * The 128x128 contiguous-row case runs the single-pass vector kernel; every other block shape
 * or layout runs a generic kernel with identical results. */
int wq_fp8_block_quant(const void *x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                       void *y, int64_t sy_m, float *s, int bm, int bn, int mode, void *stream);

/* One launch over many tensors (a weight-sync bucket or a whole state dict; the per-parameter
 * loop it replaces is slime/backends/megatron_utils/update_weight/hf_weight_iterator_direct.py:50-67
 * calling quantizer_fp8.py:98-118 once per tensor).  `descs` is a DEVICE array of n_desc
 * descriptors; `tile_start` is a DEVICE array of n_desc+1 int64: exclusive prefix sum of
 * ceil(M/bm)*ceil(N/bn) over the descriptors; total_tiles = tile_start[n_desc] (passed by value). */
typedef struct wq_fp8_quant_desc {
    const void *x;   /* bf16 */
    void *y;         /* e4m3fn bytes */
    float *s;        /* fp32 scales, contiguous [ceil(M/bm), ceil(N/bn)] */
    int64_t M, N;
    int64_t sx_m, sx_n;
    int64_t sy_m;
} wq_fp8_quant_desc;

int wq_fp8_block_quant_grouped(const wq_fp8_quant_desc *descs, const int64_t *tile_start, int n_desc,
                               int64_t total_tiles, int bm, int bn, int mode, void *stream);

/* The grouped launch for up to WQ_FP8_FEW_MAX tensors, with the descriptors in the kernel arguments: `descs` is a
 * HOST array that the call reads before it returns - no device table to build, upload, cache or keep valid.  Meant for
 * the q/k/v or gate/up group of ONE weight-sync parameter (quantize_params_fp8, quantizer_fp8.py:69-95, calls
 * _quantize_param once per tensor of the group), whose tensors are fresh allocations on every sync.  With out_base
 * non-NULL the y and s fields are byte offsets from it (one allocation for all outputs of the group).  Descriptors
 * with M == 0 or N == 0 are skipped. */
#define WQ_FP8_FEW_MAX 4
int wq_fp8_block_quant_few(const wq_fp8_quant_desc *descs, int n_desc, void *out_base, int bm, int bn, int mode,
                           void *stream);

/* The same launch with every tile resolved beforehand: `tiles` is a DEVICE array with one descriptor per
 * (bm x bn) tile, moved to the tile's origin - x and y point at the tile's first element, s at the tile's scale,
 * M and N are the rows and columns of the tensor from there on (the kernel uses min(bm, M) x min(bn, N)), strides
 * as in the tensor.  Costs 64 bytes of table per tile and saves the per-workgroup search; meant for plans that
 * are built once and run every weight sync. */
int wq_fp8_block_quant_tiles(const wq_fp8_quant_desc *tiles, int64_t n_tiles, int bm, int bn, int mode, void *stream);

/* A whole weight-sync bucket in ONE launch, written into ONE caller-owned byte buffer: the loop over
 * convert_to_hf / quantize_params in HfWeightIteratorDirect._convert_to_hf_named_tensors
 * (slime/backends/megatron_utils/update_weight/hf_weight_iterator_direct.py:50-67) followed by the flatten copy of
 * FlattenedTensorBucket (update_weight_from_tensor.py:30-48).  `items` is a DEVICE array like the `tiles` of
 * wq_fp8_block_quant_tiles, except that y and s hold BYTE OFFSETS from `out_base` (so a table built once serves a
 * fresh output buffer on every sync), and that a descriptor with sx_m == WQ_BUCKET_COPY_MARK is a pass-through item:
 * M bytes (at most WQ_BUCKET_COPY_BYTES) are copied from x to out_base + y, any alignment.  Quantised tiles need y
 * 4-byte aligned for the vector kernel (other alignments take the generic one) and s 4-byte aligned. */
#define WQ_BUCKET_COPY_MARK (-1)
#define WQ_BUCKET_COPY_BYTES 32768
int wq_fp8_bucket_convert(const wq_fp8_quant_desc *items, int64_t n_items, void *out_base, int bm, int bn, int mode,
                          void *stream);

/* wq_fp8_bucket_convert for items whose code rows do NOT start on 64-byte boundaries (out_base + y or sy_m not a multiple of
 * 64): same items, same results, plain instead of streaming stores, so that the two tiles that share every 128-byte line of
 * such a tensor have their halves merged in the L2 (65-70 % of HBM peak wherever the rows start, where the streaming form
 * falls to 44-55 %; for aligned rows the streaming form's 80 % is 8-10 points ahead).  A caller that packs tensors back to
 * back, as FlattenedTensorBucket does (update_weight_from_tensor.py:30-48), knows every offset when it builds its tables and
 * puts the items of each kind into the launch made for it. */
int wq_fp8_bucket_convert_rows_off_lines(const wq_fp8_quant_desc *items, int64_t n_items, void *out_base, int bm, int bn,
                                         int mode, void *stream);

/* The bucket tables above hold the ADDRESS of every item's input, while the inputs of a weight-sync bucket are fresh
 * tensors on every sync as soon as the model is sharded: all_gather_param fills torch.empty_like partitions and
 * concatenates them (slime/backends/megatron_utils/update_weight/common.py:97,120) before
 * HfWeightIteratorDirect._convert_to_hf_named_tensors (hf_weight_iterator_direct.py:50-67) sees them.  So that a moved
 * bucket costs one small upload and one launch instead of a new table, the caller keeps the table as a TEMPLATE -
 * `item_template`: DEVICE int64[n_items * words_per_item], the item descriptors of wq_fp8_bucket_convert (8 words),
 * wq_int4_bucket_convert (4) or wq_int4_group_quant_pack_asym_items (5) with word 0 (x) holding the byte OFFSET of the
 * item's input inside its tensor - plus `owner`: DEVICE int32[n_items], the index of that tensor, and passes the
 * tensors' current addresses as `bases`: DEVICE int64[n_tensors].  Writes items[i] = item_template[i] with
 * bases[owner[i]] added to word 0.  `items` must not alias `item_template`. */
int wq_bucket_resolve_items(const int64_t *item_template, const int32_t *owner, const int64_t *bases,
                            int64_t n_items, int words_per_item, int64_t *items, void *stream);

/* wq_fp8_block_quant for bf16, fp16 or fp32 weights (`dtype` = WQ_DTYPE_*): the reference functions take any
 * floating dtype - block_fp8 computes amax and the 1e-12 floor in the weight dtype (the floor rounds to 0 in
 * fp16), the Triton cast converts to fp32 on load (fp8_kernel.py:50).  A plain two-pass kernel: bf16 weights
 * should go through wq_fp8_block_quant, which gives the same bytes several times faster. */
int wq_fp8_block_quant_any(const void *x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                           void *y, int64_t sy_m, float *s, int bm, int bn, int mode, void *stream);

/* Per-row and per-tensor scaling: channel_fp8 / tensor_fp8, tools/convert_hf_to_fp8.py:78-91, and the
 * per-tensor branch of _quantize_param, quantizer_fp8.py:112-117.  s has M entries (row) or 1 (tensor).
 * wq_fp8_tensor_quant needs `workspace`: one zero-initialised uint32 in device memory that the call
 * may overwrite (the cross-workgroup amax).  `mode` is WQ_FP8_MODE_TORCH or WQ_FP8_MODE_TORCH_DEVICE. */
int wq_fp8_row_quant(const void *x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                     void *y, int64_t sy_m, float *s, int mode, void *stream);
int wq_fp8_tensor_quant(const void *x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                        void *y, int64_t sy_m, float *s, uint32_t *workspace, int mode, void *stream);
/* tensor_fp8 for the other floating dtypes the reference function takes (dtype: WQ_DTYPE_BF16 / F32 / F16): the
 * quotient is rounded to the weight's dtype before the clamp, as torch's type promotion with a 0-dim scale makes it;
 * plain two-pass kernels.  (channel_fp8 on those dtypes is wq_fp8_block_quant_any with bm = 1, bn = N: a row is a
 * block, and both divide by a dimensioned fp32 scale.) */
int wq_fp8_tensor_quant_any(const void *x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                            void *y, int64_t sy_m, float *s, uint32_t *workspace, int mode, void *stream);

/* ---------------------------------------------------------------------------------------------
 * bf16 [M,N] -> bf16 [M,N] carrying the values the weight has after block-FP8 quantisation: per block
 * the codes of wq_fp8_block_quant (same `mode`, all four accepted) are formed in registers and expanded
 * again as wq_fp8_block_dequant does (f32(code) * scale, one RNE rounding to bf16), in ONE pass of
 * 2 + 2 bytes per element.  Replaces the pair blockwise_cast_to_fp8_triton / quant_weight_ue8m0 ->
 * block_quant_dequant of _get_fp8_aligned_absorb_weight (slime_plugins/models/glm5/glm5.py:105-165;
 * modes WQ_FP8_MODE_TRITON and WQ_FP8_MODE_UE8M0 there) and is bit-identical to the two calls.
 * Strides in elements (y: unit column stride); `s` [ceil(M/bm), ceil(N/bn)] contiguous receives the
 * block scales, or NULL. */
int wq_fp8_block_quant_dequant(const void *x, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n, void *y,
                               int64_t sy_m, float *s, int bm, int bn, int mode, void *stream);

/* ---------------------------------------------------------------------------------------------
 * e4m3fn [M,N] contiguous + fp32 scale [ceil(M/block), ceil(N/block)] contiguous -> y [M,N]
 * contiguous, of type out_dtype: WQ_DTYPE_BF16 or WQ_DTYPE_F16 (product rounded once, RNE; fp16 with
 * mode WQ_DEQ_MODE_F32SCALE only) or WQ_DTYPE_F32 (the fp32 product itself).  Replaces weight_dequant (tools/fp8_cast_bf16.py:31-41), which asserts the same
 * contiguity and writes torch's default dtype (bf16 in the tool, :45). */
int wq_fp8_block_dequant(const void *x, const float *s, void *y, int out_dtype, int64_t M, int64_t N,
                         int block, int mode, void *stream);

typedef struct wq_fp8_dequant_desc {
    const void *x;
    const float *s;
    void *y;
    int64_t M, N;
} wq_fp8_dequant_desc;

/* Grouped form: `descs` DEVICE array, `work_start` DEVICE int64[n_desc+1] exclusive prefix sum of
 * per-tensor work items, where a tensor has ceil(M * ceil(N/WQ_DEQ_SEG) / WQ_DEQ_SEGS_PER_WG) items
 * (rows are cut into segments of WQ_DEQ_SEG codes; a work item is WQ_DEQ_SEGS_PER_WG consecutive segments).
 * Per tensor, N and M * ceil(N/WQ_DEQ_SEG) must be below 2^31 (the single-tensor entry point checks this and
 * returns WQ_ERR_TOO_LARGE; for the grouped form it is the caller's obligation). */
#define WQ_DEQ_SEG 512
#define WQ_DEQ_SEGS_PER_WG 16
int wq_fp8_block_dequant_grouped(const wq_fp8_dequant_desc *descs, const int64_t *work_start, int n_desc,
                                 int64_t total_work, int out_dtype, int block, int mode, void *stream);

/* The grouped form with the owner of every work item resolved beforehand: one descriptor per work item - the tensor
 * (x, s, y, M, N as in wq_fp8_dequant_desc) and the index of the item inside it.  48 bytes of table per 24 KiB of
 * traffic; saves the per-workgroup search. */
typedef struct wq_fp8_dequant_item {
    const void *x;
    const float *s;
    void *y;
    int64_t M, N;
    int64_t item;
} wq_fp8_dequant_item;
int wq_fp8_block_dequant_items(const wq_fp8_dequant_item *items, int64_t n_items, int out_dtype, int block, int mode,
                               void *stream);

/* ---------------------------------------------------------------------------------------------
 * "Fake" INT4 quantisation: per (bm x bn) group, q = rintf(x/scale) [+ zero] stored in the input
 * dtype, plus scale and zero point [ceil(M/bm), ceil(N/bn)] in the input dtype.
 * Replaces fake_int4_quant_cuda(x, block_size, sym),
 * slime/backends/megatron_utils/kernels/int4_qat/fake_int4_quant_cuda.cu:327-378 (kernels :37-267).
 * dtype: WQ_DTYPE_BF16, WQ_DTYPE_F32 or WQ_DTYPE_F64 - the types the reference dispatches on (.cu:352-354); the
 * arithmetic is fp32 for all of them (elements are converted on load, results on store).  x has any strides;
 * q/scale/zero are contiguous.
 * Group shapes: (1, 32k), or bn dividing 32 with bm*bn a multiple of 32 (the shapes for which the
 * reference kernels are well defined); others return WQ_ERR_UNSUPPORTED. */
int wq_int4_fake_quant(const void *x, int dtype, int64_t M, int64_t N, int64_t sx_m, int64_t sx_n,
                       int bm, int bn, int sym, void *q, void *scale, void *zero, void *stream);

/* Fused symmetric group quantise + nibble pack: bf16 [M,N] (row stride sx_m, unit column stride,
 * N % group == 0, group % 32 == 0) -> packed int32 [M, N/8] + bf16 scale [M, N/group], both contiguous.
 * Word c of row i holds sum_j (q[i,8c+j]+8) << 4j.  Replaces pack_layer(weight, group_size, sym=True),
 * tools/convert_hf_to_int4_direct.py:123-153 == quantizer_compressed_tensors.py:235-265. */
int wq_int4_group_quant_pack(const void *x, int64_t M, int64_t N, int64_t sx_m, int group,
                             int32_t *packed, void *scale, void *stream);

typedef struct wq_int4_pack_desc {
    const void *x;   /* bf16, contiguous [M,N] */
    int32_t *packed; /* [M, N/8] */
    void *scale;     /* bf16 [M, N/group] */
    int64_t n_groups; /* M * N / group */
} wq_int4_pack_desc;

/* Grouped form for contiguous tensors (e.g. all experts of a layer).  `descs` DEVICE array;
 * `work_start` DEVICE int64[n_desc+1] exclusive prefix sum of ceil(n_groups / WQ_INT4_GROUPS_PER_WG). */
#define WQ_INT4_GROUPS_PER_WG 64
int wq_int4_group_quant_pack_grouped(const wq_int4_pack_desc *descs, const int64_t *work_start, int n_desc,
                                     int64_t total_work, int group, void *stream);

/* The same launch with the owner of every work item resolved beforehand: `items` is a DEVICE array with one
 * descriptor per work item - x, packed and scale pointing at the item's first group, n_groups = the groups of the
 * item (at most WQ_INT4_GROUPS_PER_WG; every item but a tensor's last has exactly that many).  Costs 32 bytes of
 * table per 16 KiB of weights and saves the per-workgroup search; meant for plans that are built once and run
 * every weight sync. */
int wq_int4_group_quant_pack_items(const wq_int4_pack_desc *items, int64_t n_items, int group, void *stream);

/* The INT4 counterpart of wq_fp8_bucket_convert (the per-parameter loop it replaces calls
 * quantize_params_compressed_tensors, quantizer_compressed_tensors.py:268-297, once per parameter): `items` as in
 * wq_int4_group_quant_pack_items with packed and scale holding BYTE OFFSETS from `out_base`; an item with
 * n_groups < 0 is a pass-through item that copies -n_groups bytes (at most WQ_BUCKET_COPY_BYTES) from x to
 * out_base + packed, any alignment.  packed offsets 4-byte aligned, scale offsets 2-byte aligned. */
int wq_int4_bucket_convert(const wq_int4_pack_desc *items, int64_t n_items, void *out_base, int group, void *stream);

/* Asymmetric form of wq_int4_group_quant_pack (pack_layer(weight, group, sym=False),
 * tools/convert_hf_to_int4_direct.py:123-153): codes rintf(x/scale) + zero with scale = max((max-min)/15, 1e-5)
 * and zero = clamp(-rintf(min/scale), 0, 15) (fake_int4_quant_cuda.cu:61-75), passed through the reference's
 * dequantise / re-quantise / clamp-to-uint8 chain and packed without masking, as pack_to_int32 does.
 * Outputs: packed int32 [M,N/8], scale bf16 [M,N/group], zero bf16 [M,N/group] (the caller packs the zero points
 * in AWQ order from it, :134-141).  x bf16, unit column stride, 16-byte aligned rows; group in {32, 64, 128}. */
int wq_int4_group_quant_pack_asym(const void *x, int64_t M, int64_t N, int64_t sx_m, int group,
                                  int32_t *packed, void *scale, void *zero, void *stream);

/* wq_int4_group_quant_pack_asym over many contiguous tensors in one launch (the experts of a layer under an asymmetric
 * compressed-tensors configuration): one descriptor per work item of WQ_INT4_GROUPS_PER_WG groups, pointing at the
 * item's first group in x (16-byte aligned), packed, scale and zero; n_groups = the groups of the item.  With a
 * non-NULL out_base (zero_base) the packed and scale (zero) fields are byte offsets from it, and an item with
 * n_groups < 0 copies -n_groups bytes (at most WQ_BUCKET_COPY_BYTES) from x to out_base + packed: the asymmetric
 * counterpart of wq_int4_bucket_convert. */
typedef struct wq_int4_pack_asym_item {
    const void *x;
    int32_t *packed;
    void *scale;     /* bf16 */
    void *zero;      /* bf16 */
    int64_t n_groups;
} wq_int4_pack_asym_item;
int wq_int4_group_quant_pack_asym_items(const wq_int4_pack_asym_item *items, int64_t n_items, void *out_base,
                                        void *zero_base, int group, void *stream);

/* The zero points of many tensors packed into the AWQ layout of pack_layer (tools/convert_hf_to_int4_direct.py:134-141)
 * in one launch: per tensor `zero` bf16 [M, G] as wq_int4_group_quant_pack_asym writes it -> `out` int32 [G, M/8],
 * word (g, r) = sum over k < 8 of zero[8r + k, g] << 4 * (0,4,1,5,2,6,3,7)[k].  M must be a multiple of 8 (the
 * reference's reshape fails otherwise).  `descs` DEVICE array, `word_start` DEVICE int64[n_desc + 1] exclusive prefix
 * sum of G * M / 8.  `zero` / `out` are addresses, or byte offsets from zero_base / out_base when those are non-NULL. */
typedef struct wq_int4_zp_desc {
    const void *zero;
    int32_t *out;
    int64_t M, G;
} wq_int4_zp_desc;
int wq_int4_zero_point_pack_grouped(const wq_int4_zp_desc *descs, const int64_t *word_start, int n_desc,
                                    int64_t total_words, const void *zero_base, void *out_base, void *stream);

/* INT4 pack-quantized -> bf16: y[i,j] = bf16((nibble(i,j) - 8) * f32(scale[i, j/group])), nibble j of word c at
 * bits [4j,4j+4).  packed int32 [M,N/8], scale bf16 [M,N/group], y bf16 [M,N], all contiguous; N % group == 0,
 * group % 8 == 0.  Replaces _dequantize_tensor, tools/convert_k2_thinking_int4_to_bf16.py:55-84 (whose unpacking
 * is compressed_tensors.unpack_from_int32). */
int wq_int4_dequant(const int32_t *packed, const void *scale, void *y, int64_t M, int64_t N, int group, void *stream);

/* wq_int4_dequant for the inputs the tuned kernel does not take: scales stored as WQ_DTYPE_BF16, WQ_DTYPE_F16 or
 * WQ_DTYPE_F32 (the reference converts any dtype with .to(float32), convert_k2_thinking_int4_to_bf16.py:69), any
 * group >= 1 dividing N (group 1 with one scale per element is the reference's group_size <= 0 branch, :74-75), and N
 * that is not a multiple of 8 (packed is [M, ceil(N/8)]; unpack_from_int32 cuts the last word of a row).  With an fp32
 * scale the product is rounded to fp32 and then to bf16, as in the reference.  A plain kernel. */
int wq_int4_dequant_any(const int32_t *packed, const void *scale, int scale_dtype, void *y, int64_t M, int64_t N,
                        int group, void *stream);

/* wq_int4_dequant over a bucket of tensors in one launch.  `items` is a DEVICE array with one entry per work item
 * of WQ_INT4_DEQ_WORDS_PER_ITEM packed words (a tensor's last item may be shorter): pointers to the item's first
 * packed word, to the scale of its first element and to its first output element, and its number of words.
 * `group` must be a power of two between 8 and 8 * WQ_INT4_DEQ_WORDS_PER_ITEM, so that an item starts on a group
 * boundary; y pointers 16-byte aligned. */
#define WQ_INT4_DEQ_WORDS_PER_ITEM 512
typedef struct wq_int4_dequant_item {
    const int32_t *packed;
    const void *scale;   /* bf16 */
    void *y;             /* bf16 */
    int64_t n_words;
} wq_int4_dequant_item;
int wq_int4_dequant_items(const wq_int4_dequant_item *items, int64_t n_items, int group, void *stream);

/* Forward of the INT4 QAT straight-through estimator: per (1 x group) group of a contiguous bf16 [M,N],
 * s = max(f32(amax) / 7, 1e-5), y = bf16(clamp(round_half_even(f32(x) / s), -7, 7) * s); N % group == 0 and
 * group in {32, 64, 128}.  Replaces _FakeInt4QuantizationSTE.forward, docker/patch/latest/megatron.patch:212-246
 * (it dequantises with the unrounded fp32 scale, unlike pack_layer).  `div7` selects how `amax / 7` is evaluated:
 * WQ_DIV7_IEEE as torch does on CPU tensors (a division), WQ_DIV7_DEVICE as torch does on GPU tensors
 * (amax * RN(1/7), which is also what fake_int4_quant_cuda.cu:59 computes); x / s is an IEEE division in both. */
enum { WQ_DIV7_IEEE = 0, WQ_DIV7_DEVICE = 1 };
int wq_int4_fake_quant_ste(const void *x, void *y, int64_t M, int64_t N, int group, int div7, void *stream);

/* The same forward over many contiguous tensors in one launch (the expert weights of a grouped linear layer, which
 * the patched forward quantises one by one, docker/patch/latest/megatron.patch:256-279): one descriptor per work item
 * of WQ_INT4_GROUPS_PER_WG groups, pointing at the item's first group in x and y (16-byte aligned).  With a non-NULL
 * y_base the y fields are byte offsets from it, so that a table built once serves a fresh output buffer every step. */
typedef struct wq_int4_ste_item {
    const void *x;
    void *y;
    int64_t n_groups;
} wq_int4_ste_item;
int wq_int4_fake_quant_ste_items(const wq_int4_ste_item *items, int64_t n_items, void *y_base, int group, int div7,
                                 void *stream);

/* ---------------------------------------------------------------------------------------------
 * Byte-level delta of a tensor against its snapshot (delta weight sync).
 *
 * wq_delta_xor replaces, for one tensor, the xor branch of diff_and_compress in
 * UpdateWeightFromDiskDelta._encode_delta, slime/backends/megatron_utils/update_weight/
 * update_weight_from_disk_delta.py:224-246 - `diff = new ^ old; changed = count_nonzero(diff)`, the snapshot
 * update `snapshot[name] = new` - and checksum("adler32", new), slime/utils/disk_delta.py:28-58, in one pass:
 *   diff[i] = new[i] ^ old[i]            (skipped when diff == NULL)
 *   old[i]  = new[i]                     (when update_old != 0)
 *   result[0] = number of bytes with new[i] != old[i];  result[1] = zlib-compatible adler32 of new[0..n)
 * All buffers are DEVICE memory; new/old/diff 16-byte aligned, n in bytes (any value >= 0).  `workspace` is
 * device scratch of wq_delta_workspace_bytes(n) bytes (8-byte aligned) that needs no initialisation and, after
 * the call, holds the per-chunk counts wq_delta_overwrite_encode consumes.  `result` is 2 x uint64, device.
 *
 * wq_delta_overwrite_encode replaces overwrite_encode(new, new != old), slime/utils/disk_delta.py:21-25:
 *   out = [count u32 LE][positions u32 LE x count, ascending][new[position] x count]
 * Call wq_delta_xor (or wq_delta_xor_xxh3) first on the same (new, old, n, workspace) with update_old == 0, read back
 * count = result[0], size `out` to 4 + 5 * count bytes (4-byte aligned), then call this.  n <= 2^32 - 1.
 * With update_old != 0 the same pass brings the snapshot up to date (old[i] = new[i]; `collect`:
 * snapshot[name] = new, update_weight_from_disk_delta.py:246-251), so the encoding needs no third pass. */
#define WQ_DELTA_CHUNK 16384
int64_t wq_delta_workspace_bytes(int64_t n);
int wq_delta_xor(const void *new_bytes, void *old_bytes, void *diff, int64_t n, int update_old,
                 void *workspace, uint64_t *result, void *stream);
int wq_delta_overwrite_encode(const void *new_bytes, void *old_bytes, int64_t n, void *workspace,
                              uint32_t count, void *out, int update_old, void *stream);

/* wq_delta_xor without the workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The per-chunk partial sums go to a device array inside the library (24 bytes per WQ_DELTA_CHUNK of input,
 * 6 MiB per GPU, held until the process ends); the call allocates and frees nothing.  n may not exceed
 * WQ_DELTA_NOALLOC_MAX_BYTES (WQ_ERR_TOO_LARGE otherwise; split larger tensors).  Arguments, alignment rules and
 * results are those of wq_delta_xor.  All calls on one GPU share the array: calls that may overlap on one GPU
 * (different streams, or several host threads) race - order them on one stream.  Nothing has to be cleared
 * between calls.  The first call on a device looks up the array's address (no stream work); make that call
 * outside a graph capture.  The array does not hold the scan slots of wq_delta_overwrite_encode. */
#define WQ_DELTA_NOALLOC_MAX_BYTES (4294967296LL)
int wq_delta_xor_noalloc(const void *new_bytes, void *old_bytes, void *diff, int64_t n, int update_old,
                         uint64_t *result, void *stream);

/* wq_delta_xor over a bucket of tensors with two launches in total (the shape a weight-sync bucket wants:
 * update_weight_from_disk_delta.py:252-270 walks the gathered tensors one by one).  `descs` is a DEVICE array
 * whose fields mean what the arguments of wq_delta_xor mean (a tensor with n == 0 is allowed); `chunk_start`
 * is a DEVICE int64[n_desc+1] exclusive prefix sum of ceil(n / WQ_DELTA_CHUNK); total_chunks = chunk_start[n_desc].
 * With write_diff == 0 the `diff` fields are ignored.  The entry point cannot check alignment of the pointers
 * inside `descs`: the caller guarantees what wq_delta_xor checks.
 *
 * with_xxh3 != 0 adds the XXH3-128 digest of the new bytes of every tensor that changed - checksum("xxh3-128", new),
 * the digest diff_and_compress attaches by default (slime/utils/disk_delta.py:40-58) - to the same pass: the bytes
 * the diff reads anyway also feed the per-block sums (written to `xxh3_sums`: wq_xxh3_workspace_bytes(n) bytes,
 * 16-byte aligned), and one more small launch walks them into `xxh3_digest` ({low64, high64}, as wq_xxh3_128).  A
 * tensor with result[0] == 0 gets the digest {0, 0}: nothing is published for it.  With with_xxh3 == 0 the two
 * fields are ignored. */
typedef struct wq_delta_desc {
    const void *new_bytes;
    void *old_bytes;
    void *diff;
    int64_t n;
    void *workspace;        /* wq_delta_workspace_bytes(n) bytes */
    uint64_t *result;       /* 2 x uint64 */
    uint64_t *xxh3_sums;    /* with_xxh3: wq_xxh3_workspace_bytes(n) bytes */
    uint64_t *xxh3_digest;  /* with_xxh3: 2 x uint64 */
} wq_delta_desc;
int wq_delta_xor_grouped(const wq_delta_desc *descs, const int64_t *chunk_start, int n_desc,
                         int64_t total_chunks, int write_diff, int update_old, int with_xxh3, void *stream);

/* wq_delta_xor_grouped with the owner of every chunk resolved beforehand: `items` holds one descriptor per
 * WQ_DELTA_CHUNK of every tensor (the tensor's buffers and the chunk's index inside it; 64 bytes, so that an item is
 * one aligned scalar load); `descs` is still needed, per tensor, by the passes that fold the per-chunk sums into
 * `result` and walk the digest. */
typedef struct wq_delta_chunk_item {
    const void *new_bytes;
    void *old_bytes;
    void *diff;
    int64_t n;
    void *workspace;
    int64_t chunk;
    uint64_t *xxh3_sums;    /* the tensor's, as in its wq_delta_desc */
    int64_t reserved;
} wq_delta_chunk_item;
int wq_delta_xor_items(const wq_delta_chunk_item *items, int64_t n_items, const wq_delta_desc *descs, int n_desc,
                       int write_diff, int update_old, int with_xxh3, void *stream);

/* wq_delta_xor plus the digest, for one tensor: xxh3_workspace and digest as in wq_xxh3_128. */
int wq_delta_xor_xxh3(const void *new_bytes, void *old_bytes, void *diff, int64_t n, int update_old,
                      void *workspace, uint64_t *result, uint64_t *xxh3_workspace, uint64_t *digest, void *stream);

/* ---------------------------------------------------------------------------------------------
 * XXH3-128 (seed 0) of n >= 0 bytes in device memory: the digest checksum("xxh3-128", new) attaches to every
 * changed tensor of a published delta (slime/utils/disk_delta.py:40-58; the default of
 * --update-weight-delta-checksum, slime/utils/arguments.py:186-188), computed where the tensor lives instead of
 * after a copy to the host.  digest: DEVICE uint64[2] = {low64, high64}; the reference's hexdigest() is
 * high64 then low64, most significant byte first.  workspace: DEVICE, wq_xxh3_workspace_bytes(n) bytes
 * (64 per KiB of input), 16-byte aligned, overwritten.  Any alignment of `data` (16-byte aligned inputs take
 * the fast path; NULL allowed for n = 0).  Inputs up to 240 bytes take XXH3's short forms on one lane. */
int64_t wq_xxh3_workspace_bytes(int64_t n);
int wq_xxh3_128(const void *data, int64_t n, uint64_t *workspace, uint64_t *digest, void *stream);

/* Many tensors, two launches.  `descs` DEVICE array; item_start DEVICE int64[n_desc+1], exclusive prefix sum of
 * ceil(((n - 1) / 1024) / 16) per tensor (work items of 16 KiB; 0 for n <= 1024). */
typedef struct wq_xxh3_desc {
    const void *data;
    int64_t n;
    uint64_t *sums;    /* this tensor's workspace: wq_xxh3_workspace_bytes(n) bytes, 16-byte aligned */
    uint64_t *digest;  /* uint64[2] */
} wq_xxh3_desc;
int wq_xxh3_128_grouped(const wq_xxh3_desc *descs, const int64_t *item_start, int n_desc, int64_t total_items,
                        void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SLIME_AMD_WQ_H */
