// Per-sync address resolution of a weight-sync bucket's work-item table.
//
// The bucket launches (wq_fp8_bucket_convert, wq_int4_bucket_convert, wq_int4_group_quant_pack_asym_items) read one
// pre-resolved descriptor per work item.  Everything in such a table but the input address is a property of the
// bucket's layout - names, shapes, strides, output offsets - and stays the same from one weight sync to the next,
// while the inputs themselves are fresh tensors on every sync whenever the model is sharded (gathered partitions,
// concatenated experts).  The layout is therefore kept as a TEMPLATE whose first field is a byte offset inside the
// item's input tensor plus the index of that tensor, and this kernel adds the current base address of every
// tensor: one small upload (8 bytes per tensor) and one pass over the table replace the host-side rebuild.

#include "wq_common.h"

namespace wq {

// One 8-byte word per lane: word c of item i is copied, and word 0 gets bases[owner[i]] added.
__global__ __launch_bounds__(256) void bucket_resolve_kernel(const int64_t* __restrict__ tmpl,
                                                            const int32_t* __restrict__ owner,
                                                            const int64_t* __restrict__ bases, int64_t n_words,
                                                            int width, int64_t* __restrict__ out)
{
    const int64_t w = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * 256 + threadIdx.x;
    if (w >= n_words) return;
    const int64_t item = w / width;
    int64_t v = tmpl[w];
    if (w - item * width == 0) v += bases[owner[item]];
    out[w] = v;
}

}  // namespace wq

using namespace wq;

WQ_EXPORT int wq_bucket_resolve_items(const int64_t* item_template, const int32_t* owner, const int64_t* bases,
                                      int64_t n_items, int words_per_item, int64_t* items, void* stream)
{
    if (n_items < 0 || words_per_item <= 0 || words_per_item > 16) return WQ_ERR_SHAPE;
    if (n_items == 0) return WQ_OK;
    if (!item_template || !owner || !bases || !items) return WQ_ERR_NULL;
    if (item_template == items) return WQ_ERR_UNSUPPORTED;      // the template must survive: it serves the next sync
    const int64_t n_words = n_items * words_per_item;
    bucket_resolve_kernel<<<grid_for_items(cdiv64(n_words, 256)), 256, 0, (hipStream_t)stream>>>(
        item_template, owner, bases, n_words, words_per_item, items);
    WQ_LAUNCH_CHECK();
    return WQ_OK;
}
