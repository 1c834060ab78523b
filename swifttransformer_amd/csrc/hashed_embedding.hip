// Token embedding with a factor, plus a row of a second table chosen by a hash of the token and the one
// before it in its sequence:
//
//   x[t] = table[id_t] * scale + pairs[(id_(t-1) * mul_prev + id_t * mul_cur) mod buckets]
//   (a sequence's first token takes row `buckets`, the table's last)
//
// The token before a step's first row of an item is the last token of the item's request in an earlier
// step: it waits in the request's state slot (one int), which a second small kernel moves on after the
// rows are made.  Sums are float; the result is the float residual stream.
#include "api.h"
#include "common.h"

namespace st {

template <typename T>
__global__ __launch_bounds__(256) void hashed_embed_kernel(
    float* __restrict__ out, const int* __restrict__ ids, const int* __restrict__ positions,
    const int* __restrict__ token_item, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    const int* __restrict__ last_token, const T* __restrict__ table, const T* __restrict__ pairs, int vocab,
    int buckets, int64_t mul_prev, int64_t mul_cur, float scale, int width) {
    const int t = blockIdx.x;
    const int item = token_item[t];
    float* dst = out + (int64_t)t * width;
    const int id = ids[t];
    if (item < 0 || id < 0 || id >= vocab) {                  // a padding row
        for (int c = threadIdx.x; c < width; c += 256) dst[c] = 0.f;
        return;
    }
    if (!pairs) {                                            // no second table: the token's row times the factor
        const T* e0 = table + (int64_t)id * width;
        for (int c = threadIdx.x; c < width; c += 256) dst[c] = Elem<T>::load(e0 + c) * scale;
        return;
    }
    int64_t row = buckets;
    if (positions[t] > 0) {
        const int prev = t > item_tok_off[item] ? ids[t - 1] : last_token[item_slot[item]];
        row = ((int64_t)prev * mul_prev + (int64_t)id * mul_cur) % buckets;
        if (row < 0) row += buckets;
    }
    const T* e = table + (int64_t)id * width;
    const T* p = pairs + row * width;
    for (int c = threadIdx.x; c < width; c += 256) dst[c] = fmaf(Elem<T>::load(e + c), scale, Elem<T>::load(p + c));
}

__global__ void last_token_kernel(int* __restrict__ last_token, const int* __restrict__ ids,
                                  const int* __restrict__ item_len, const int* __restrict__ item_tok_off,
                                  const int* __restrict__ item_slot, int num_items) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= num_items) return;
    const int n = item_len[b], slot = item_slot[b];
    if (n <= 0 || slot < 0) return;
    last_token[slot] = ids[item_tok_off[b] + n - 1];
}

}  // namespace st

using namespace st;

// out [num_tokens, width] float; table [vocab, width], pairs [buckets + 1, width] of `dtype` (null: none);
// last_token: one int a state slot (read for an item's first row, then set to the item's last token of this step).
extern "C" int st_hashed_embed(float* out, const int* ids, const int* positions, const int* token_item,
                               const int* item_len, const int* item_tok_off, const int* item_slot, int* last_token,
                               const void* table, const void* pairs, int num_tokens, int num_items, int vocab,
                               int buckets, int64_t mul_prev, int64_t mul_cur, float scale, int width, int dtype,
                               hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && num_items >= 0 && vocab > 0 && width > 0, "hashed_embed: bad sizes");
    if (num_tokens == 0) return 0;
    ST_CHECK(out && ids && positions && token_item && table, "hashed_embed: null operand");
    ST_CHECK(!pairs || (buckets > 0 && item_len && item_tok_off && item_slot && last_token),
             "hashed_embed: the table of pairs needs buckets, the items and the requests' last tokens");
    if (dtype == kF32)
        hashed_embed_kernel<float><<<num_tokens, 256, 0, stream>>>(out, ids, positions, token_item, item_tok_off,
            item_slot, last_token, (const float*)table, (const float*)pairs, vocab, buckets, mul_prev, mul_cur, scale,
            width);
    else if (dtype == kBF16)
        hashed_embed_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(out, ids, positions, token_item, item_tok_off,
            item_slot, last_token, (const bf16_t*)table, (const bf16_t*)pairs, vocab, buckets, mul_prev, mul_cur, scale,
            width);
    else ST_CHECK(false, "hashed_embed: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("hashed_embed");
    if (pairs && num_items > 0) {
        last_token_kernel<<<(num_items + 63) / 64, 64, 0, stream>>>(last_token, ids, item_len, item_tok_off, item_slot,
                                                                    num_items);
        ST_LAUNCH_CHECK("hashed_embed (state)");
    }
    return 0;
}
