// The cache of a latent attention: per token one normalised vector that every head's keys and
// values are linear functions of.  It lives in a page pool of one "head" whose entries are the
// latent vectors (padded with zeros to the width the attention kernels take), so the paged
// attention kernels read it as the keys and as the values of one shared head.
#include "api.h"
#include "common.h"

namespace st {

// One wave per token: c = x * rsqrt(mean(x^2) + eps) * gain in float, stored in the pool's type.
template <typename T>
__global__ __launch_bounds__(256) void latent_write_kernel(
    T* __restrict__ cache, int64_t page_stride, const float* __restrict__ x, int64_t x_stride,
    const float* __restrict__ gain, const int* __restrict__ token_item, const int* __restrict__ positions,
    const int* __restrict__ block_table, int max_pages, int page_size, int num_tokens, int rank, int entry,
    float eps, int tail, const float* __restrict__ freq, float tail_mult) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= num_tokens) return;
    const int item = token_item[t], pos = positions[t];
    if (item < 0 || pos < 0) return;                 // a padding row
    const int page = block_table[(int64_t)item * max_pages + pos / page_size];
    if (page < 0) return;
    const float* xp = x + (int64_t)t * x_stride;
    float ss = 0.f;
    for (int j = lane; j < rank; j += 64) { const float v = xp[j]; ss = fmaf(v, v, ss); }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)rank + eps);
    T* dst = cache + (int64_t)page * page_stride + (int64_t)(pos % page_size) * entry;
    for (int j = lane; j < entry; j += 64) {
        float v = 0.f;
        if (j < rank) {
            v = xp[j] * r * gain[j];
        } else if (j < rank + tail) {
            v = xp[j];
            if (freq) {                               // pairs (2i, 2i + 1) of the tail turn with the position
                const int i = (j - rank) >> 1;
                const float a = (float)pos * freq[i];
                const float c = cosf(a) * tail_mult, s = sinf(a) * tail_mult;
                const int ju = rank + 2 * i;
                const float u = xp[ju], w = xp[ju + 1];
                v = ((j - rank) & 1) ? w * c + u * s : u * c - w * s;
            }
        }
        Elem<T>::store(dst + j, v);
    }
}

}  // namespace st

using namespace st;

extern "C" int st_latent_write(void* cache, int64_t page_stride, const float* x, int64_t x_stride, const float* gain,
                               const int* token_item, const int* positions, const int* block_table, int max_pages,
                               int page_size, int num_tokens, int rank, int entry, float eps, int tail,
                               const float* freq, float tail_mult, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && rank > 0 && tail >= 0 && entry >= rank + tail && page_size > 0 && max_pages > 0,
             "latent_write: bad sizes");
    ST_CHECK(!freq || tail % 2 == 0, "latent_write: a turned tail has an even size");
    ST_CHECK(cache && x && gain && token_item && positions && block_table, "latent_write: null operand");
    ST_CHECK(eps > 0.f, "latent_write: eps must be positive");
    if (num_tokens == 0) return 0;
    const unsigned grid = (unsigned)((num_tokens + 3) / 4);
    if (dtype == kF32)
        latent_write_kernel<float><<<grid, 256, 0, stream>>>((float*)cache, page_stride, x, x_stride, gain, token_item,
            positions, block_table, max_pages, page_size, num_tokens, rank, entry, eps, tail, freq, tail_mult);
    else if (dtype == kBF16)
        latent_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)cache, page_stride, x, x_stride, gain, token_item,
            positions, block_table, max_pages, page_size, num_tokens, rank, entry, eps, tail, freq, tail_mult);
    else ST_CHECK(false, "latent_write: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("latent_write");
    return 0;
}
