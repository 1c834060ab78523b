// Rotary position encoding on the queries and keys of a step, in place, and the write of one
// paged pool (keys, or values with an optional per-head unit norm) from a step's rows.
//
// Rotation: of every head the `rot_dims` coordinates from `offset` on are turned, coordinate i paired with
// i + rot_dims / 2 (or, `interleaved`, 2i with 2i + 1):  (u, v) -> (u c - v s, v c + u s),  c = m cos(p f_i), s = m sin(p f_i), p the
// row's position, f the table of angles a position step (any scaling of the frequencies is in the
// table), m a factor on both.  Position, angle, cosine and sine are float.
#include "api.h"
#include "common.h"

namespace st {

template <typename T>
__global__ __launch_bounds__(256) void rotary_kernel(
    T* __restrict__ q, int64_t q_stride, int q_heads, T* __restrict__ k, int64_t k_stride, int k_heads,
    int head_dim, int half, int offset, int interleaved, const float* __restrict__ freq, float mult,
    const int* __restrict__ positions, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int per_row = (q_heads + k_heads) * half;
    const int64_t t = idx / per_row;
    int r = (int)(idx - t * per_row);
    const int head = r / half, i = r - head * half;
    const int pos = positions[t];
    if (pos < 0) return;                               // a padding row
    T* p = (head < q_heads ? q + t * q_stride + (int64_t)head * head_dim
                           : k + t * k_stride + (int64_t)(head - q_heads) * head_dim) + offset;
    const float a = (float)pos * freq[i];
    const float c = cosf(a) * mult, s = sinf(a) * mult;
    const int iu = interleaved ? 2 * i : i, iv = interleaved ? 2 * i + 1 : i + half;
    const float u = Elem<T>::load(p + iu), v = Elem<T>::load(p + iv);
    Elem<T>::store(p + iu, u * c - v * s);
    Elem<T>::store(p + iv, v * c + u * s);
}

// a wave a (row, head): src[t, head, :] (optionally divided by its root mean square) -> its page entry
template <typename T>
__global__ __launch_bounds__(256) void paged_write_kernel(
    T* __restrict__ cache, int64_t page_stride, const T* __restrict__ src, int64_t src_stride,
    const int* __restrict__ token_item, const int* __restrict__ positions, const int* __restrict__ block_table,
    int max_pages, int page_size, int64_t units, int heads, int head_dim, int norm, float eps) {
    const int64_t u = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= units) return;
    const int lane = threadIdx.x & 63;
    const int64_t t = u / heads;
    const int h = (int)(u - t * heads);
    const int item = token_item[t], pos = positions[t];
    if (item < 0 || pos < 0) return;
    const int pi = pos / page_size;
    const int page = block_table[(int64_t)item * max_pages + pi];
    if (page < 0) return;
    const T* s = src + t * src_stride + (int64_t)h * head_dim;
    T* d = cache + (int64_t)page * page_stride + ((int64_t)h * page_size + (pos - pi * page_size)) * head_dim;
    float r = 1.f;
    if (norm) {
        float ss = 0.f;
        for (int j = lane; j < head_dim; j += 64) {
            const float x = Elem<T>::load(s + j);
            ss = fmaf(x, x, ss);
        }
        ss = wave_sum(ss);
        r = 1.f / sqrtf(ss / (float)head_dim + eps);
    }
    for (int j = lane; j < head_dim; j += 64) Elem<T>::store(d + j, Elem<T>::load(s + j) * r);
}

// out[t] = (a[t] | b[t]) in the storage type, from float rows
template <typename T>
__global__ __launch_bounds__(256) void concat_cast_kernel(T* __restrict__ out, const float* __restrict__ a, int wa,
                                                          const float* __restrict__ b, int wb, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int w = wa + wb;
    const int64_t t = idx / w;
    const int c = (int)(idx - t * w);
    Elem<T>::store(out + idx, c < wa ? a[t * wa + c] : b[t * wb + (c - wa)]);
}

}  // namespace st

using namespace st;

extern "C" int st_rotary(void* q, int64_t q_stride, int q_heads, void* k, int64_t k_stride, int k_heads,
                         int head_dim, int rot_dims, int offset, int interleaved, const float* freq, float mult,
                         const int* positions, int num_tokens, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && q_heads >= 0 && k_heads >= 0 && head_dim > 0, "rotary: bad sizes");
    ST_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && offset >= 0 && offset + rot_dims <= head_dim,
             "rotary: %d turned coordinates from %d on in heads of %d", rot_dims, offset, head_dim);
    if (num_tokens == 0 || rot_dims == 0 || q_heads + k_heads == 0) return 0;
    ST_CHECK((q || q_heads == 0) && (k || k_heads == 0) && freq && positions, "rotary: null operand");
    const int half = rot_dims / 2;
    const int64_t total = (int64_t)num_tokens * (q_heads + k_heads) * half;
    const unsigned grid = (unsigned)((total + 255) / 256);
    if (dtype == kF32)
        rotary_kernel<float><<<grid, 256, 0, stream>>>((float*)q, q_stride, q_heads, (float*)k, k_stride, k_heads,
                                                       head_dim, half, offset, interleaved, freq, mult, positions, total);
    else if (dtype == kBF16)
        rotary_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)q, q_stride, q_heads, (bf16_t*)k, k_stride, k_heads,
                                                        head_dim, half, offset, interleaved, freq, mult, positions, total);
    else ST_CHECK(false, "rotary: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("rotary");
    return 0;
}

extern "C" int st_paged_write(void* cache, int64_t page_stride, const void* src, int64_t src_stride,
                              const int* token_item, const int* positions, const int* block_table, int max_pages,
                              int page_size, int num_tokens, int heads, int head_dim, int norm, float eps, int dtype,
                              hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && head_dim > 0 && page_size > 0 && max_pages > 0, "paged_write: bad sizes");
    ST_CHECK(!norm || eps > 0.f, "paged_write: eps must be positive");
    if (num_tokens == 0) return 0;
    ST_CHECK(cache && src && token_item && positions && block_table, "paged_write: null operand");
    const int64_t units = (int64_t)num_tokens * heads;
    const unsigned grid = (unsigned)((units + 3) / 4);
    if (dtype == kF32)
        paged_write_kernel<float><<<grid, 256, 0, stream>>>((float*)cache, page_stride, (const float*)src, src_stride,
            token_item, positions, block_table, max_pages, page_size, units, heads, head_dim, norm, eps);
    else if (dtype == kBF16)
        paged_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)cache, page_stride, (const bf16_t*)src,
            src_stride, token_item, positions, block_table, max_pages, page_size, units, heads, head_dim, norm, eps);
    else ST_CHECK(false, "paged_write: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("paged_write");
    return 0;
}

extern "C" int st_concat_cast(void* out, const float* a, int wa, const float* b, int wb, int num_rows, int dtype,
                              hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && wa > 0 && wb >= 0, "concat_cast: bad sizes");
    if (num_rows == 0) return 0;
    ST_CHECK(out && a && (b || wb == 0), "concat_cast: null operand");
    const int64_t total = (int64_t)num_rows * (wa + wb);
    const unsigned grid = (unsigned)((total + 255) / 256);
    if (dtype == kF32)
        concat_cast_kernel<float><<<grid, 256, 0, stream>>>((float*)out, a, wa, b, wb, total);
    else if (dtype == kBF16)
        concat_cast_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, a, wa, b, wb, total);
    else ST_CHECK(false, "concat_cast: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("concat_cast");
    return 0;
}
