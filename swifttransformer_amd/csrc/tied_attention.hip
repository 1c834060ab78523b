// Queries and keys of an attention whose values are its keys: both are normalised over their whole
// projection (all heads at once, one gain an output), the normalised keys are what the scores read and the
// keys as projected are what the weights sum.
//
//   q' = q * rsqrt(mean(q^2) + eps) * gq   -> out_q [T, heads, head_pad] in the storage type
//   k' = k * rsqrt(mean(k^2) + eps) * gk   -> the token's entry of the key pool
//   k                                      -> the token's entry of the value pool
//
// q and k are the float results of their product (rows of `stride` floats, k behind q); a head's `head_dim`
// numbers are followed by zeros up to `head_pad` (the attention kernels take multiples of 16).  One
// workgroup a token.
#include "api.h"
#include "common.h"

namespace st {

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_write_kernel(
    T* __restrict__ out_q, T* __restrict__ k_cache, T* __restrict__ v_cache, int64_t page_stride,
    const float* __restrict__ qk, int64_t stride, const float* __restrict__ gq, const float* __restrict__ gk,
    const int* __restrict__ token_item, const int* __restrict__ positions, const int* __restrict__ block_table,
    int max_pages, int page_size, int heads, int kv_heads, int head_dim, int head_pad, float eps, int write) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const int item = token_item[t], pos = positions[t];
    const int nq = heads * head_dim, nk = kv_heads * head_dim;
    const float* q = qk + (int64_t)t * stride;
    const float* k = q + nq;
    T* oq = out_q + (int64_t)t * heads * head_pad;
    if (item < 0 || pos < 0) {                                // a padding row: queries of zeros, nothing cached
        for (int i = threadIdx.x; i < heads * head_pad; i += 256) Elem<T>::store(oq + i, 0.f);
        return;
    }
    // (the page's number is asked for before the sums: its trip to memory runs beside theirs)
    const int page = write ? block_table[(int64_t)item * max_pages + pos / page_size] : -1;
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += 256) sq = fmaf(q[i], q[i], sq);
    for (int i = threadIdx.x; i < nk; i += 256) sk = fmaf(k[i], k[i], sk);
    {   // both sums over the workgroup with one exchange through LDS
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        sq = wave_sum(sq);
        sk = wave_sum(sk);
        if (lane == 0) { red[wave] = sq; red[4 + wave] = sk; }
        __syncthreads();
        sq = red[0] + red[1] + red[2] + red[3];
        sk = red[4] + red[5] + red[6] + red[7];
    }
    const float rq = 1.f / sqrtf(sq / (float)nq + eps), rk = 1.f / sqrtf(sk / (float)nk + eps);
    for (int i = threadIdx.x; i < heads * head_pad; i += 256) {
        const int h = i / head_pad, d = i - h * head_pad;
        const int j = h * head_dim + d;
        Elem<T>::store(oq + i, d < head_dim ? q[j] * rq * gq[j] : 0.f);
    }
    if (!write || page < 0) return;
    const int64_t base = (int64_t)page * page_stride + (int64_t)(pos % page_size) * head_pad;
    for (int i = threadIdx.x; i < kv_heads * head_pad; i += 256) {
        const int h = i / head_pad, d = i - h * head_pad;
        const int j = h * head_dim + d;
        const int64_t off = base + (int64_t)h * page_size * head_pad + d;
        const bool in = d < head_dim;
        Elem<T>::store(k_cache + off, in ? k[j] * rk * gk[j] : 0.f);
        Elem<T>::store(v_cache + off, in ? k[j] : 0.f);
    }
}

}  // namespace st

using namespace st;

// Pools [pages, kv_heads, page_size, head_pad] of `dtype`; write == 0: the queries only.
extern "C" int st_qk_norm_write(void* out_q, void* k_cache, void* v_cache, int64_t page_stride, const float* qk,
                                int64_t stride, const float* gain_q, const float* gain_k, const int* token_item,
                                const int* positions, const int* block_table, int max_pages, int page_size,
                                int num_tokens, int heads, int kv_heads, int head_dim, int head_pad, float eps,
                                int write, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && head_pad >= head_dim && page_size > 0 &&
             max_pages > 0, "qk_norm_write: bad sizes");
    ST_CHECK(stride >= (int64_t)(heads + kv_heads) * head_dim, "qk_norm_write: rows shorter than q and k");
    ST_CHECK(eps > 0.f, "qk_norm_write: eps must be positive");
    if (num_tokens == 0) return 0;
    ST_CHECK(out_q && qk && gain_q && gain_k && token_item && positions && (!write || (k_cache && v_cache && block_table)),
             "qk_norm_write: null operand");
    if (dtype == kF32)
        qk_norm_write_kernel<float><<<num_tokens, 256, 0, stream>>>((float*)out_q, (float*)k_cache, (float*)v_cache,
            page_stride, qk, stride, gain_q, gain_k, token_item, positions, block_table, max_pages, page_size, heads,
            kv_heads, head_dim, head_pad, eps, write);
    else if (dtype == kBF16)
        qk_norm_write_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((bf16_t*)out_q, (bf16_t*)k_cache, (bf16_t*)v_cache,
            page_stride, qk, stride, gain_q, gain_k, token_item, positions, block_table, max_pages, page_size, heads,
            kv_heads, head_dim, head_pad, eps, write);
    else ST_CHECK(false, "qk_norm_write: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("qk_norm_write");
    return 0;
}
